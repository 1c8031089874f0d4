/*
 * Rotary-position tables generated on the device (include/iris_rope.h,
 * iris_dev_rope_*): the host hands over positions [seq, naxes] and one
 * frequency per table column, the kernel writes cos / sin [seq, half].
 *
 * The angle is formed as on the host, a single multiply in the table's
 * arithmetic type (float: (float)p * freq, the form of iris_transformer_flux.c:823-1013,
 * iris_transformer_zimage.c:604-622 and iris_qwen3.c:277-291; double: p * freq,
 * iris_transformer_flux3.c:282-294), and cosine and sine are evaluated in
 * double and rounded once to float. The host's cosf / sinf are faithful but
 * not always correctly rounded, so the two tables may differ by one float ulp
 * in a few entries and are identical elsewhere; position 0 gives exactly (1, 0).
 *
 * One thread per table entry; consecutive threads write consecutive floats.
 * A table is a few hundred thousand entries, built once per forward pass.
 */
#include <hip/hip_runtime.h>

#include "iris_kernels_hip.h"

namespace {

constexpr int THREADS = 256;

template <bool F64>
__global__ void __launch_bounds__(THREADS)
k_rope_tables(float *__restrict__ cos_t, float *__restrict__ sin_t, const void *__restrict__ freq,
              const int *__restrict__ col_axis, const void *__restrict__ pos, int half, int naxes, size_t n) {
    const size_t i = (size_t)blockIdx.x * THREADS + threadIdx.x;
    if (i >= n) return;
    const size_t s = i / half;
    const int col = (int)(i % half);
    const size_t at = s * naxes + col_axis[col];
    double angle;
    if (F64) {
        angle = (double)static_cast<const float *>(pos)[at] * static_cast<const double *>(freq)[col];
    } else {
        const float a = (float)static_cast<const int *>(pos)[at] * static_cast<const float *>(freq)[col];
        angle = (double)a;
    }
    double sn, cs;
    sincos(angle, &sn, &cs);
    cos_t[i] = (float)cs;
    sin_t[i] = (float)sn;
}

}  // namespace

extern "C" int iris_hip_rope_tables(void *stream, float *cos_t, float *sin_t, const void *freq,
                                    const int *col_axis, const void *pos, int seq, int half, int naxes,
                                    int use_double) {
    const size_t n = (size_t)seq * half;
    if (!n) return 0;
    const unsigned blocks = (unsigned)((n + THREADS - 1) / THREADS);
    hipStream_t st = (hipStream_t)stream;
    if (use_double)
        hipLaunchKernelGGL(k_rope_tables<true>, dim3(blocks), dim3(THREADS), 0, st, cos_t, sin_t, freq, col_axis, pos,
                           half, naxes, n);
    else
        hipLaunchKernelGGL(k_rope_tables<false>, dim3(blocks), dim3(THREADS), 0, st, cos_t, sin_t, freq, col_axis, pos,
                           half, naxes, n);
    return (int)hipGetLastError();
}
