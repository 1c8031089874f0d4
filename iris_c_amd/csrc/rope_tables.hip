/*
 * Rotary-position tables expanded on the device (include/iris_rope.h,
 * iris_dev_rope_*).
 *
 * A table row is the concatenation, over the axes, of the cos / sin row of
 * that axis at the token's position, and a sequence has few distinct
 * (axis, position) pairs: an h x w image has h + w of them, not h * w. The
 * host evaluates each distinct pair once, with the libm calls of the
 * reference's routines (iris_transformer_flux.c:823-1013,
 * iris_transformer_zimage.c:604-622, iris_qwen3.c:277-291: float angles,
 * cosf / sinf; iris_transformer_flux3.c:282-294: double angles, cos / sin
 * rounded to float), and hands over that dictionary plus one 32-bit offset
 * per (token, axis): 16 bytes a token for four axes instead of the 512 bytes
 * of its two table rows. This kernel only copies, so the device tables carry
 * the bits of the host builders' tables.
 *
 * One thread per table entry; consecutive threads write consecutive floats
 * and read consecutive dictionary entries within an axis.
 */
#include <hip/hip_runtime.h>

#include "iris_kernels_hip.h"

namespace {

constexpr int THREADS = 256;

__global__ void __launch_bounds__(THREADS)
k_rope_gather(float *__restrict__ cos_t, float *__restrict__ sin_t, const float *__restrict__ values,
              const uint32_t *__restrict__ index, const int4 *__restrict__ columns, int half, int naxes, size_t n) {
    const size_t i = (size_t)blockIdx.x * THREADS + threadIdx.x;
    if (i >= n) return;
    const size_t s = i / half;
    const int4 c = columns[(int)(i % half)];              /* x: axis, y: column inside the axis, z: columns of the axis */
    const float *row = values + index[s * naxes + c.x];
    cos_t[i] = row[c.y];
    sin_t[i] = row[c.z + c.y];
}

}  // namespace

extern "C" int iris_hip_rope_gather(void *stream, float *cos_t, float *sin_t, const float *values,
                                    const uint32_t *index, const void *columns, int seq, int half, int naxes) {
    const size_t n = (size_t)seq * half;
    if (!n) return 0;
    const unsigned blocks = (unsigned)((n + THREADS - 1) / THREADS);
    hipLaunchKernelGGL(k_rope_gather, dim3(blocks), dim3(THREADS), 0, (hipStream_t)stream, cos_t, sin_t, values, index,
                       static_cast<const int4 *>(columns), half, naxes, n);
    return (int)hipGetLastError();
}
