/*
 * Linear layers and convolution for gfx950 (reference iris_dev.h:48-53, 111-121;
 * iris_cuda.cu:456-505, 959-1016).
 *
 *   y[M, N] = x[M, K] @ W[N, K]^T      bf16 inputs, f32 accumulation, f32 or bf16 output
 *
 * Both operands are K-contiguous, which is exactly what the matrix-core operand
 * layout wants (a lane holds 8 consecutive K elements of one row), so tiles go
 * HBM -> registers -> LDS unchanged. The product is issued transposed,
 * D^T = W_tile x_tile^T with v_mfma_f32_16x16x32_bf16 (A = W rows, B = x rows): in
 * the 16x16 accumulator a lane then holds four consecutive n of one output row m,
 * a single 16-byte (f32) or 8-byte (bf16) store.
 *
 * Workgroup = WM x WN waves (2 x 2 in use), tile 128 (m) x 128 (n), K in steps of 64; a wave owns
 * 64 x 64 = 4 x 4 accumulator blocks and reads 8 operands from LDS per 16 MFMAs. One
 * LDS stage of [W tile | x tile], rows padded to 160 B so that the 16 lanes the LDS
 * serves together on a 128-bit read fall in distinct bank windows; the next K tile
 * waits in registers while the current one is multiplied (two barriers per tile,
 * two workgroups per CU to cover them).
 *
 * Any M and N (rows are clamped on load, stores are bounded); K must be a multiple
 * of 8 with 16-byte aligned rows, otherwise the scalar kernel below takes over (the
 * only such caller is the 3-channel input convolution of the VAE encoder).
 *
 * Convolution = gather of the k x k input patches as bf16 rows (what the reference
 * does, iris_cuda.cu:959-985) into scratch, then the same GEMM, chunked by output
 * pixels so the scratch stays bounded.
 */
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "iris_kernels_hip.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int TK = 64;
constexpr int LS = TK + 16;            /* LDS row stride in elements (160 B) */

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    f32x2 p = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(p, bf16x2));
}

__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

__device__ __forceinline__ void store4(float *p, f32x4 v, int n_left) {
    if (n_left >= 4 && ((uintptr_t)p & 15) == 0) { *reinterpret_cast<f32x4 *>(p) = v; return; }
    for (int r = 0; r < 4 && r < n_left; r++) p[r] = v[r];
}
__device__ __forceinline__ void store4(uint16_t *p, f32x4 v, int n_left) {
    if (n_left >= 4 && ((uintptr_t)p & 7) == 0) { *reinterpret_cast<uint2 *>(p) = make_uint2(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3])); return; }
    for (int r = 0; r < 4 && r < n_left; r++) p[r] = (uint16_t)(pack_bf16(v[r], 0.0f) & 0xffffu);
}

/* WM x WN waves of 64 x 64 outputs each: tile (64 WM) x (64 WN). */
template <typename OUT, int WM, int WN>
__global__ void __launch_bounds__(64 * WM * WN, 2)
k_gemm_bf16(OUT *__restrict__ y, const uint16_t *__restrict__ x, const uint16_t *__restrict__ W,
            int M, int N, int K, int tiles_m) {
    constexpr int TM = 64 * WM, TN = 64 * WN, THREADS = 64 * WM * WN;
    constexpr int RPP = THREADS / 8;                 /* rows covered by one pass of the workgroup */
    constexpr int NW = TN / RPP, NX = TM / RPP;      /* 16 B chunks of W and of x per thread and K tile */
    __shared__ __align__(16) uint16_t lds[(TN + TM) * LS];
    uint16_t *Ws = lds, *Xs = lds + TN * LS;

    const int bm = blockIdx.x % tiles_m, bn = blockIdx.x / tiles_m;
    const int m0 = bm * TM, n0 = bn * TN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 15, lg = lane >> 4;
    const int wm = wave % WM, wn = wave / WM;

    /* staging: this thread moves 16 B chunk (tid % 8) of rows tid / 8 + RPP c of both tiles */
    const int srow = tid >> 3, scol = (tid & 7) * 8;
    const uint16_t *wsrc[NW], *xsrc[NX];
#pragma unroll
    for (int c = 0; c < NW; c++) wsrc[c] = W + (size_t)min(n0 + srow + RPP * c, N - 1) * K + scol;
#pragma unroll
    for (int c = 0; c < NX; c++) xsrc[c] = x + (size_t)min(m0 + srow + RPP * c, M - 1) * K + scol;
    u32x4 wreg[NW], xreg[NX];
    auto fetch = [&](int k0) {
        const bool inside = k0 + scol < K;                 /* K % 8 == 0: a chunk is inside or outside */
#pragma unroll
        for (int c = 0; c < NW; c++) wreg[c] = inside ? *reinterpret_cast<const u32x4 *>(wsrc[c] + k0) : u32x4{0, 0, 0, 0};
#pragma unroll
        for (int c = 0; c < NX; c++) xreg[c] = inside ? *reinterpret_cast<const u32x4 *>(xsrc[c] + k0) : u32x4{0, 0, 0, 0};
    };
    auto store = [&]() {
#pragma unroll
        for (int c = 0; c < NW; c++) *reinterpret_cast<u32x4 *>(&Ws[(srow + RPP * c) * LS + scol]) = wreg[c];
#pragma unroll
        for (int c = 0; c < NX; c++) *reinterpret_cast<u32x4 *>(&Xs[(srow + RPP * c) * LS + scol]) = xreg[c];
    };

    f32x4 acc[4][4];
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
        for (int b = 0; b < 4; b++) acc[a][b] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    const int a_rd = (64 * wn + li) * LS + 8 * lg;          /* W rows: n = 64 wn + 16 a + li */
    const int b_rd = (64 * wm + li) * LS + 8 * lg;          /* x rows: m = 64 wm + 16 b + li */
    const int nk = (K + TK - 1) / TK;

    fetch(0);
    store();
    fetch(TK);                                              /* past the end: zeros */
    __syncthreads();

    for (int kt = 0; kt < nk; kt++) {
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
            u32x4 av[4], bv[4];
#pragma unroll
            for (int a = 0; a < 4; a++) av[a] = *reinterpret_cast<const u32x4 *>(&Ws[a_rd + 16 * a * LS + 32 * ks]);
#pragma unroll
            for (int b = 0; b < 4; b++) bv[b] = *reinterpret_cast<const u32x4 *>(&Xs[b_rd + 16 * b * LS + 32 * ks]);
#pragma unroll
            for (int a = 0; a < 4; a++)
#pragma unroll
                for (int b = 0; b < 4; b++)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, av[a]),
                                                                       __builtin_bit_cast(bf16x8, bv[b]), acc[a][b], 0, 0, 0);
        }
        lds_barrier();                                      /* every wave is done with this tile */
        store();
        fetch((kt + 2) * TK);
        lds_barrier();
    }

    /* acc[a][b][r] = y[m0 + 64 wm + 16 b + li][n0 + 64 wn + 16 a + 4 lg + r] */
#pragma unroll
    for (int b = 0; b < 4; b++) {
        const int m = m0 + 64 * wm + 16 * b + li;
        if (m >= M) continue;
#pragma unroll
        for (int a = 0; a < 4; a++) {
            const int n = n0 + 64 * wn + 16 * a + 4 * lg;
            if (n < N) store4(y + (size_t)m * N + n, acc[a][b], N - n);
        }
    }
}

/* Any K / alignment: one thread per output element. */
template <typename OUT>
__global__ void __launch_bounds__(256)
k_gemm_scalar(OUT *__restrict__ y, const uint16_t *__restrict__ x, const uint16_t *__restrict__ W, int M, int N, int K) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)M * N) return;
    const int m = (int)(i / N), n = (int)(i % N);
    const uint16_t *xr = x + (size_t)m * K, *wr = W + (size_t)n * K;
    float s = 0.0f;
    for (int k = 0; k < K; k++) s = fmaf(__uint_as_float((uint32_t)xr[k] << 16), __uint_as_float((uint32_t)wr[k] << 16), s);
    f32x4 v = {s, 0.0f, 0.0f, 0.0f};
    store4(y + i, v, 1);
}

template <typename OUT>
int gemm(hipStream_t st, OUT *y, const uint16_t *x, const uint16_t *W, int M, int N, int K) {
    if (M <= 0 || N <= 0) return 0;
    if (K > 0 && K % 8 == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)W & 15) == 0) {
        /* 2 x 2 waves (128 x 128 tiles) measured best on the transformer shapes: 4 x 2 and 2 x 4 are
         * 5-8 % slower on the wide projections, 4 x 1 and 2 x 1 15-30 % slower. */
        constexpr int WM = 2, WN = 2, TM = 64 * WM, TN = 64 * WN;
        const int tiles_m = (M + TM - 1) / TM, tiles_n = (N + TN - 1) / TN;
        hipLaunchKernelGGL((k_gemm_bf16<OUT, WM, WN>), dim3((unsigned)tiles_m * tiles_n), dim3(64 * WM * WN), 0, st, y, x, W, M, N, K, tiles_m);
    } else {
        const size_t n = (size_t)M * N;
        hipLaunchKernelGGL(k_gemm_scalar<OUT>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, y, x, W, M, N, K);
    }
    return (int)hipGetLastError();
}

/* Patches of output pixels [p0, p0 + np) as bf16 rows of k * k * cin in (ky, kx, c) order,
 * zeros outside the image. VEC = channels per thread (8 when cin % 8 == 0). */
template <int VEC>
__global__ void __launch_bounds__(256)
k_im2col(uint16_t *__restrict__ cols, const float *__restrict__ in, int h, int w, int cin, int k, int stride,
         int pad, int ow, int p0, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int row_groups = k * k * cin / VEC;
    const int p = p0 + (int)(i / row_groups);
    const int r = (int)(i % row_groups) * VEC;
    const int tap = r / cin, c = r % cin;
    const int yy = (p / ow) * stride + tap / k - pad, xx = (p % ow) * stride + tap % k - pad;
    const bool inside = yy >= 0 && yy < h && xx >= 0 && xx < w;
    const float *src = in + ((size_t)yy * w + xx) * cin + c;
    if (VEC == 8) {
        float4 a = make_float4(0.0f, 0.0f, 0.0f, 0.0f), b = a;
        if (inside) { a = reinterpret_cast<const float4 *>(src)[0]; b = reinterpret_cast<const float4 *>(src)[1]; }
        *reinterpret_cast<uint4 *>(cols + i * 8) = make_uint4(pack_bf16(a.x, a.y), pack_bf16(a.z, a.w), pack_bf16(b.x, b.y), pack_bf16(b.z, b.w));
    } else {
        cols[i] = inside ? (uint16_t)(pack_bf16(src[0], 0.0f) & 0xffffu) : (uint16_t)0;
    }
}

__global__ void __launch_bounds__(256)
k_add_bias_rows(float *__restrict__ y, const float *__restrict__ bias, int cols, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) y[i] += bias[i % cols];
}

}  // namespace

extern "C" {

int iris_hip_linear_f32(void *stream, float *y, const uint16_t *x, const uint16_t *W, int rows, int in, int out) {
    return gemm<float>((hipStream_t)stream, y, x, W, rows, out, in);
}
int iris_hip_linear_bf16(void *stream, uint16_t *y, const uint16_t *x, const uint16_t *W, int rows, int in, int out) {
    return gemm<uint16_t>((hipStream_t)stream, y, x, W, rows, out, in);
}

/* scratch: device buffer of scratch_bytes (>= one patch row) for the bf16 patches */
int iris_hip_conv2d(void *stream, uint16_t *scratch, size_t scratch_bytes, float *out, const float *in,
                    const uint16_t *w, const float *bias, int h, int width, int cin, int cout, int k,
                    int stride, int pad_before, int pad_after) {
    hipStream_t st = (hipStream_t)stream;
    const int oh = (h + pad_before + pad_after - k) / stride + 1;
    const int ow = (width + pad_before + pad_after - k) / stride + 1;
    if (oh <= 0 || ow <= 0) return 0;
    const int ohw = oh * ow, row_len = k * k * cin;
    long chunk = (long)(scratch_bytes / ((size_t)row_len * sizeof(uint16_t)));
    if (chunk < 1) return (int)hipErrorInvalidValue;
    if (chunk > ohw) chunk = ohw;
    const bool vec = cin % 8 == 0 && ((uintptr_t)in & 15) == 0;
    for (int p0 = 0; p0 < ohw; p0 += (int)chunk) {
        const int np = ohw - p0 < chunk ? ohw - p0 : (int)chunk;
        const size_t n = (size_t)np * row_len / (vec ? 8 : 1);
        if (vec) hipLaunchKernelGGL(k_im2col<8>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, scratch, in, h, width, cin, k, stride, pad_before, ow, p0, n);
        else hipLaunchKernelGGL(k_im2col<1>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, scratch, in, h, width, cin, k, stride, pad_before, ow, p0, n);
        int e = gemm<float>(st, out + (size_t)p0 * cout, scratch, w, np, cout, row_len);
        if (e) return e;
    }
    if (bias) {
        const size_t n = (size_t)ohw * cout;
        hipLaunchKernelGGL(k_add_bias_rows, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, out, bias, cout, n);
    }
    return (int)hipGetLastError();
}

}  // extern "C"
