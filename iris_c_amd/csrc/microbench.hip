/*
 * Machine-ceiling microbenchmarks reported next to the kernel numbers:
 * what this GPU sustains for back-to-back bf16 MFMA, for a plain HBM copy,
 * for 128-bit LDS reads and for v_exp_f32. Bench infrastructure, built into
 * its own library (libiris_microbench.so); the product library does not
 * contain it.
 */
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

namespace {

/* 4 independent accumulator chains per wave, `iters` x 4 MFMAs each. */
__global__ void __launch_bounds__(256) k_mfma_peak(float *sink, int iters) {
    f32x16 acc[4];
    for (int a = 0; a < 4; a++)
        for (int r = 0; r < 16; r++) acc[a][r] = 0.0f;
    uint4 raw = make_uint4(0x3f803f80u + threadIdx.x, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u);
    bf16x8 x = __builtin_bit_cast(bf16x8, raw), y = x;
    for (int i = 0; i < iters; i++) {
#pragma unroll
        for (int a = 0; a < 4; a++) acc[a] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, acc[a], 0, 0, 0);
    }
    float s = 0.0f;
    for (int a = 0; a < 4; a++)
        for (int r = 0; r < 16; r++) s += acc[a][r];
    if (s == 12345.678f) sink[0] = s;
}

/* The same loop with operands taken from memory (8 x 16 B per lane): the matrix
 * cores draw more power on real data than on constants, and the clock follows,
 * so the sustained rate depends on what is multiplied. */
__global__ void __launch_bounds__(256) k_mfma_data(const uint4 *__restrict__ ops, float *sink, int iters) {
    f32x16 acc[4];
    for (int a = 0; a < 4; a++)
        for (int r = 0; r < 16; r++) acc[a][r] = 0.0f;
    bf16x8 x[4], y[4];
    for (int i = 0; i < 4; i++) {
        x[i] = __builtin_bit_cast(bf16x8, ops[(2 * i) * 256 + threadIdx.x]);
        y[i] = __builtin_bit_cast(bf16x8, ops[(2 * i + 1) * 256 + threadIdx.x]);
    }
    for (int i = 0; i < iters; i++) {
#pragma unroll
        for (int a = 0; a < 4; a++)
#pragma unroll
            for (int j = 0; j < 4; j++)
                acc[a] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x[j], y[(j + a) & 3], acc[a], 0, 0, 0);
    }
    float s = 0.0f;
    for (int a = 0; a < 4; a++)
        for (int r = 0; r < 16; r++) s += acc[a][r];
    if (s == 12345.678f) sink[0] = s;
}

/* Same flops per wave and iteration with the 16x16x32 shape (32 MFMAs of half the size):
 * a quarter of the accumulator registers per flop, and measurably less power. */
__global__ void __launch_bounds__(256) k_mfma_data16(const uint4 *__restrict__ ops, float *sink, int iters) {
    f32x4 acc[8];
    for (int a = 0; a < 8; a++)
        for (int r = 0; r < 4; r++) acc[a][r] = 0.0f;
    bf16x8 x[4], y[4];
    for (int i = 0; i < 4; i++) {
        x[i] = __builtin_bit_cast(bf16x8, ops[(2 * i) * 256 + threadIdx.x]);
        y[i] = __builtin_bit_cast(bf16x8, ops[(2 * i + 1) * 256 + threadIdx.x]);
    }
    for (int i = 0; i < iters; i++) {
#pragma unroll
        for (int a = 0; a < 8; a++)
#pragma unroll
            for (int j = 0; j < 4; j++)
                acc[a] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(x[j], y[(j + a) & 3], acc[a], 0, 0, 0);
    }
    float s = 0.0f;
    for (int a = 0; a < 8; a++)
        for (int r = 0; r < 4; r++) s += acc[a][r];
    if (s == 12345.678f) sink[0] = s;
}

__global__ void __launch_bounds__(256) k_copy(uint4 *__restrict__ dst, const uint4 *__restrict__ src, size_t n) {
    size_t i = (size_t)blockIdx.x * 256 * 4 + threadIdx.x;
#pragma unroll
    for (int u = 0; u < 4; u++) {
        size_t j = i + (size_t)u * 256;
        if (j < n) dst[j] = src[j];
    }
}

/* Read-only and write-only streams, 16 B per lane, the same shape as the copy: what the memory system
 * gives one direction alone. The sum of the read is kept alive by a store that never happens. */
__global__ void __launch_bounds__(256) k_read_only(const uint4 *__restrict__ src, size_t n, unsigned *sink) {
    size_t i = (size_t)blockIdx.x * 256 * 4 + threadIdx.x;
    uint4 v[4];
#pragma unroll
    for (int u = 0; u < 4; u++) {
        size_t j = i + (size_t)u * 256;
        v[u] = j < n ? src[j] : make_uint4(0, 0, 0, 0);
    }
    unsigned acc = 0;
#pragma unroll
    for (int u = 0; u < 4; u++) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    if (acc == 0x9e3779b9u && n == 1) sink[0] = acc;
}

__global__ void __launch_bounds__(256) k_write_only(uint4 *__restrict__ dst, size_t n, unsigned value) {
    size_t i = (size_t)blockIdx.x * 256 * 4 + threadIdx.x;
#pragma unroll
    for (int u = 0; u < 4; u++) {
        size_t j = i + (size_t)u * 256;
        if (j < n) dst[j] = make_uint4(value, value + 1, value + 2, value + 3);
    }
}

/* In-place read-modify-write of the same buffer (the norm+rope access pattern). */
__global__ void __launch_bounds__(256) k_rmw(uint4 *__restrict__ buf, size_t n) {
    size_t i = (size_t)blockIdx.x * 256 * 4 + threadIdx.x;
    uint4 v[4];
#pragma unroll
    for (int u = 0; u < 4; u++) {
        size_t j = i + (size_t)u * 256;
        v[u] = j < n ? buf[j] : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int u = 0; u < 4; u++) {
        size_t j = i + (size_t)u * 256;
        v[u].x ^= 1u;
        if (j < n) buf[j] = v[u];
    }
}

/* Every wave reads 16 B per lane from a padded row layout (row stride 272 B),
 * the access pattern of an MFMA A operand; `iters` x 8 reads. */
__global__ void __launch_bounds__(256) k_lds_read(float *sink, int iters) {
    __shared__ __align__(16) uint16_t lds[64 * 136];
    for (int i = threadIdx.x; i < 64 * 136; i += 256) lds[i] = (uint16_t)i;
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const uint16_t *p = &lds[(lane & 31) * 136 + 8 * (lane >> 5)];
    uint4 acc = make_uint4(0, 0, 0, 0);
    for (int i = 0; i < iters; i++) {
#pragma unroll
        for (int t = 0; t < 8; t++) {
            u32x4 v = *reinterpret_cast<const volatile u32x4 *>(p + 16 * t + ((i & 1) ? 32 * 136 : 0));
            acc.x ^= v.x; acc.y ^= v.y; acc.z ^= v.z; acc.w ^= v.w;
        }
    }
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678u) sink[0] = 1.0f;
}

__global__ void __launch_bounds__(256) k_exp(float *sink, int iters) {
    float v[8];
    for (int j = 0; j < 8; j++) v[j] = -1.0f - threadIdx.x * 1e-3f - j;
    for (int i = 0; i < iters; i++) {
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = __builtin_amdgcn_exp2f(v[j]) - 2.0f;
    }
    float s = 0.0f;
    for (int j = 0; j < 8; j++) s += v[j];
    if (s == 12345.678f) sink[0] = s;
}

/* Do a SIMD's matrix core and its vector ALU work at the same time? A block of eight waves, two per SIMD: waves 0-3
 * issue `mfma_iters` x 8 independent 16x16x32 products, waves 4-7 `valu_iters` x 16 independent vector instructions of
 * one kind (1: v_fma_f32, 2: v_exp_f32, 3: the softmax's mix, one exponential per two others). Either count may be 0.
 * Timed three ways by the host (each alone, both together): together = the longer of the two means they overlap,
 * together = the sum means the SIMD does one or the other. Constant operands, so that the clock does not move. */
template <int KIND, int ACC>
__global__ void __launch_bounds__(512) k_mfma_with_valu(float *sink, int mfma_iters, int valu_iters) {
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    if (wave < 4) {
        f32x4 acc[8];
        for (int a = 0; a < 8; a++) acc[a] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        uint4 raw = make_uint4(0x3f803f80u + threadIdx.x, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u);
        bf16x8 x = __builtin_bit_cast(bf16x8, raw), y = x;
        for (int i = 0; i < mfma_iters; i++) {
#pragma unroll
            for (int a = 0; a < 8; a++) {
                if (ACC == 0) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(acc[a]) : "v"(x), "v"(y));
                else asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[a]) : "v"(x), "v"(y));
            }
        }
        float t = 0.0f;
        for (int a = 0; a < 8; a++) t += acc[a][0] + acc[a][3];
        if (t == 12345.678f) sink[0] = t;
    } else {
        float v[16];
        for (int j = 0; j < 16; j++) v[j] = -0.5f - threadIdx.x * 1e-3f - 0.01f * j;
        const float c = 0.999f, d = -1e-3f;
        for (int i = 0; i < valu_iters; i++) {
#pragma unroll
            for (int j = 0; j < 16; j++) {
                if (KIND == 1 || (KIND == 3 && j % 3 != 0)) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(v[j]) : "v"(c), "v"(d));
                else asm volatile("v_exp_f32 %0, %0" : "+v"(v[j]));
            }
        }
        float t = 0.0f;
        for (int j = 0; j < 16; j++) t += v[j];
        if (t == 12345.678f) sink[0] = t;
    }
}

}  // namespace

extern "C" {
int iris_mb_mfma_with_valu(void *stream, float *sink, int blocks, int mfma_iters, int valu_iters, int kind) {
    /* kind: 1 v_fma_f32, 2 v_exp_f32, 3 their mix; + 16: the products' accumulators in AGPRs instead of VGPRs */
    const dim3 g(blocks), b(512);
    hipStream_t st = (hipStream_t)stream;
    switch (kind) {
    case 1: hipLaunchKernelGGL((k_mfma_with_valu<1, 0>), g, b, 0, st, sink, mfma_iters, valu_iters); break;
    case 2: hipLaunchKernelGGL((k_mfma_with_valu<2, 0>), g, b, 0, st, sink, mfma_iters, valu_iters); break;
    case 3: hipLaunchKernelGGL((k_mfma_with_valu<3, 0>), g, b, 0, st, sink, mfma_iters, valu_iters); break;
    case 17: hipLaunchKernelGGL((k_mfma_with_valu<1, 1>), g, b, 0, st, sink, mfma_iters, valu_iters); break;
    case 18: hipLaunchKernelGGL((k_mfma_with_valu<2, 1>), g, b, 0, st, sink, mfma_iters, valu_iters); break;
    default: hipLaunchKernelGGL((k_mfma_with_valu<3, 1>), g, b, 0, st, sink, mfma_iters, valu_iters); break;
    }
    return (int)hipGetLastError();
}
int iris_mb_mfma(void *stream, float *sink, int blocks, int iters) {
    hipLaunchKernelGGL(k_mfma_peak, dim3(blocks), dim3(256), 0, (hipStream_t)stream, sink, iters);
    return (int)hipGetLastError();
}
/* ops: device buffer of 8 * 256 * 16 B operand data; iters x 16 MFMAs per wave */
int iris_mb_mfma_data(void *stream, const void *ops, float *sink, int blocks, int iters) {
    hipLaunchKernelGGL(k_mfma_data, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (const uint4 *)ops, sink, iters);
    return (int)hipGetLastError();
}
int iris_mb_mfma_data16(void *stream, const void *ops, float *sink, int blocks, int iters) {
    hipLaunchKernelGGL(k_mfma_data16, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (const uint4 *)ops, sink, iters);
    return (int)hipGetLastError();
}
int iris_mb_copy(void *stream, void *dst, const void *src, size_t bytes) {
    size_t n = bytes / 16;
    hipLaunchKernelGGL(k_copy, dim3((unsigned)((n + 1023) / 1024)), dim3(256), 0, (hipStream_t)stream,
                       (uint4 *)dst, (const uint4 *)src, n);
    return (int)hipGetLastError();
}
int iris_mb_read(void *stream, const void *src, size_t bytes, void *sink) {
    size_t n = bytes / 16;
    hipLaunchKernelGGL(k_read_only, dim3((unsigned)((n + 1023) / 1024)), dim3(256), 0, (hipStream_t)stream,
                       (const uint4 *)src, n, (unsigned *)sink);
    return (int)hipGetLastError();
}
int iris_mb_write(void *stream, void *dst, size_t bytes) {
    size_t n = bytes / 16;
    hipLaunchKernelGGL(k_write_only, dim3((unsigned)((n + 1023) / 1024)), dim3(256), 0, (hipStream_t)stream,
                       (uint4 *)dst, n, 7u);
    return (int)hipGetLastError();
}
int iris_mb_rmw(void *stream, void *buf, size_t bytes) {
    size_t n = bytes / 16;
    hipLaunchKernelGGL(k_rmw, dim3((unsigned)((n + 1023) / 1024)), dim3(256), 0, (hipStream_t)stream, (uint4 *)buf, n);
    return (int)hipGetLastError();
}
int iris_mb_lds(void *stream, float *sink, int blocks, int iters) {
    hipLaunchKernelGGL(k_lds_read, dim3(blocks), dim3(256), 0, (hipStream_t)stream, sink, iters);
    return (int)hipGetLastError();
}
int iris_mb_exp(void *stream, float *sink, int blocks, int iters) {
    hipLaunchKernelGGL(k_exp, dim3(blocks), dim3(256), 0, (hipStream_t)stream, sink, iters);
    return (int)hipGetLastError();
}
}
