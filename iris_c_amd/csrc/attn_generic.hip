/*
 * Attention for every argument combination the matrix-core kernel does not
 * take (head_dim != 128, unaligned pointers or strides, non-positive scale):
 * any head_dim <= 512, grouped kv heads, causal limit, key mask. A
 * correctness path, not a fast one: same mathematics as
 * reference iris_cuda.cu:514-536 (max-subtracted softmax with expf over the
 * valid keys, zero row when there is none), computed with an online softmax
 * so no score matrix is materialised.
 *
 * One wave per workgroup handles QB queries of one head. Per 64-key tile:
 * phase 1 puts one key on each lane (the K tile sits in LDS, rows padded to
 * an odd number of 32-bit words), phase 2 puts output dims on lanes and
 * streams the V rows from memory with coalesced reads.
 */
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "iris_kernels_hip.h"

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

namespace {

constexpr int QB = 8;
constexpr int KT = 64;
constexpr int MAX_HD = 512;
constexpr int DSLOTS = MAX_HD / 64;

__device__ __forceinline__ float bf2f(uint16_t v) { return __uint_as_float((uint32_t)v << 16); }

__device__ __forceinline__ uint16_t f2bf(float f) {
    f32x2 p = {f, 0.0f};
    return (uint16_t)(__builtin_bit_cast(uint32_t, __builtin_convertvector(p, bf16x2)) & 0xffffu);
}

__device__ __forceinline__ float wave_max(float v) {
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

__global__ void __launch_bounds__(64)
k_attention_generic(uint16_t *out, int ldo, const uint16_t *q, const uint16_t *k, const uint16_t *v,
                    int ldq, int ldi, int seq_q, int seq_k, int kv_group, int hd, int kstride, float scale,
                    int causal, const int *key_mask) {
    extern __shared__ __align__(16) unsigned char smem[];
    float *qs = reinterpret_cast<float *>(smem);                 /* [QB][hd] */
    float *ps = qs + QB * hd;                                     /* [QB][KT] */
    uint16_t *kt = reinterpret_cast<uint16_t *>(ps + QB * KT);    /* [KT][kstride] */

    const int lane = threadIdx.x;
    const int head = blockIdx.y, kvh = head / kv_group;
    const int q0 = blockIdx.x * QB;
    const int nq = min(QB, seq_q - q0);

    for (int idx = lane; idx < QB * hd; idx += 64) {
        int qq = idx / hd, d = idx - qq * hd;
        qs[idx] = qq < nq ? bf2f(q[(size_t)(q0 + qq) * ldq + (size_t)head * hd + d]) : 0.0f;
    }

    float acc[QB][DSLOTS];
    float m_run[QB], l_run[QB], alpha[QB];
#pragma unroll
    for (int qq = 0; qq < QB; qq++) {
        m_run[qq] = -INFINITY; l_run[qq] = 0.0f; alpha[qq] = 1.0f;
#pragma unroll
        for (int t = 0; t < DSLOTS; t++) acc[qq][t] = 0.0f;
    }

    int k_end = seq_k;
    if (causal) k_end = min(seq_k, q0 + nq);
    const uint16_t *kb = k + (size_t)kvh * hd, *vb = v + (size_t)kvh * hd;

    for (int k0 = 0; k0 < k_end; k0 += KT) {
        const int nk = min(KT, k_end - k0);
        __syncthreads();
        for (int idx = lane; idx < KT * hd; idx += 64) {
            int key = idx / hd, d = idx - key * hd;
            kt[key * kstride + d] = key < nk ? kb[(size_t)(k0 + key) * ldi + d] : (uint16_t)0;
        }
        __syncthreads();

        const int key = k0 + lane;
        const bool in_range = lane < nk && (!key_mask || key_mask[key] != 0);
#pragma unroll
        for (int qq = 0; qq < QB; qq++) {
            float dot = 0.0f;
            const float *qv = qs + qq * hd;
            const uint16_t *kv = kt + lane * kstride;
            for (int d = 0; d < hd; d++) dot = fmaf(qv[d], bf2f(kv[d]), dot);
            const bool ok = in_range && qq < nq && (!causal || key <= q0 + qq);
            const float s = ok ? dot * scale : -INFINITY;
            const float m_new = fmaxf(m_run[qq], wave_max(s));
            const float m_ref = m_new == -INFINITY ? 0.0f : m_new;
            alpha[qq] = expf(m_run[qq] - m_ref);
            const float p = ok ? expf(s - m_ref) : 0.0f;
            l_run[qq] = l_run[qq] * alpha[qq] + wave_sum(p);
            m_run[qq] = m_new;
            ps[qq * KT + lane] = p;
        }
        __syncthreads();

#pragma unroll
        for (int t = 0; t < DSLOTS; t++) {
            const int d = lane + 64 * t;
            if (d >= hd) break;
#pragma unroll
            for (int qq = 0; qq < QB; qq++) acc[qq][t] *= alpha[qq];
            for (int j = 0; j < nk; j++) {
                const float vv = bf2f(vb[(size_t)(k0 + j) * ldi + d]);
#pragma unroll
                for (int qq = 0; qq < QB; qq++) acc[qq][t] = fmaf(ps[qq * KT + j], vv, acc[qq][t]);
            }
        }
    }

#pragma unroll
    for (int qq = 0; qq < QB; qq++) {
        if (qq >= nq) break;
        const float inv = l_run[qq] > 0.0f ? 1.0f / l_run[qq] : 0.0f;
#pragma unroll
        for (int t = 0; t < DSLOTS; t++) {
            const int d = lane + 64 * t;
            if (d < hd) out[(size_t)(q0 + qq) * ldo + (size_t)head * hd + d] = f2bf(acc[qq][t] * inv);
        }
    }
}

}  // namespace

extern "C" int iris_hip_attention_generic(void *stream, uint16_t *out, int ldo, const uint16_t *q, int ldq,
                                          const uint16_t *k, const uint16_t *v, int ldi, int seq_q,
                                          int seq_k, int heads, int kv_heads, int head_dim,
                                          float scale, int causal, const int *key_mask) {
    if (seq_q <= 0 || heads <= 0) return 0;
    /* K rows padded to an odd number of 32-bit words: lanes reading the same
     * column of 64 different rows then hit 64 different banks. */
    int kstride = ((head_dim + 1) & ~1) + 2;
    if ((kstride / 2) % 2 == 0) kstride += 2;
    const size_t smem = (size_t)QB * head_dim * 4 + (size_t)QB * KT * 4 + (size_t)KT * kstride * 2;
    static bool big_lds = false;
    if (!big_lds) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(k_attention_generic),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 120 * 1024);
        if (e != hipSuccess) return (int)e;
        big_lds = true;
    }
    dim3 grid((seq_q + QB - 1) / QB, heads);
    hipLaunchKernelGGL(k_attention_generic, grid, dim3(64), smem, (hipStream_t)stream, out, ldo, q, k, v,
                       ldq, ldi, seq_q, seq_k, heads / kv_heads, head_dim, kstride, scale, causal, key_mask);
    return (int)hipGetLastError();
}
