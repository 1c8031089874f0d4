/*
 * Attention for the argument combinations the matrix-core kernels do not
 * take as they are. Two routes: (1) a padded, 16-byte aligned copy of q, k
 * and v (k_pack_heads), on which the matrix-core kernels then run, for any
 * head_dim <= 512 and any stride or alignment; (2) a scalar kernel for the
 * rest (non-positive scale, no keys, masked sequences beyond the matrix-core
 * kernel's limit): grouped kv heads, causal limit, key mask. The scalar
 * kernel is a correctness path, not a fast one: same mathematics as
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

/* head_dim beyond MAX_HD: the dot products are accumulated over chunks of MAX_HD dims (the K tile in LDS
 * holds one chunk at a time), and the output is produced MAX_HD dims at a time, each such pass walking the
 * keys again with its own softmax state.
 * Q_IN_LDS: the workgroup's 8 queries are kept in the LDS as f32 (head_dim <= 2048: 64 KB); beyond that they are
 * read from global memory where they are used (they stay in the caches: every lane reads the same addresses). */
template <bool Q_IN_LDS>
__global__ void __launch_bounds__(64)
k_attention_generic(uint16_t *out, int ldo, const uint16_t *q, const uint16_t *k, const uint16_t *v,
                    int ldq, int ldi, int seq_q, int seq_k, int kv_group, int hd, int kstride, float scale,
                    int causal, const int *key_mask) {
    extern __shared__ __align__(16) unsigned char smem[];
    float *qs = reinterpret_cast<float *>(smem);                 /* [QB][hd], or nothing */
    float *ps = qs + (Q_IN_LDS ? QB * hd : 0);                    /* [QB][KT] */
    uint16_t *kt = reinterpret_cast<uint16_t *>(ps + QB * KT);    /* [KT][kstride]: one chunk of dims */

    const int lane = threadIdx.x;
    const int head = blockIdx.y, kvh = head / kv_group;
    const int q0 = blockIdx.x * QB;
    const int nq = min(QB, seq_q - q0);

    if (Q_IN_LDS) {
        for (int idx = lane; idx < QB * hd; idx += 64) {
            int qq = idx / hd, d = idx - qq * hd;
            qs[idx] = qq < nq ? bf2f(q[(size_t)(q0 + qq) * ldq + (size_t)head * hd + d]) : 0.0f;
        }
    }

    int k_end = seq_k;
    if (causal) k_end = min(seq_k, q0 + nq);
    const uint16_t *kb = k + (size_t)kvh * hd, *vb = v + (size_t)kvh * hd;

    for (int oc = 0; oc < hd; oc += MAX_HD) {                     /* output dims oc .. oc + MAX_HD - 1 */
        float acc[QB][DSLOTS];
        float m_run[QB], l_run[QB], alpha[QB];
#pragma unroll
        for (int qq = 0; qq < QB; qq++) {
            m_run[qq] = -INFINITY; l_run[qq] = 0.0f; alpha[qq] = 1.0f;
#pragma unroll
            for (int t = 0; t < DSLOTS; t++) acc[qq][t] = 0.0f;
        }

        for (int k0 = 0; k0 < k_end; k0 += KT) {
            const int nk = min(KT, k_end - k0);
            float dot[QB];
#pragma unroll
            for (int qq = 0; qq < QB; qq++) dot[qq] = 0.0f;
            for (int dc = 0; dc < hd; dc += MAX_HD) {             /* this lane's key against every query, chunk by chunk */
                const int cw = min(MAX_HD, hd - dc);
                __syncthreads();
                for (int idx = lane; idx < KT * cw; idx += 64) {
                    int key = idx / cw, d = idx - key * cw;
                    kt[key * kstride + d] = key < nk ? kb[(size_t)(k0 + key) * ldi + dc + d] : (uint16_t)0;
                }
                __syncthreads();
                const uint16_t *kv = kt + lane * kstride;
#pragma unroll
                for (int qq = 0; qq < QB; qq++) {
                    float part = dot[qq];
                    if (Q_IN_LDS) {
                        const float *qv = qs + qq * hd + dc;
                        for (int d = 0; d < cw; d++) part = fmaf(qv[d], bf2f(kv[d]), part);
                    } else {
                        /* rows past the last query repeat it: their scores are never used */
                        const uint16_t *qg = q + (size_t)(q0 + min(qq, nq - 1)) * ldq + (size_t)head * hd + dc;
                        for (int d = 0; d < cw; d++) part = fmaf(bf2f(qg[d]), bf2f(kv[d]), part);
                    }
                    dot[qq] = part;
                }
            }

            const int key = k0 + lane;
            const bool in_range = lane < nk && (!key_mask || key_mask[key] != 0);
#pragma unroll
            for (int qq = 0; qq < QB; qq++) {
                const bool ok = in_range && qq < nq && (!causal || key <= q0 + qq);
                const float s = ok ? dot[qq] * scale : -INFINITY;
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
                const int d = oc + lane + 64 * t;
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
                const int d = oc + lane + 64 * t;
                if (d < hd) out[(size_t)(q0 + qq) * ldo + (size_t)head * hd + d] = f2bf(acc[qq][t] * inv);
            }
        }
    }
}

/* ---- padded, aligned copies for the matrix-core kernels --------------------------------------
 * pack: q, k, v (rows of `heads` / `kv_heads` heads of hd elements, any stride and alignment) ->
 * one fused row buffer [rows][(heads + 2 kv_heads) * hdp], every head padded with zeros to hdp
 * dims: q | k | v side by side, the layout the callers' own fused projections have. Zero dims
 * add nothing to q . k, and the extra output dims they produce are not copied back.
 * One thread per 16 B of the destination. */
struct PackSrc {
    const uint16_t *p[3];
    int ld[3], rows[3], heads[3];
};

template <bool VEC>
__global__ void __launch_bounds__(256)
k_pack_heads(uint16_t *__restrict__ dst, PackSrc src, int rows, int hd, int hdp) {
    const int cph = hdp / 8;                                   /* chunks per head */
    const int chunks = (src.heads[0] + src.heads[1] + src.heads[2]) * cph;
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)rows * chunks) return;
    const int r = (int)(i / chunks);
    const int at = (int)(i - (size_t)r * chunks);              /* chunk inside the destination row */
    int c = at, t = 0;                                         /* -> tensor t (q, k, v), chunk c inside its columns */
    while (c >= src.heads[t] * cph) { c -= src.heads[t] * cph; t++; }
    const int h = c / cph, d0 = 8 * (c - h * cph);
    uint32_t w[4] = {0, 0, 0, 0};
    if (r < src.rows[t] && d0 < hd) {
        const uint16_t *sp = src.p[t] + (size_t)r * src.ld[t] + (size_t)h * hd + d0;
        if (VEC) {                                             /* hd % 8 == 0: the chunk is whole, and 16-byte aligned */
            const uint4 v = *reinterpret_cast<const uint4 *>(sp);
            w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
        } else {
#pragma unroll
            for (int j = 0; j < 8; j++)
                if (d0 + j < hd) w[j >> 1] |= (uint32_t)sp[j] << (16 * (j & 1));
        }
    }
    *reinterpret_cast<uint4 *>(dst + ((size_t)r * chunks + at) * 8) = make_uint4(w[0], w[1], w[2], w[3]);
}

/* out[r][h * hd + d] = src[r][h * hdp + d], d < hd; out may have any stride and alignment */
__global__ void __launch_bounds__(256)
k_unpack_heads(uint16_t *__restrict__ out, int ldo, const uint16_t *__restrict__ src, int lds_, int rows, int heads,
               int hd, int hdp) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t per_row = (size_t)heads * hd;
    if (i >= (size_t)rows * per_row) return;
    const int r = (int)(i / per_row);
    const int c = (int)(i - (size_t)r * per_row), h = c / hd, d = c - h * hd;
    out[(size_t)r * ldo + c] = src[(size_t)r * lds_ + (size_t)h * hdp + d];
}

}  // namespace

extern "C" int iris_hip_attention_generic(void *stream, uint16_t *out, int ldo, const uint16_t *q, int ldq,
                                          const uint16_t *k, const uint16_t *v, int ldi, int seq_q,
                                          int seq_k, int heads, int kv_heads, int head_dim,
                                          float scale, int causal, const int *key_mask) {
    if (seq_q <= 0 || heads <= 0) return 0;
    /* K rows (one chunk of at most MAX_HD dims) padded to an odd number of 32-bit words: lanes
     * reading the same column of 64 different rows then hit 64 different banks. */
    const int chunk = head_dim < MAX_HD ? head_dim : MAX_HD;
    int kstride = ((chunk + 1) & ~1) + 2;
    if ((kstride / 2) % 2 == 0) kstride += 2;
    const bool q_in_lds = head_dim <= IRIS_ATTENTION_Q_IN_LDS_MAX_HEAD_DIM;
    const size_t smem = (q_in_lds ? (size_t)QB * head_dim * 4 : 0) + (size_t)QB * KT * 4 + (size_t)KT * kstride * 2;
    if (smem > 160 * 1024) return (int)hipErrorInvalidValue;
    static bool big_lds = false;
    if (!big_lds) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(k_attention_generic<true>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e == hipSuccess)
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(k_attention_generic<false>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return (int)e;
        big_lds = true;
    }
    dim3 grid((seq_q + QB - 1) / QB, heads);
    if (q_in_lds)
        hipLaunchKernelGGL(k_attention_generic<true>, grid, dim3(64), smem, (hipStream_t)stream, out, ldo, q, k, v,
                           ldq, ldi, seq_q, seq_k, heads / kv_heads, head_dim, kstride, scale, causal, key_mask);
    else
        hipLaunchKernelGGL(k_attention_generic<false>, grid, dim3(64), smem, (hipStream_t)stream, out, ldo, q, k, v,
                           ldq, ldi, seq_q, seq_k, heads / kv_heads, head_dim, kstride, scale, causal, key_mask);
    return (int)hipGetLastError();
}

extern "C" int iris_hip_pack_heads(void *stream, uint16_t *dst, const uint16_t *q, int ldq, int seq_q,
                                   const uint16_t *k, const uint16_t *v, int ldkv, int seq_k,
                                   int heads, int kv_heads, int hd, int hdp) {
    const int rows = seq_q > seq_k ? seq_q : seq_k;
    if (rows <= 0) return 0;
    PackSrc src = {{q, k, v}, {ldq, ldkv, ldkv}, {seq_q, seq_k, seq_k}, {heads, kv_heads, kv_heads}};
    const size_t n = (size_t)rows * (heads + 2 * kv_heads) * (hdp / 8);
    const unsigned blocks = (unsigned)((n + 255) / 256);
    const bool vec = hd % 8 == 0 && ldq % 8 == 0 && ldkv % 8 == 0 && (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v) & 15) == 0;
    if (vec) hipLaunchKernelGGL(k_pack_heads<true>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, dst, src, rows, hd, hdp);
    else hipLaunchKernelGGL(k_pack_heads<false>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, dst, src, rows, hd, hdp);
    return (int)hipGetLastError();
}

extern "C" int iris_hip_unpack_heads(void *stream, uint16_t *out, int ldo, const uint16_t *src, int ld_src,
                                     int rows, int heads, int hd, int hdp) {
    const size_t n = (size_t)rows * heads * hd;
    if (!n) return 0;
    hipLaunchKernelGGL(k_unpack_heads, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, out, ldo, src,
                       ld_src, rows, heads, hd, hdp);
    return (int)hipGetLastError();
}
