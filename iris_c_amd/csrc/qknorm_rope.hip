/*
 * Fused per-head Q/K RMSNorm + rotary embedding for gfx950, in place on bf16.
 *
 * Semantics (reference iris_cuda.cu:402-420): for token s and head h, with
 * v = x + s*ld + h*hd:  r = 1/sqrt(mean(v^2) + eps);  a = v[i0]*r*w[i0],
 * b = v[i1]*r*w[i1];  v[i0] = a*c - b*sn, v[i1] = b*c + a*sn with
 * (c, sn) = (cos, sin)[s*hd/2 + i] and (i0, i1) = (2i, 2i+1), or (i, i+hd/2)
 * when split_half. f32 math, one round-to-nearest-even at the store.
 *
 * Mapping for head_dim 128 (the only size the models use): one (token, head)
 * vector is 256 B = 16 lanes x 16 B, so a wave64 moves four vectors per
 * 128-bit load/store and the four are contiguous in memory (heads of one
 * token are adjacent). The sum of squares is reduced inside the 16-lane DPP
 * row (row_ror 8/4/2/1), so there is no LDS and no barrier. Each wave keeps
 * UNROLL independent vectors in flight. Q and K of the same rows can go in
 * one launch: the unit index then runs over q_heads + k_heads per token.
 *
 * HBM traffic per vector: 256 B read + 256 B written; the cos/sin rows
 * (512 B per token) are shared by all heads of the token and stay in L2.
 */
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "iris_kernels_hip.h"
#include "norm_rope_math.h"

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int kThreads = 256;
/* Measured on C2 (cold rows): 2 -> 13.2 us, 1 -> 14.1, 4 -> 14.0, 8 -> 16.3. Workgroups of 512
 * threads change nothing, 1024 cost 10 %; a persistent grid (4 or 8 workgroups per CU striding over
 * the units) is within 3 % either way; nontemporal loads cost 5 %. */
constexpr int kUnroll = 2;                       /* vectors in flight per 16-lane row */
constexpr int kUnitsPerBlock = (kThreads / 16) * kUnroll;

/* A second weight pair for the rows from `rows_a` on (STREAMS): the double-stream block normalises the text rows
 * and the image rows of the joint q | k | v buffer with different weights (reference
 * iris_transformer_flux.c:3796-3803, four calls); here they are one launch over all rows. */
struct SecondStream {
    const float *wq, *wk;
    int first_unit;                               /* rows_a * heads_total */
};

template <bool SPLIT, bool STREAMS, bool STREAMING_STORES>
__global__ void __launch_bounds__(kThreads)
k_norm_rope_hd128(uint16_t *__restrict__ xq, uint16_t *__restrict__ xk, int ld,
                  const float *__restrict__ wq, const float *__restrict__ wk,
                  const float *__restrict__ rope_cos, const float *__restrict__ rope_sin,
                  int units, int q_heads, int heads_total, uint32_t magic, float eps, SecondStream second) {
    const int sub = threadIdx.x & 15;             /* which 16 B of the 256 B vector */
    const int row = threadIdx.x >> 4;             /* 16-lane row inside the block */
    const int first = blockIdx.x * kUnitsPerBlock + row;

    /* Table columns this lane needs: consecutive pairs -> i = 4*sub..4*sub+3;
     * split-half -> i = 8*(sub&7)..+7 (shared with the partner lane). */
    const int tcol = SPLIT ? 8 * (sub & 7) : 4 * sub;

    /* Phase 1: request everything this thread needs for its kUnroll vectors --
     * the 16 B of x and the matching cos/sin entries -- before touching any of
     * it, so all the loads are in flight together. */
    constexpr int TN = SPLIT ? 2 : 1;               /* float4 table loads per vector */
    u32x4 raw[kUnroll];
    float4 ct[kUnroll][TN], st[kUnroll][TN];
    uint16_t *ptr[kUnroll];
    float4 wv[kUnroll][2];                          /* the norm weights of this lane's 8 dims */
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        int unit = first + u * (kThreads / 16);
        const bool live = unit < units;
        unit = live ? unit : 0;
        const bool later = STREAMS && unit >= second.first_unit;
        /* unit / heads_total; one head per token has no 32-bit magic (it would be 2^32) */
        const int s = heads_total == 1 ? unit : (int)__umulhi((uint32_t)unit, magic);
        const int h = unit - s * heads_total;
        const bool isk = h >= q_heads;
        uint16_t *base = isk ? xk + (size_t)(h - q_heads) * 128 : xq + (size_t)h * 128;
        /* the vector's weights: Q's or K's, of the first or (STREAMS) of the second row range */
        const float *wsel = isk ? (later ? second.wk : wk) : (later ? second.wq : wq);
        wv[u][0] = *reinterpret_cast<const float4 *>(wsel + sub * 8);
        wv[u][1] = *reinterpret_cast<const float4 *>(wsel + sub * 8 + 4);
        ptr[u] = live ? base + (size_t)s * ld + sub * 8 : nullptr;
        raw[u] = live ? *reinterpret_cast<const u32x4 *>(ptr[u]) : u32x4{0, 0, 0, 0};
        const float *cp = rope_cos + (size_t)s * 64 + tcol;
        const float *sp = rope_sin + (size_t)s * 64 + tcol;
#pragma unroll
        for (int i = 0; i < TN; i++) {
            ct[u][i] = *reinterpret_cast<const float4 *>(cp + 4 * i);
            st[u][i] = *reinterpret_cast<const float4 *>(sp + 4 * i);
        }
    }
    /* Phase 2: normalise, rotate, store. */
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        if (!ptr[u]) continue;
        float cv[8], sv[8];
        cv[0] = ct[u][0].x; cv[1] = ct[u][0].y; cv[2] = ct[u][0].z; cv[3] = ct[u][0].w;
        cv[4] = ct[u][TN - 1].x; cv[5] = ct[u][TN - 1].y; cv[6] = ct[u][TN - 1].z; cv[7] = ct[u][TN - 1].w;
        sv[0] = st[u][0].x; sv[1] = st[u][0].y; sv[2] = st[u][0].z; sv[3] = st[u][0].w;
        sv[4] = st[u][TN - 1].x; sv[5] = st[u][TN - 1].y; sv[6] = st[u][TN - 1].z; sv[7] = st[u][TN - 1].w;
        const float w8[8] = {wv[u][0].x, wv[u][0].y, wv[u][0].z, wv[u][0].w, wv[u][1].x, wv[u][1].y, wv[u][1].z, wv[u][1].w};
        const u32x4 out = nr_vector_hd128<SPLIT>(raw[u], w8, cv, sv, eps, sub);
        /* Write-through store (sc0 sc1): the rows leave the L2 as they are produced instead of at the
         * end-of-kernel write-back, 2-5 % faster on 59-118 MB calls whether the rows were cached or not.
         * Adding the streaming hint `nt` takes the two-tensor call on uncached rows from 23.0 to 21.2 us
         * but a call on rows that sit in the Infinity Cache from 9.4 to 12.7 us: it is taken
         * (STREAMING_STORES) only by calls so large that their rows cannot be resident in that cache. */
        if (STREAMING_STORES)
            asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1 nt" :: "v"(ptr[u]), "v"(out) : "memory");
        else
            asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" :: "v"(ptr[u]), "v"(out) : "memory");
    }
}

/* Any even head_dim: one wave per (token, head), lanes stride over pairs. */
__global__ void __launch_bounds__(64)
k_norm_rope_generic(uint16_t *x, int ld, const float *w, const float *rope_cos,
                    const float *rope_sin, int heads, int head_dim, float eps, int split_half) {
    const int s = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int half = head_dim / 2;
    uint16_t *v = x + (size_t)s * ld + (size_t)h * head_dim;
    float ss = 0.0f;
    for (int d = lane; d < head_dim; d += 64) {
        float f = __uint_as_float((uint32_t)v[d] << 16);
        ss = fmaf(f, f, ss);
    }
    for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
    const float inv = 1.0f / sqrtf(ss / (float)head_dim + eps);
    for (int i = lane; i < half; i += 64) {
        int i0 = split_half ? i : 2 * i, i1 = split_half ? i + half : 2 * i + 1;
        float a = __uint_as_float((uint32_t)v[i0] << 16) * (inv * w[i0]);
        float b = __uint_as_float((uint32_t)v[i1] << 16) * (inv * w[i1]);
        float c = rope_cos[(size_t)s * half + i], sn = rope_sin[(size_t)s * half + i];
        uint32_t packed = nr_pack_bf16(fmaf(-b, sn, a * c), fmaf(a, sn, b * c));
        v[i0] = (uint16_t)(packed & 0xffffu);
        v[i1] = (uint16_t)(packed >> 16);
    }
}

}  // namespace

/* unit / heads_total == umulhi(unit, magic) for unit < 2^24 and 2 <= heads_total < 2^8. For one
 * head the constant would be 2^32, which does not fit: 0 is returned and the kernel takes
 * unit / 1 = unit without it. */
extern "C" uint32_t iris_norm_rope_magic(int heads_total) {
    if (heads_total <= 1) return 0u;
    return (uint32_t)((0x100000000ull + (uint64_t)heads_total - 1) / (uint64_t)heads_total);
}

/* Rows that a call touches, from which size on they cannot all be resident in the 256 MB Infinity Cache together
 * with what else a model keeps there: such calls store with the streaming hint. */
static const long long kStreamingStoreBytes = 128ll << 20;

extern "C" int iris_norm_rope_streaming_stores(int seq, int heads_total) {
    return (long long)seq * heads_total * 256 >= kStreamingStoreBytes;
}

template <bool SPLIT, bool STREAMS>
static int launch_norm_rope(hipStream_t st, int blocks, bool streaming, uint16_t *xq, uint16_t *xk, int ld, const float *wq,
                            const float *wk, const float *rope_cos, const float *rope_sin, int units, int q_heads,
                            int heads_total, uint32_t magic, float eps, SecondStream second) {
    if (streaming)
        hipLaunchKernelGGL((k_norm_rope_hd128<SPLIT, STREAMS, true>), dim3(blocks), dim3(kThreads), 0, st, xq, xk, ld,
                           wq, wk, rope_cos, rope_sin, units, q_heads, heads_total, magic, eps, second);
    else
        hipLaunchKernelGGL((k_norm_rope_hd128<SPLIT, STREAMS, false>), dim3(blocks), dim3(kThreads), 0, st, xq, xk, ld,
                           wq, wk, rope_cos, rope_sin, units, q_heads, heads_total, magic, eps, second);
    return (int)hipGetLastError();
}

/* wq_b == NULL: one weight pair for all rows. Otherwise rows [rows_a, seq) take (wq_b, wk_b). */
extern "C" int iris_hip_norm_rope_hd128_streams(void *stream, uint16_t *xq, uint16_t *xk, int ld,
                                                const float *wq, const float *wk, const float *wq_b, const float *wk_b,
                                                int rows_a, const float *rope_cos, const float *rope_sin,
                                                int seq, int q_heads, int k_heads, float eps, int split_half) {
    const int heads_total = q_heads + k_heads;
    const int units = seq * heads_total;
    if (units <= 0) return 0;
    const uint32_t magic = iris_norm_rope_magic(heads_total);
    const int blocks = (units + kUnitsPerBlock - 1) / kUnitsPerBlock;
    hipStream_t st = (hipStream_t)stream;
    const bool streaming = iris_norm_rope_streaming_stores(seq, heads_total) != 0;
    const SecondStream second = {wq_b, wk_b, rows_a * heads_total};
    if (wq_b) {
        if (split_half)
            return launch_norm_rope<true, true>(st, blocks, streaming, xq, xk, ld, wq, wk, rope_cos, rope_sin, units, q_heads,
                                                heads_total, magic, eps, second);
        return launch_norm_rope<false, true>(st, blocks, streaming, xq, xk, ld, wq, wk, rope_cos, rope_sin, units, q_heads,
                                             heads_total, magic, eps, second);
    }
    if (split_half)
        return launch_norm_rope<true, false>(st, blocks, streaming, xq, xk, ld, wq, wk, rope_cos, rope_sin, units, q_heads,
                                             heads_total, magic, eps, second);
    return launch_norm_rope<false, false>(st, blocks, streaming, xq, xk, ld, wq, wk, rope_cos, rope_sin, units, q_heads,
                                          heads_total, magic, eps, second);
}

extern "C" int iris_hip_norm_rope_hd128(void *stream, uint16_t *xq, uint16_t *xk, int ld,
                                        const float *wq, const float *wk,
                                        const float *rope_cos, const float *rope_sin,
                                        int seq, int q_heads, int k_heads, float eps,
                                        int split_half) {
    return iris_hip_norm_rope_hd128_streams(stream, xq, xk, ld, wq, wk, nullptr, nullptr, 0, rope_cos, rope_sin, seq,
                                            q_heads, k_heads, eps, split_half);
}

extern "C" int iris_hip_norm_rope_generic(void *stream, uint16_t *x, int ld, const float *w,
                                          const float *rope_cos, const float *rope_sin,
                                          int seq, int heads, int head_dim, float eps,
                                          int split_half) {
    if (seq <= 0 || heads <= 0) return 0;
    hipLaunchKernelGGL(k_norm_rope_generic, dim3(seq, heads), dim3(64), 0, (hipStream_t)stream, x, ld,
                       w, rope_cos, rope_sin, heads, head_dim, eps, split_half);
    return (int)hipGetLastError();
}
