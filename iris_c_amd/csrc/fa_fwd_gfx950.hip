/*
 * Flash-attention forward for gfx950 (MI355X), head_dim 128, bf16 inputs,
 * f32 accumulation on the matrix cores (v_mfma_f32_32x32x16_bf16).
 *
 * What it computes (reference iris_dev.h:83-92, iris_cuda.cu:597-682 for the
 * online-softmax recurrence): for every head h and query i
 *     out[i] = softmax_j(scale * q_i . k_j) v_j   over the valid keys j
 * where key j is valid when j < seq_k, (causal ? j <= i : true) and
 * (key_mask ? key_mask[j] != 0 : true). A query without valid keys gives a
 * zero row. P is rounded to bf16 for the P.V product while the row sum uses
 * the unrounded f32 values (reference iris_cuda.cu:656-665).
 *
 * Shape of the computation on CDNA4
 * ---------------------------------
 * One workgroup = 4 waves = 128 queries of one head; each wave owns 32
 * queries for the whole kernel. Keys/values stream through LDS in tiles of
 * 64, the next tile travelling HBM -> registers while the current one is
 * being multiplied.
 *
 * Both products are issued transposed so that a query is a COLUMN of every
 * accumulator: S^T = K Q^T (A = K tile from LDS, B = Q^T held in registers)
 * and O^T += V^T P^T (A = V^T from LDS, B = P^T). In the 32x32 accumulator
 * layout lane l holds column l%32, so each lane carries one query: its
 * running max, its running sum and its rescale factor are plain per-lane
 * scalars, the 32 scores of a 64-key tile that a lane holds all belong to
 * that query, and exp2(S^T) converted to bf16 IS the B operand of the second
 * product -- no LDS round trip, no cross-lane shuffles except one
 * v_permlane32_swap per tile to combine the two half-waves' row maxima.
 *
 * LDS layout: K tile row-major [64][128+8] bf16 (272 B rows = 16 B x odd, so
 * the 16 consecutive keys a ds_read_b128 phase touches fall in distinct
 * banks). V tile transposed [128][64+8] with the 16 keys of every MFMA
 * k-step stored in the order the P^T registers hold them
 * (pos = 8*((key/4)&1) + 4*((key/8)&1) + key%4), which makes every A operand
 * of the second product a single ds_read_b128.
 *
 * Workgroups are numbered so that each XCD (own L2) walks a contiguous range
 * of (head, query-tile) pairs: the K/V of a head are then fetched into one
 * L2 instead of eight.
 */
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "iris_kernels_hip.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

namespace {

constexpr int BM = 128;            /* queries per workgroup (32 per wave) */
constexpr int BN = 64;             /* keys per tile */
constexpr int HD = 128;
constexpr int THREADS = 256;
constexpr int KS = HD + 8;         /* K tile row stride in elements */
constexpr int VS = BN + 8;         /* V^T tile row stride in elements */
constexpr int XCDS = 8;

struct TileRegs {
    uint4 k[4];
    uint4 v[4];
};

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    f32x2 p = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(p, bf16x2));
}

/* Max (or sum) of a value with the same lane of the other half-wave. */
__device__ __forceinline__ float half_swap_max(float v) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float half_swap_sum(float v) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

/* HBM -> registers: this thread's share of the 64-key tile starting at k0.
 * K: 16 B pieces in row order. V: four consecutive keys x eight dims, so the
 * 4x8 block can be transposed in registers. Rows past seq_k read as zero. */
__device__ __forceinline__ void fetch_tile(TileRegs &t, const uint16_t *kbase, const uint16_t *vbase,
                                           int ldi, int k0, int seq_k, int tid) {
    const int krow = tid >> 4, kcol = (tid & 15) * 8;
    const int lane = tid & 63, wave = tid >> 6;
    const int vkey = 4 * (lane & 15), vcol = (4 * wave + (lane >> 4)) * 8;
#pragma unroll
    for (int c = 0; c < 4; c++) {
        int kk = k0 + krow + 16 * c;
        t.k[c] = kk < seq_k ? *reinterpret_cast<const uint4 *>(kbase + (size_t)kk * ldi + kcol)
                            : make_uint4(0, 0, 0, 0);
        int vk = k0 + vkey + c;
        t.v[c] = vk < seq_k ? *reinterpret_cast<const uint4 *>(vbase + (size_t)vk * ldi + vcol)
                            : make_uint4(0, 0, 0, 0);
    }
}

/* Registers -> LDS. */
__device__ __forceinline__ void store_tile(const TileRegs &t, uint16_t *Ks, uint16_t *Vt, int tid) {
    const int krow = tid >> 4, kcol = (tid & 15) * 8;
#pragma unroll
    for (int c = 0; c < 4; c++)
        *reinterpret_cast<uint4 *>(&Ks[(krow + 16 * c) * KS + kcol]) = t.k[c];

    const int lane = tid & 63, wave = tid >> 6;
    const int m = lane & 15;                       /* group of 4 keys */
    const int d0 = (4 * wave + (lane >> 4)) * 8;
    /* position of key 4m inside its 16-key k-step, in P^T register order */
    const int pos = 16 * (m >> 2) + 8 * (m & 1) + 4 * ((m >> 1) & 1);
    const uint32_t a0[4] = {t.v[0].x, t.v[0].y, t.v[0].z, t.v[0].w};
    const uint32_t a1[4] = {t.v[1].x, t.v[1].y, t.v[1].z, t.v[1].w};
    const uint32_t a2[4] = {t.v[2].x, t.v[2].y, t.v[2].z, t.v[2].w};
    const uint32_t a3[4] = {t.v[3].x, t.v[3].y, t.v[3].z, t.v[3].w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        uint2 even, odd;
        even.x = __builtin_amdgcn_perm(a1[i], a0[i], 0x05040100u);
        even.y = __builtin_amdgcn_perm(a3[i], a2[i], 0x05040100u);
        odd.x = __builtin_amdgcn_perm(a1[i], a0[i], 0x07060302u);
        odd.y = __builtin_amdgcn_perm(a3[i], a2[i], 0x07060302u);
        *reinterpret_cast<uint2 *>(&Vt[(d0 + 2 * i) * VS + pos]) = even;
        *reinterpret_cast<uint2 *>(&Vt[(d0 + 2 * i + 1) * VS + pos]) = odd;
    }
}

template <bool CAUSAL, bool MASK>
__global__ void __launch_bounds__(THREADS, 2)
k_fa_fwd_hd128(uint16_t *__restrict__ out, int ldo, const uint16_t *__restrict__ q,
               const uint16_t *__restrict__ k, const uint16_t *__restrict__ v, int ldi,
               int seq_q, int seq_k, int q_tiles, int total_work, int work_per_xcd,
               int kv_group, float scale_log2, const int *__restrict__ key_mask) {
    __shared__ __align__(16) uint16_t Ks[BN * KS];
    __shared__ __align__(16) uint16_t Vt[HD * VS];

    /* XCD-aware numbering: hardware deals workgroups round-robin to the 8
     * XCDs, so id%8 is the XCD; give each XCD a contiguous slice of the
     * head-major work list. */
    const int work = (blockIdx.x % XCDS) * work_per_xcd + blockIdx.x / XCDS;
    if (work >= total_work) return;
    const int head = work / q_tiles;
    int qt = work - head * q_tiles;
    if (CAUSAL) qt = q_tiles - 1 - qt;             /* longest rows first */
    const int kvh = head / kv_group;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, hh = lane >> 5;
    const int q0 = qt * BM, wq0 = q0 + wave * 32, qrow = wq0 + col;

    const uint16_t *kbase = k + (size_t)kvh * HD;
    const uint16_t *vbase = v + (size_t)kvh * HD;

    /* Q^T as B operands: lane (query col, half hh) holds dims 16t + 8hh .. +7. */
    bf16x8 qb[8];
    {
        const uint16_t *qp = q + (size_t)qrow * ldi + (size_t)head * HD + 8 * hh;
#pragma unroll
        for (int t = 0; t < 8; t++) {
            uint4 raw = qrow < seq_q ? *reinterpret_cast<const uint4 *>(qp + 16 * t) : make_uint4(0, 0, 0, 0);
            qb[t] = __builtin_bit_cast(bf16x8, raw);
        }
    }

    f32x16 o[4];
#pragma unroll
    for (int db = 0; db < 4; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[db][r] = 0.0f;
    float m_run = -INFINITY, l_run = 0.0f;

    int k_end = seq_k;
    if (CAUSAL) k_end = min(seq_k, q0 + BM);       /* keys beyond the last query of the block are never valid */
    const int ntiles = (k_end + BN - 1) / BN;

    TileRegs tile;
    if (ntiles > 0) fetch_tile(tile, kbase, vbase, ldi, 0, seq_k, tid);

    for (int it = 0; it < ntiles; it++) {
        const int k0 = it * BN;
        __syncthreads();                           /* everyone is done reading the previous tile */
        store_tile(tile, Ks, Vt, tid);
        __syncthreads();
        if (it + 1 < ntiles) fetch_tile(tile, kbase, vbase, ldi, k0 + BN, seq_k, tid);

        /* ---- S^T = K Q^T : two 32-key blocks, 8 k-steps over the head dim ---- */
        f32x16 s0, s1;
#pragma unroll
        for (int r = 0; r < 16; r++) { s0[r] = 0.0f; s1[r] = 0.0f; }
#pragma unroll
        for (int t = 0; t < 8; t++) {
            bf16x8 ka = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(&Ks[col * KS + 16 * t + 8 * hh]));
            bf16x8 kb = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(&Ks[(32 + col) * KS + 16 * t + 8 * hh]));
            s0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, qb[t], s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kb, qb[t], s1, 0, 0, 0);
        }
        /* register r of block b holds key k0 + 32b + 8(r/4) + 4hh + r%4 for query qrow */

        /* ---- validity: range / key mask (wave-uniform 64-bit set), causal (per lane) ---- */
        unsigned long long valid = ~0ull;
        if (k0 + BN > seq_k) valid = (1ull << (seq_k - k0)) - 1ull;
        if (MASK) valid &= __ballot((k0 + lane < seq_k) && key_mask[min(k0 + lane, seq_k - 1)] != 0);
        if (valid != ~0ull) {
            const unsigned long long mine = valid >> (4 * hh);
            const uint32_t lo = (uint32_t)mine, hi = (uint32_t)(mine >> 32);
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int bit = 8 * (r >> 2) + (r & 3);
                if (!((lo >> bit) & 1u)) s0[r] = -INFINITY;
                if (!((hi >> bit) & 1u)) s1[r] = -INFINITY;
            }
        }
        if (CAUSAL && k0 + BN - 1 > wq0) {
            const int lim = qrow - k0 - 4 * hh;    /* key offset const_r valid iff const_r <= lim */
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int off = 8 * (r >> 2) + (r & 3);
                if (off > lim) s0[r] = -INFINITY;
                if (off + 32 > lim) s1[r] = -INFINITY;
            }
        }

        /* ---- online softmax, one query per lane ---- */
        float mx = fmaxf(s0[0], s1[0]);
#pragma unroll
        for (int r = 1; r < 16; r++) mx = fmaxf(mx, fmaxf(s0[r], s1[r]));
        mx = half_swap_max(mx);
        const float m_new = fmaxf(m_run, mx * scale_log2);
        const float m_ref = m_new == -INFINITY ? 0.0f : m_new;   /* finite while every key so far is masked */
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_ref);
        m_run = m_new;
        const float neg_m = -m_ref;

        float psum = 0.0f;
        uint32_t pw[16];                            /* P^T as bf16 pairs: pw[4*t + j] = k-step t, elements 2j, 2j+1 */
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
            float p0 = __builtin_amdgcn_exp2f(fmaf(s0[r], scale_log2, neg_m));
            float p1 = __builtin_amdgcn_exp2f(fmaf(s0[r + 1], scale_log2, neg_m));
            float p2 = __builtin_amdgcn_exp2f(fmaf(s1[r], scale_log2, neg_m));
            float p3 = __builtin_amdgcn_exp2f(fmaf(s1[r + 1], scale_log2, neg_m));
            psum += (p0 + p1) + (p2 + p3);
            pw[r >> 1] = pack_bf16(p0, p1);
            pw[8 + (r >> 1)] = pack_bf16(p2, p3);
        }
        l_run = fmaf(l_run, alpha, psum);           /* per half-wave partial; halves are added at the end */

        if (__any(alpha != 1.0f)) {
#pragma unroll
            for (int db = 0; db < 4; db++)
#pragma unroll
                for (int r = 0; r < 16; r++) o[db][r] *= alpha;
        }

        /* ---- O^T += V^T P^T : 4 dim blocks x 4 k-steps of 16 keys ---- */
#pragma unroll
        for (int t = 0; t < 4; t++) {
            uint4 praw = make_uint4(pw[4 * t], pw[4 * t + 1], pw[4 * t + 2], pw[4 * t + 3]);
            bf16x8 pb = __builtin_bit_cast(bf16x8, praw);
#pragma unroll
            for (int db = 0; db < 4; db++) {
                bf16x8 va = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(&Vt[(32 * db + col) * VS + 16 * t + 8 * hh]));
                o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, pb, o[db], 0, 0, 0);
            }
        }
    }

    /* ---- normalise and store: lane holds dims 32db + 8g + 4hh + {0..3} of query qrow ---- */
    const float l_tot = half_swap_sum(l_run);
    const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
    if (qrow < seq_q) {
        uint16_t *op = out + (size_t)qrow * ldo + (size_t)head * HD + 4 * hh;
#pragma unroll
        for (int db = 0; db < 4; db++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                uint2 w;
                w.x = pack_bf16(o[db][4 * g] * inv, o[db][4 * g + 1] * inv);
                w.y = pack_bf16(o[db][4 * g + 2] * inv, o[db][4 * g + 3] * inv);
                *reinterpret_cast<uint2 *>(op + 32 * db + 8 * g) = w;
            }
    }
}

}  // namespace

extern "C" int iris_hip_fa_hd128(void *stream, uint16_t *out, int ldo, const uint16_t *q,
                                 const uint16_t *k, const uint16_t *v, int ldi, int seq_q,
                                 int seq_k, int heads, int kv_heads, float scale, int causal,
                                 const int *key_mask) {
    const int q_tiles = (seq_q + BM - 1) / BM;
    const int total = q_tiles * heads;
    const int per_xcd = (total + XCDS - 1) / XCDS;
    const dim3 grid(per_xcd * XCDS), block(THREADS);
    const float scale_log2 = scale * 1.4426950408889634f;
    const int kv_group = heads / kv_heads;
    hipStream_t st = (hipStream_t)stream;
#define FA_LAUNCH(C, M)                                                                          \
    hipLaunchKernelGGL((k_fa_fwd_hd128<C, M>), grid, block, 0, st, out, ldo, q, k, v, ldi, seq_q, \
                       seq_k, q_tiles, total, per_xcd, kv_group, scale_log2, key_mask)
    if (causal) {
        if (key_mask) FA_LAUNCH(true, true); else FA_LAUNCH(true, false);
    } else {
        if (key_mask) FA_LAUNCH(false, true); else FA_LAUNCH(false, false);
    }
#undef FA_LAUNCH
    return (int)hipGetLastError();
}
