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
 * One workgroup = 8 waves = 256 queries of one head (4 waves = 128 queries
 * when that would leave CUs without work); each wave owns 32 queries for the
 * whole kernel, two waves share a SIMD. Keys/values stream through two LDS
 * stages in tiles of 64: while tile i is multiplied, tile i+1 moves
 * registers -> LDS and tile i+2 moves HBM -> registers; one barrier per tile.
 * Every wave reads the whole K and V tile, so 256 queries per workgroup mean
 * half the L2 -> LDS traffic and half the LDS writes per query of 128.
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
 * banks). V tile row-major too, [64][128+32] (320 B rows); the V^T operand
 * is produced by the LDS transpose read ds_read_b64_tr_b16, which hands lane
 * i of a 16-lane group column i of a 4-row x 16-column block: four
 * consecutive keys of one head dim, which is exactly the group of keys that
 * four consecutive P^T registers of that lane belong to. With 320 B rows the
 * four rows of a group fall in disjoint banks.
 *
 * The running max is only raised when some query of the wave exceeds it by
 * more than 2^8 (the accumulators are then rescaled); otherwise the
 * exponentials are taken against the older max. Softmax is invariant to that
 * shift, and exp2 arguments stay <= 8, far from overflow.
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
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

namespace {

/* A workgroup is WAVES (4 or 8) waves of 32 queries: BM = 32 * WAVES queries, 64 * WAVES threads. */
constexpr int BN = 64;             /* keys per tile */
constexpr int HD = 128;
constexpr int KS = HD + 8;         /* K tile row stride in elements (272 B) */
constexpr int VS = HD + 32;        /* V tile row stride in elements (320 B) */
constexpr int K_TILE = BN * KS;    /* elements */
constexpr int V_TILE = BN * VS;
constexpr int STAGE = K_TILE + V_TILE;
constexpr int XCDS = 8;
constexpr float RESCALE_THRESHOLD = 8.0f;   /* log2 units */

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

/* This thread's share of one K/V tile: NP = 1024 / threads pieces of 16 B of K and of V,
 * RSTEP = threads / 16 rows apart. */
template <int NP>
struct TileRegs {
    u32x4 k[NP], v[NP];
};

/* Workgroup barrier that only waits for this wave's LDS traffic. __syncthreads()
 * would also wait for outstanding global loads (vmcnt(0)), i.e. for the tile
 * that was requested precisely so that it arrives later. */
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    f32x2 p = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(p, bf16x2));
}

__device__ __forceinline__ float max3(float a, float b, float c) {
    float d;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
    return d;
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

/* HBM -> registers: 16 B pieces of the 64-key tile whose first row is at
 * `kt` / `vt` (wave-uniform pointers), at this thread's four row offsets. */
template <int NP>
__device__ __forceinline__ void fetch_tile(TileRegs<NP> &t, const uint16_t *kt, const uint16_t *vt,
                                           const uint32_t *off) {
    const char *kc = reinterpret_cast<const char *>(kt), *vc = reinterpret_cast<const char *>(vt);
#pragma unroll
    for (int c = 0; c < NP; c++) {
        t.k[c] = *reinterpret_cast<const u32x4 *>(kc + off[c]);
        t.v[c] = *reinterpret_cast<const u32x4 *>(vc + off[c]);
    }
}

/* Registers -> LDS stage. */
template <int NP>
__device__ __forceinline__ void store_tile(const TileRegs<NP> &t, uint16_t *stage, int tid) {
    constexpr int RSTEP = 64 / NP;
    const int row = tid >> 4, col = (tid & 15) * 8;
    uint16_t *kp = &stage[row * KS + col], *vp = &stage[K_TILE + row * VS + col];
#pragma unroll
    for (int c = 0; c < NP; c++) {
        *reinterpret_cast<u32x4 *>(kp + c * RSTEP * KS) = t.k[c];
        *reinterpret_cast<u32x4 *>(vp + c * RSTEP * VS) = t.v[c];
    }
}

/* Byte offsets of this thread's four rows of a tile starting at key k0; rows
 * past the end are redirected to the last valid row (their scores are masked
 * and their probabilities are exactly zero, so the values never matter). */
template <int NP>
__device__ __forceinline__ void tile_offsets(uint32_t (&off)[NP], int tid, int ldi, int k0, int seq_k) {
    const int row = tid >> 4, col = (tid & 15) * 8;
    constexpr int RSTEP = 64 / NP;
#pragma unroll
    for (int c = 0; c < NP; c++) {
        int r = min(row + RSTEP * c, seq_k - 1 - k0);
        off[c] = (uint32_t)(r * ldi + col) * 2u;
    }
}

template <int WAVES, bool CAUSAL, bool MASK>
__global__ void __launch_bounds__(64 * WAVES, 2)
k_fa_fwd_hd128(uint16_t *__restrict__ out, int ldo, const uint16_t *__restrict__ q,
               const uint16_t *__restrict__ k, const uint16_t *__restrict__ v, int ldi,
               int seq_q, int seq_k, int q_tiles, int total_work, int work_per_xcd,
               int kv_group, float scale_log2, const int *__restrict__ key_mask) {
    extern __shared__ __align__(16) uint16_t lds[];     /* two stages of [K tile | V tile] */
    constexpr int BM = 32 * WAVES, NP = 16 / WAVES;

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
        const uint16_t *qp = q + (size_t)min(qrow, seq_q - 1) * ldi + (size_t)head * HD + 8 * hh;
#pragma unroll
        for (int t = 0; t < 8; t++) qb[t] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(qp + 16 * t));
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

    /* LDS read addresses (elements, relative to a stage).
     * K operand: row = key (col [+32]), 16 B at dims 16t + 8hh.
     * V^T operand: transpose read; lane supplies row 4hh + (lane%16)/4 (+16t, +8)
     * and columns 16*((lane/16)%2) + 4*(lane%4) (+32db). */
    const int k_rd = col * KS + 8 * hh;
    const int v_rd = K_TILE + (4 * hh + ((lane & 15) >> 2)) * VS + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

    /* Row offsets of this thread's 16 B pieces: one set for full tiles, one for
     * the last tile (rows past seq_k redirected to the last valid row). */
    const int last_k0 = (ntiles - 1) * BN;
    uint32_t off_full[NP], off_last[NP];
    tile_offsets(off_full, tid, ldi, 0, BN);
    tile_offsets(off_last, tid, ldi, last_k0, seq_k);

    /* ---- prologue: tile 0 -> stage 0, tile 1 -> registers. Tile indices past
     * the end are clamped to the last tile: the copy is redundant but keeps the
     * pipeline free of control flow. ---- */
    TileRegs<NP> tile;
    {
        uint32_t off[NP];
#pragma unroll
        for (int c = 0; c < NP; c++) off[c] = ntiles > 1 ? off_full[c] : off_last[c];
        fetch_tile(tile, kbase, vbase, off);
        store_tile(tile, lds, tid);
        const int kn = min(BN, last_k0);
#pragma unroll
        for (int c = 0; c < NP; c++) off[c] = kn == last_k0 ? off_last[c] : off_full[c];
        fetch_tile(tile, kbase + (size_t)kn * ldi, vbase + (size_t)kn * ldi, off);
    }
    __syncthreads();

    for (int it = 0; it < ntiles; it++) {
        const int k0 = it * BN;
        uint16_t *cur = lds + (it & 1) * STAGE;

        /* tile it+1: registers -> the other stage (its last readers passed the barrier
         * that ended the previous iteration); tile it+2: HBM -> registers */
        store_tile(tile, lds + ((it + 1) & 1) * STAGE, tid);
        {
            const int kn = min(k0 + 2 * BN, last_k0);
            const bool is_last = kn == last_k0;
            uint32_t off[NP];
#pragma unroll
            for (int c = 0; c < NP; c++) off[c] = is_last ? off_last[c] : off_full[c];
            fetch_tile(tile, kbase + (size_t)kn * ldi, vbase + (size_t)kn * ldi, off);
        }

        /* ---- S^T = K Q^T : two 32-key blocks, 8 k-steps over the head dim.
         * All 16 A operands are requested from LDS up front so their latency
         * overlaps instead of gating every MFMA. ---- */
        f32x16 s0, s1;
        {
            u32x4 ka[8], kb[8];
#pragma unroll
            for (int t = 0; t < 8; t++) {
                ka[t] = *reinterpret_cast<const u32x4 *>(&cur[k_rd + 16 * t]);
                kb[t] = *reinterpret_cast<const u32x4 *>(&cur[k_rd + 32 * KS + 16 * t]);
            }
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_setprio(1);
            const f32x16 zero = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
            s0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ka[0]), qb[0], zero, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kb[0]), qb[0], zero, 0, 0, 0);
#pragma unroll
            for (int t = 1; t < 8; t++) {
                s0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ka[t]), qb[t], s0, 0, 0, 0);
                s1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kb[t]), qb[t], s1, 0, 0, 0);
            }
            __builtin_amdgcn_s_setprio(0);
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
                const int koff = 8 * (r >> 2) + (r & 3);
                if (koff > lim) s0[r] = -INFINITY;
                if (koff + 32 > lim) s1[r] = -INFINITY;
            }
        }

        /* ---- online softmax, one query per lane ---- */
        float mx = max3(s0[0], s0[1], s1[0]);
        mx = max3(mx, s1[1], s0[2]);
#pragma unroll
        for (int r = 3; r < 16; r += 2) mx = max3(mx, s0[r], s0[r + 1 < 16 ? r + 1 : r]);
#pragma unroll
        for (int r = 2; r < 16; r += 2) mx = max3(mx, s1[r], s1[r + 1]);
        mx = half_swap_max(mx) * scale_log2;

        if (__any(mx > m_run + RESCALE_THRESHOLD)) {
            const float m_new = fmaxf(m_run, mx);
            const float alpha = __builtin_amdgcn_exp2f(m_run - (m_new == -INFINITY ? 0.0f : m_new));
            m_run = m_new;
            l_run *= alpha;
#pragma unroll
            for (int db = 0; db < 4; db++)
#pragma unroll
                for (int r = 0; r < 16; r++) o[db][r] *= alpha;
        }
        const float neg_m = m_run == -INFINITY ? 0.0f : -m_run;   /* finite while every key so far is masked */

        float psum0 = 0.0f, psum1 = 0.0f;
        uint32_t pw[16];                            /* P^T as bf16 pairs: pw[4*t + j] = k-step t, elements 2j, 2j+1 */
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
            float p0 = __builtin_amdgcn_exp2f(fmaf(s0[r], scale_log2, neg_m));
            float p1 = __builtin_amdgcn_exp2f(fmaf(s0[r + 1], scale_log2, neg_m));
            float p2 = __builtin_amdgcn_exp2f(fmaf(s1[r], scale_log2, neg_m));
            float p3 = __builtin_amdgcn_exp2f(fmaf(s1[r + 1], scale_log2, neg_m));
            psum0 += p0 + p1;
            psum1 += p2 + p3;
            pw[r >> 1] = pack_bf16(p0, p1);
            pw[8 + (r >> 1)] = pack_bf16(p2, p3);
        }
        l_run += psum0 + psum1;                     /* per half-wave partial; halves are added at the end */

        /* ---- O^T += V^T P^T : 4 k-steps of 16 keys x 4 dim blocks; the V^T
         * operands of two k-steps are requested together ---- */
#pragma unroll
        for (int tp = 0; tp < 4; tp += 2) {
            s16x4 lo[2][4], hi[2][4];
#pragma unroll
            for (int u = 0; u < 2; u++)
#pragma unroll
                for (int db = 0; db < 4; db++) {
                    const uint16_t *vp = &cur[v_rd + 16 * (tp + u) * VS + 32 * db];
                    lo[u][db] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(vp));
                    hi[u][db] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(vp + 8 * VS));
                }
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_setprio(1);
#pragma unroll
            for (int u = 0; u < 2; u++) {
                const int t = tp + u;
                uint4 praw = make_uint4(pw[4 * t], pw[4 * t + 1], pw[4 * t + 2], pw[4 * t + 3]);
                bf16x8 pb = __builtin_bit_cast(bf16x8, praw);
#pragma unroll
                for (int db = 0; db < 4; db++) {
                    s16x8 both = __builtin_shufflevector(lo[u][db], hi[u][db], 0, 1, 2, 3, 4, 5, 6, 7);
                    o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, both), pb, o[db], 0, 0, 0);
                }
            }
            __builtin_amdgcn_s_setprio(0);
        }
        lds_barrier();
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

constexpr size_t LDS_BYTES = 2 * STAGE * sizeof(uint16_t);
constexpr int CUS = 256;

template <int W, bool C, bool M>
int launch(hipStream_t st, uint16_t *out, int ldo, const uint16_t *q, const uint16_t *k,
           const uint16_t *v, int ldi, int seq_q, int seq_k, int heads, int kv_heads,
           float scale, const int *key_mask) {
    static bool configured = false;
    if (!configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(k_fa_fwd_hd128<W, C, M>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_BYTES);
        if (e != hipSuccess) return (int)e;
        configured = true;
    }
    const int q_tiles = (seq_q + 32 * W - 1) / (32 * W);
    const int total = q_tiles * heads;
    const int per_xcd = (total + XCDS - 1) / XCDS;
    hipLaunchKernelGGL((k_fa_fwd_hd128<W, C, M>), dim3(per_xcd * XCDS), dim3(64 * W), LDS_BYTES, st, out, ldo,
                       q, k, v, ldi, seq_q, seq_k, q_tiles, total, per_xcd, heads / kv_heads,
                       scale * 1.4426950408889634f, key_mask);
    return (int)hipGetLastError();
}

template <int W>
int launch_w(hipStream_t st, uint16_t *out, int ldo, const uint16_t *q, const uint16_t *k,
             const uint16_t *v, int ldi, int seq_q, int seq_k, int heads, int kv_heads, float scale,
             int causal, const int *key_mask) {
    if (causal) {
        if (key_mask) return launch<W, true, true>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, key_mask);
        return launch<W, true, false>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, key_mask);
    }
    if (key_mask) return launch<W, false, true>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, key_mask);
    return launch<W, false, false>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, key_mask);
}

}  // namespace

extern "C" int iris_hip_fa_hd128(void *stream, uint16_t *out, int ldo, const uint16_t *q,
                                 const uint16_t *k, const uint16_t *v, int ldi, int seq_q,
                                 int seq_k, int heads, int kv_heads, float scale, int causal,
                                 const int *key_mask) {
    hipStream_t st = (hipStream_t)stream;
    /* 256 queries per workgroup halve the K/V traffic from L2 and the LDS writes per query;
     * 128 give twice the workgroups when the problem is too small to fill the CUs. */
    const long wg256 = (long)((seq_q + 255) / 256) * heads;
    if (wg256 >= CUS)
        return launch_w<8>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, causal, key_mask);
    return launch_w<4>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, causal, key_mask);
}
