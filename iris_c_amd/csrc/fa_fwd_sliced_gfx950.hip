/*
 * Flash-attention forward for gfx950, head_dim 256 or 512 (the VAE mid-block
 * attention of the reference is one head of 512, iris_vae.c:1112-1124), bf16
 * in, f32 accumulation on the matrix cores. Same operator as the head_dim 128
 * kernel (reference iris_dev.h:83-92): causal limit, key mask, grouped kv
 * heads, zero row for a query without valid keys.
 *
 * A wave cannot hold a 512-wide output row block in registers, so the head
 * dimension is cut into NS slices of 128 and a group of NS waves shares 32
 * queries: wave (g, s) keeps Q[:, 128s .. 128s+127] and O[:, same] of group
 * g's queries. Workgroup = 8 waves = 8/NS query groups (64 queries at 512,
 * 128 at 256). For every tile of 32 keys
 *   A  each wave multiplies its slice, S_part^T = K[:, slice] Q[:, slice]^T
 *      (8 MFMAs 32x32x16), and leaves the partial scores in the LDS;
 *   B  the keys of the tile are dealt out to the NS waves of the group (8 each
 *      at 512): a wave adds the NS partial scores of ITS keys only, so the
 *      softmax is done once per group and not once per wave. The running max
 *      of a query is shared by the group: every wave publishes the largest of
 *      its 8 scores per query, all read the NS maxima and take the same
 *      decision (the max is only raised, and the accumulators rescaled, when a
 *      score exceeds it by more than 2^8). Then exp2 of the own keys, rounded
 *      to bf16, goes to the LDS in the layout of the B operand;
 *   C  every wave reads the whole P^T of the tile and adds
 *      O[:, slice]^T += V[:, slice]^T P^T (8 MFMAs).
 * Three barriers per tile (partial scores, maxima, probabilities). As in the
 * 128 kernel both products are transposed and a lane owns one query. The row
 * sum of a query is kept per wave over its own keys and added up at the end.
 *
 * K and V tiles have two LDS stages each (K two tiles ahead, V one) and are
 * fetched a further tile ahead into registers. Rows are unpadded; the 16 B
 * chunk c of row r sits in slot c ^ sw(r) of its 256 B group,
 * sw(r) = 4 (r % 4) + (r / 4) % 4: the 16 rows of a ds_read_b128 pass land in
 * 16 different slots, and the four rows of a transposing read in four
 * different 64 B windows.
 *
 * Where the time goes (16384 tokens x 1 head x 512, 0.90-0.93 ms, 24 % of the
 * bf16 matrix peak): a tile of 32 keys takes about 4000 cycles per wave, the
 * sum of a chain of dependent steps, each an LDS round trip of about 350
 * cycles or a chain of eight products that wait for one another (570): K
 * operands, partial scores out and in, maxima out and in, probabilities out
 * and in, V operands; the two waves of a SIMD are in the same step at the same
 * time (the barriers), so they do not fill each other's waits. What does NOT
 * bound it, each tried with the rest unchanged: the tile loads (direct loads,
 * register-staged loads or none at all: 0.90-0.93 ms), the second or the third
 * barrier (removed, wrong results: 0.90), the softmax arithmetic (done once
 * per wave instead of once per group: 0.93), two accumulator chains in the
 * score product (0.94), four waves of 64 queries with the whole register file
 * each instead of eight of 32 (every K and V operand then feeds two products:
 * 1.30 ms, a wave alone on its SIMD walks the chain more slowly than it saves).
 * The K/V tiles come from the L2 (96 % hits).
 */
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "iris_kernels_hip.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int BN = 32;             /* keys per tile */
constexpr int THREADS = 512;
constexpr int XCDS = 8;
constexpr float RESCALE_THRESHOLD = 8.0f;   /* log2 units */

__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    f32x2 p = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(p, bf16x2));
}

__device__ __forceinline__ float half_swap_max(float v) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float half_swap_sum(float v) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

__device__ __forceinline__ int sw(int row) { return ((row & 3) << 2) | ((row >> 2) & 3); }
/* slot of chunk c (16 B) of tile row r */
__device__ __forceinline__ int slot_of(int c, int row) { return (c & ~15) | ((c ^ sw(row)) & 15); }

template <int NS, bool CAUSAL, bool MASK>
__global__ void __launch_bounds__(THREADS, 2)
k_fa_fwd_sliced(uint16_t *__restrict__ out, int ldo, const uint16_t *__restrict__ q,
                const uint16_t *__restrict__ k, const uint16_t *__restrict__ v, int ldi,
                int seq_q, int seq_k, int q_tiles, int total_work, int work_per_xcd,
                int kv_group, float scale_log2, const int *__restrict__ key_mask) {
    constexpr int HD = 128 * NS;
    constexpr int QG = 8 / NS;             /* query groups per workgroup */
    constexpr int BM = 32 * QG;
    constexpr int TILE = BN * HD;          /* elements of a K (or V) tile */
    constexpr int CH = HD / 8;             /* 16 B chunks per row */
    constexpr int OWN = 4 / NS;            /* blocks of 8 keys a wave owns in a tile */
    constexpr int SLOTS = NS == 4 ? 3 : 4; /* blocks of partial scores a wave leaves for the others (at 512 its own one stays in registers) */

    extern __shared__ __align__(16) uint16_t lds[];     /* K stage 0, 1 | V stage 0, 1 | partial scores | P^T | maxima */
    f32x4 *x1 = reinterpret_cast<f32x4 *>(lds + 4 * TILE);            /* [8 waves][SLOTS][64 lanes] */
    uint16_t *x2 = reinterpret_cast<uint16_t *>(x1 + 8 * SLOTS * 64);  /* [QG][2 k-steps][2][32 queries][8] */
    float *x3 = reinterpret_cast<float *>(x2 + QG * 4 * 32 * 8);       /* [8 waves][32 queries] */

    const int work = (blockIdx.x % XCDS) * work_per_xcd + blockIdx.x / XCDS;
    if (work >= total_work) return;
    const int head = work / q_tiles;
    int qt = work - head * q_tiles;
    if (CAUSAL) qt = q_tiles - 1 - qt;
    const int kvh = head / kv_group;

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int sl = wave % NS, grp = wave / NS;
    const int col = lane & 31, hh = lane >> 5;
    const int q0 = qt * BM, wq0 = q0 + grp * 32, qrow = wq0 + col;

    const uint16_t *kbase = k + (size_t)kvh * HD;
    const uint16_t *vbase = v + (size_t)kvh * HD;

    int k_end = seq_k;
    if (CAUSAL) k_end = min(seq_k, q0 + BM);
    const int ntiles = (k_end + BN - 1) / BN;
    const int last_k0 = (ntiles - 1) * BN;

    /* ---- tile loads. A thread moves NS chunks of 16 B of a K tile and of a V tile: rows row0 + RSTEP c, chunk
     * tid % CH. They wait in registers for a whole tile period (global load -> ds_write one turn later): issuing a
     * direct global -> LDS load costs a wave about 100 cycles each here, eight of them a tile, on the critical path. */
    constexpr int NP = NS, RSTEP = THREADS / CH;
    const int row0 = tid / CH, cchunk = tid % CH;
    u32x4 tk[NP], tv[NP];
    auto fetch_k = [&](int k0) {
#pragma unroll
        for (int c = 0; c < NP; c++)
            tk[c] = *reinterpret_cast<const u32x4 *>(kbase + (size_t)min(k0 + row0 + RSTEP * c, seq_k - 1) * ldi + 8 * cchunk);
    };
    auto fetch_v = [&](int k0) {
#pragma unroll
        for (int c = 0; c < NP; c++)
            tv[c] = *reinterpret_cast<const u32x4 *>(vbase + (size_t)min(k0 + row0 + RSTEP * c, seq_k - 1) * ldi + 8 * cchunk);
    };
    int st_off[NP];                         /* where the thread's chunks go inside a stage (elements) */
#pragma unroll
    for (int c = 0; c < NP; c++) st_off[c] = (row0 + RSTEP * c) * HD + 8 * slot_of(cchunk, row0 + RSTEP * c);
    auto store = [&](uint16_t *stage, const u32x4 (&t)[NP]) {
#pragma unroll
        for (int c = 0; c < NP; c++) *reinterpret_cast<u32x4 *>(&stage[st_off[c]]) = t[c];
    };
    uint16_t *kst = lds, *vst = lds + 2 * TILE;
    fetch_k(0); fetch_v(0);
    store(kst, tk); store(vst, tv);
    fetch_k(min(BN, last_k0));
    store(kst + TILE, tk);
    fetch_k(min(2 * BN, last_k0)); fetch_v(min(BN, last_k0));      /* wait in registers for the first turn */

    /* This wave's slice of Q^T as B operands: dims 128 sl + 16t + 8hh .. +7. */
    bf16x8 qb[8];
    {
        const uint16_t *qp = q + (size_t)min(qrow, seq_q - 1) * ldi + (size_t)head * HD + 128 * sl + 8 * hh;
#pragma unroll
        for (int t = 0; t < 8; t++) qb[t] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(qp + 16 * t));
    }

    f32x16 o[4];
#pragma unroll
    for (int db = 0; db < 4; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[db][r] = 0.0f;
    float m_run = -INFINITY, l_run = 0.0f;     /* l_run: over this wave's keys only */

    /* LDS read offsets (elements, relative to a stage). K operand of k-step t: row = key `col`, chunk 16 sl + 2t + hh.
     * V^T operand (k-step t of 16 keys, dim block db, half hi): transposing read of rows 16t + 8hi + 4hh + (lane%16)/4,
     * 8 B at chunk 16 sl + 4 db + 2 ((lane/16)%2) + (lane%4)/2, element 4 (lane%2) inside it. */
    int k_rd[8], v_rd[2][4];
#pragma unroll
    for (int t = 0; t < 8; t++) k_rd[t] = col * HD + 8 * slot_of(16 * sl + 2 * t + hh, col);
#pragma unroll
    for (int hi = 0; hi < 2; hi++)
#pragma unroll
        for (int db = 0; db < 4; db++) {
            const int row = 8 * hi + 4 * hh + ((lane & 15) >> 2);      /* + 16 t: sw(row) does not change with t */
            v_rd[hi][db] = row * HD + 8 * slot_of(16 * sl + 4 * db + 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1), row) + 4 * (lane & 1);
        }

    lds_barrier();

    for (int it = 0; it < ntiles; it++) {
        const int k0 = it * BN;
        const uint16_t *kcur = kst + (it & 1) * TILE, *vcur = vst + (it & 1) * TILE;

        /* ---- A: partial scores over this wave's 128 dims ---- */
        f32x16 s;
        {
            u32x4 ka[8];
#pragma unroll
            for (int t = 0; t < 8; t++) ka[t] = *reinterpret_cast<const u32x4 *>(&kcur[k_rd[t]]);
            const f32x16 zero = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
            s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ka[0]), qb[0], zero, 0, 0, 0);
#pragma unroll
            for (int t = 1; t < 8; t++)
                s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ka[t]), qb[t], s, 0, 0, 0);
        }
        /* register r holds key k0 + 8 (r/4) + 4 hh + r%4 for query qrow: block r/4 of 8 keys. This wave owns blocks
         * OWN sl .. ; the others go to the LDS for their owners. */
#pragma unroll
        for (int g = 0; g < 4; g++) {
            if (NS == 4 && g == sl) continue;
            const int slot = NS == 4 ? (g < sl ? g : g - 1) : g;
            x1[(wave * SLOTS + slot) * 64 + lane] = f32x4{s[4 * g], s[4 * g + 1], s[4 * g + 2], s[4 * g + 3]};
        }
        lds_barrier();                                                       /* 1: partial scores */
        /* K stage (it % 2) and V stage ((it + 1) % 2) have no readers any more: K of tile it + 2 and V of tile it + 1
         * go there from the registers, and the loads of the turn after are issued */
        store(kst + (it & 1) * TILE, tk);
        store(vst + ((it + 1) & 1) * TILE, tv);
        fetch_k(min(k0 + 3 * BN, last_k0));
        fetch_v(min(k0 + 2 * BN, last_k0));

        f32x4 mine[OWN];
#pragma unroll
        for (int ob = 0; ob < OWN; ob++) {
            const int g = OWN * sl + ob;
            f32x4 a = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int p = 0; p < NS; p++) {                                   /* in slice order */
                if (p == sl) {
                    f32x4 own;
                    /* block g of this wave's registers; g is wave-uniform but not a constant: selected without indexing */
#pragma unroll
                    for (int gg = 0; gg < 4; gg++)
                        if (gg == g) own = f32x4{s[4 * gg], s[4 * gg + 1], s[4 * gg + 2], s[4 * gg + 3]};
                    a += own;
                } else {
                    const int slot = NS == 4 ? (g < p ? g : g - 1) : g;
                    a += x1[((grp * NS + p) * SLOTS + slot) * 64 + lane];
                }
            }
            mine[ob] = a;
        }

        /* ---- validity of the own keys: key k0 + 8 (OWN sl + ob) + 4 hh + r ---- */
        unsigned valid = ~0u;
        if (k0 + BN > seq_k) valid = (1u << (seq_k - k0)) - 1u;
        if (MASK) {
            const unsigned long long b = __ballot(lane < BN && (k0 + lane < seq_k) && key_mask[min(k0 + lane, seq_k - 1)] != 0);
            valid &= (unsigned)b;
        }
#pragma unroll
        for (int ob = 0; ob < OWN; ob++) {
            const int kin = 8 * (OWN * sl + ob) + 4 * hh;                    /* first of the lane's four keys, inside the tile */
            if (valid != ~0u) {
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (!((valid >> (kin + r)) & 1u)) mine[ob][r] = -INFINITY;
            }
            if (CAUSAL && k0 + BN - 1 > wq0) {
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (k0 + kin + r > qrow) mine[ob][r] = -INFINITY;
            }
        }
        float mx = -INFINITY;
#pragma unroll
        for (int ob = 0; ob < OWN; ob++) mx = fmaxf(mx, fmaxf(fmaxf(mine[ob][0], mine[ob][1]), fmaxf(mine[ob][2], mine[ob][3])));
        mx = half_swap_max(mx);
        if (hh == 0) x3[wave * 32 + col] = mx;
        lds_barrier();                                                       /* 2: maxima */
        float tile_max = x3[(grp * NS) * 32 + col];
#pragma unroll
        for (int p = 1; p < NS; p++) tile_max = fmaxf(tile_max, x3[(grp * NS + p) * 32 + col]);
        tile_max *= scale_log2;
        if (__any(tile_max > m_run + RESCALE_THRESHOLD)) {                   /* the same decision in every wave of the group */
            const float m_new = fmaxf(m_run, tile_max);
            const float alpha = __builtin_amdgcn_exp2f(m_run - (m_new == -INFINITY ? 0.0f : m_new));
            m_run = m_new;
            l_run *= alpha;
#pragma unroll
            for (int db = 0; db < 4; db++)
#pragma unroll
                for (int r = 0; r < 16; r++) o[db][r] *= alpha;
        }
        const float neg_m = m_run == -INFINITY ? 0.0f : -m_run;
#pragma unroll
        for (int ob = 0; ob < OWN; ob++) {
            const float p0 = __builtin_amdgcn_exp2f(fmaf(mine[ob][0], scale_log2, neg_m));
            const float p1 = __builtin_amdgcn_exp2f(fmaf(mine[ob][1], scale_log2, neg_m));
            const float p2 = __builtin_amdgcn_exp2f(fmaf(mine[ob][2], scale_log2, neg_m));
            const float p3 = __builtin_amdgcn_exp2f(fmaf(mine[ob][3], scale_log2, neg_m));
            l_run += (p0 + p1) + (p2 + p3);
            /* P^T in the layout of the B operand, [k-step t of 16 keys][hh][query][8]: the lane (query, hh) of the product
             * multiplies keys 16t + 4hh + 0..3 and 16t + 8 + 4hh + 0..3 (the rows its V^T operand brings), i.e. this
             * lane's four keys of block 2t or 2t + 1 */
            const int kb = OWN * sl + ob;
            *reinterpret_cast<uint2 *>(&x2[((((grp * 2) + (kb >> 1)) * 2 + hh) * 32 + col) * 8 + 4 * (kb & 1)]) =
                make_uint2(pack_bf16(p0, p1), pack_bf16(p2, p3));
        }
        lds_barrier();                                                       /* 3: probabilities; V of this tile, K of the next */

        /* ---- C: O[:, slice]^T += V[:, slice]^T P^T ---- */
        {
            bf16x8 pb[2];
#pragma unroll
            for (int t = 0; t < 2; t++)
                pb[t] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4 *>(&x2[((((grp * 2) + t) * 2 + hh) * 32 + col) * 8]));
            s16x4 lo[2][4], hi[2][4];
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int db = 0; db < 4; db++) {
                    lo[t][db] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(&vcur[v_rd[0][db] + 16 * t * HD]));
                    hi[t][db] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(&vcur[v_rd[1][db] + 16 * t * HD]));
                }
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int db = 0; db < 4; db++) {
                    s16x8 both = __builtin_shufflevector(lo[t][db], hi[t][db], 0, 1, 2, 3, 4, 5, 6, 7);
                    o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, both), pb[t], o[db], 0, 0, 0);
                }
        }
    }
    /* ---- the row sums of the NS waves of a group, then normalise and store this wave's 128 dims:
     * lane holds dims 32db + 8g + 4hh + {0..3} ---- */
    lds_barrier();
    const float l_wave = half_swap_sum(l_run);
    if (hh == 0) x3[wave * 32 + col] = l_wave;
    lds_barrier();
    float l_tot = x3[(grp * NS) * 32 + col];
#pragma unroll
    for (int p = 1; p < NS; p++) l_tot += x3[(grp * NS + p) * 32 + col];
    const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
    if (qrow < seq_q) {
        uint16_t *op = out + (size_t)qrow * ldo + (size_t)head * HD + 128 * sl + 4 * hh;
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

template <int NS, bool C, bool M>
int launch(hipStream_t st, uint16_t *out, int ldo, const uint16_t *q, const uint16_t *k,
           const uint16_t *v, int ldi, int seq_q, int seq_k, int heads, int kv_heads, float scale,
           const int *key_mask) {
    constexpr int HD = 128 * NS, BM = 32 * (8 / NS);
    /* two K and two V stages, partial scores (8 waves x 3 or 4 blocks x 1 KB), P^T, maxima */
    constexpr size_t LDS_BYTES = (size_t)4 * BN * HD * sizeof(uint16_t) + (size_t)8 * (NS == 4 ? 3 : 4) * 64 * sizeof(f32x4) +
                                 (size_t)(8 / NS) * 4 * 32 * 8 * sizeof(uint16_t) + 8 * 32 * sizeof(float);
    static bool configured = false;
    if (!configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(k_fa_fwd_sliced<NS, C, M>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_BYTES);
        if (e != hipSuccess) return (int)e;
        configured = true;
    }
    const int q_tiles = (seq_q + BM - 1) / BM;
    const int total = q_tiles * heads;
    const int per_xcd = (total + XCDS - 1) / XCDS;
    hipLaunchKernelGGL((k_fa_fwd_sliced<NS, C, M>), dim3(per_xcd * XCDS), dim3(THREADS), LDS_BYTES, st, out, ldo,
                       q, k, v, ldi, seq_q, seq_k, q_tiles, total, per_xcd, heads / kv_heads,
                       scale * 1.4426950408889634f, key_mask);
    return (int)hipGetLastError();
}

template <int NS>
int launch_ns(hipStream_t st, uint16_t *out, int ldo, const uint16_t *q, const uint16_t *k,
              const uint16_t *v, int ldi, int seq_q, int seq_k, int heads, int kv_heads, float scale,
              int causal, const int *key_mask) {
    if (causal) {
        if (key_mask) return launch<NS, true, true>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, key_mask);
        return launch<NS, true, false>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, key_mask);
    }
    if (key_mask) return launch<NS, false, true>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, key_mask);
    return launch<NS, false, false>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, key_mask);
}

}  // namespace

extern "C" int iris_hip_fa_sliced(void *stream, uint16_t *out, int ldo, const uint16_t *q,
                                  const uint16_t *k, const uint16_t *v, int ldi, int seq_q,
                                  int seq_k, int heads, int kv_heads, int head_dim, float scale,
                                  int causal, const int *key_mask) {
    hipStream_t st = (hipStream_t)stream;
    if (head_dim == 512)
        return launch_ns<4>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, causal, key_mask);
    if (head_dim == 256)
        return launch_ns<2>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, causal, key_mask);
    return (int)hipErrorInvalidValue;
}
