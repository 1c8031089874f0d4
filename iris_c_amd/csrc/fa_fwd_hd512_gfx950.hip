/*
 * Flash-attention forward for gfx950, head_dim 512: the VAE mid-block
 * attention of the reference (one head of 512 over every latent position,
 * iris_vae.c:1112-1124; operator contract iris_dev.h:83-92, whose key mask
 * and causal limit are template options here). bf16 in, f32 accumulation on
 * the matrix cores (v_mfma_f32_16x16x32_bf16).
 *
 * One wave per SIMD, each with the whole register file: a wave owns 32 queries
 * and all 512 output dims of them, O^T as 64 accumulator blocks of 16 dims x 16
 * queries = 256 registers that live in AGPRs (the products that update them are
 * asm statements, so that they stay there), Q^T as 32 B operands = 128 VGPRs.
 * No wave ever needs another wave's partial scores: the only thing the four
 * waves of a workgroup (128 queries) share is the K and V tiles in the LDS.
 * Both products are transposed as in the head_dim-128 kernel, S^T = K Q^T and
 * O^T += V^T P^T, so a query is a column of every accumulator, its running
 * max, bound and rescale factor are per-lane scalars, and exp2(S^T) rounded to
 * bf16 is the B operand of the second product without leaving the registers.
 * The row sum comes from one more product per tile with an all-ones A operand.
 *
 * Tiles of 32 keys: a K or V tile is 32 KB, three K stages and two V stages are
 * all 160 KB of the LDS, filled by global_load_lds_dwordx4 (a wave has no
 * registers to stage them through): one instruction moves one 1 KB tile row,
 * each wave 8 rows of K and 8 of V per tile. The loop is skewed: turn t
 * multiplies the scores of tile t + 1, then the values of tile t, then takes
 * the softmax of tile t + 1. V of tile t + 1 is requested during the score
 * products and K of tile t + 3 during the value products, one row every
 * eighth product: the CU's one load path runs half busy all the time instead
 * of saturated for a part of the turn (a request then holds the wave about 20
 * cycles, not 100), and every request has at least half a turn to land before
 * the turn's one barrier. Rows are unpadded; the 16 B chunk c of row r sits in
 * slot c ^ 2 (r % 8) of its 256 B group, the permutation applied to the source
 * address of the lane that fills the slot (same conflict-free pattern as the
 * head_dim-128 kernel: a row is a multiple of 256 B there and here).
 *
 * What a wave that is alone on its SIMD overlaps with its own products, as
 * measured here on timing-only variants (16384 tokens, 415 us): memory
 * instructions, one per gap between two products (operand reads bunched at
 * the head of a group of four products: +2 %); vector ALU work not at all (the
 * softmax costs 58 us whether it stands in one block, as it does, or is dealt
 * out into the gaps between the score products of the next tile). Without
 * softmax, requests, operand reads and barrier the products alone run at 1.8
 * PFLOP/s, the power limit of the chip for this instruction.
 *
 * 128 queries per workgroup make few workgroups (16384 tokens: 128 for 256
 * CUs), so the keys of a head may be cut into `splits` ranges, one workgroup
 * per (query tile, range); these write their unnormalised O (f32), running max
 * and row sum to a scratch buffer and k_fa_hd512_merge combines them.
 *
 * A key mask arrives as one word per key tile (k_pack_key_mask, a launch in
 * front); the walk over the keys ends at the last tile that has a valid key.
 * A causal call walks the tiles in front of each workgroup's last query; its
 * workgroups differ in length and are numbered by falling length.
 *
 * head_dim 256 is the same kernel with half the k-steps, dim blocks and tile
 * rows (template parameter HD); the description above gives the numbers of 512.
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
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int BN = 32;              /* keys per tile */
constexpr int BM = 128;             /* queries per workgroup */
constexpr int THREADS = 256;
constexpr int XCDS = 8;
/* three K stages, two V stages of 32 keys x HD: all 160 KB at head_dim 512 */
constexpr size_t lds_bytes(int hd) { return 5 * (size_t)BN * hd * sizeof(uint16_t); }
constexpr float RESCALE_THRESHOLD = 8.0f;   /* log2 units */

/* Every lambda below is inlined by the always-inline pass, before anything else runs: a closure that is only
 * inlined later keeps what it captured (the accumulators) in memory. */
#define INLINE __attribute__((always_inline))

__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    f32x2 p = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(p, bf16x2));
}
__device__ __forceinline__ float max3(float a, float b, float c) {
    return __builtin_elementwise_maximum(__builtin_elementwise_maximum(a, b), c);
}
/* max over the four lanes l%16, +16, +32, +48, which share a query */
__device__ __forceinline__ float quad_group_max(float v) {
    auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    const float t = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(t), __float_as_uint(t), false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ int swz(int row) { return 2 * (row & 7); }
__device__ __forceinline__ uint32_t lds_address(const uint16_t *p) {
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void *)p;
}
__device__ __forceinline__ const uint16_t *scalar_ptr(const uint16_t *p) {
    const uint64_t v = (uint64_t)(uintptr_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (const uint16_t *)(uintptr_t)(((uint64_t)hi << 32) | lo);
}

/* Where the partial results of a key range live: [range][head][query] rows of HD f32, and (max, sum) pairs. */
struct Partials {
    float *o, *ml;
};

#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"

/* The workgroups of a causal call in the order of falling length. With `step` = tiles_per_split / 4 query tiles per key
 * range, the pair (query tile qt, range r) walks min(4 (qt + 1) - r * tiles_per_split, tiles_per_split) tiles, which
 * depends on qt - r * step only; pairs with qt - r * step < 0 have none and get no number. Number j -> how far the
 * pair's qt - r * step lies behind the last query tile, and r: at distance u the ranges 0 .. min(u / step, splits - 1)
 * exist. */
__host__ __device__ inline void causal_pair(int j, int step, int splits, int &behind, int &r) {
    if (step == 0) { behind = j / splits; r = j % splits; return; }
    int k = 0, first = 0;                            /* first: the number of the first pair with u / step == k */
    while (k < splits - 1 && j >= first + step * (k + 1)) { first += step * (k + 1); k++; }
    behind = k * step + (j - first) / (k + 1);
    r = (j - first) % (k + 1);
}
__host__ inline int causal_pairs(int q_tiles, int step, int splits) {
    if (step == 0) return q_tiles * splits;
    int n = 0;
    for (int u = 0; u < q_tiles; u++) n += u / step + 1 < splits ? u / step + 1 : splits;
    return n;
}

/* HD: 512, or 256 (the same kernel with half the k-steps, dim blocks and tile rows: a tile row is then half of what one
 * load instruction moves, and a wave's eight rows of a tile are four instructions of two rows). SPLIT: one of several
 * key ranges (partial results to `part`). CAUSAL: query i ignores keys j > i; a workgroup walks
 * the tiles of its range up to its last query, and the workgroups are numbered by falling length. MASK:
 * `mask_words[t]` holds the valid keys of key tile t as k_pack_key_mask left them. */
template <int HD, bool SPLIT, bool CAUSAL, bool MASK>
__global__ void __launch_bounds__(THREADS, 1)
k_fa_fwd_hd512(uint16_t *__restrict__ out, int ldo, const uint16_t *__restrict__ q,
               const uint16_t *__restrict__ k, const uint16_t *__restrict__ v, int ldi,
               int seq_q, int seq_k, int heads, int q_tiles, int splits, int tiles_per_split,
               int total_work, int work_per_xcd, int kv_group, float scale_log2, Partials part,
               const uint32_t *__restrict__ mask_words) {
    static_assert(HD == 512 || HD == 256, "rows of one or half a load instruction");
    constexpr int TILE = BN * HD;                       /* elements of a K (or V) tile */
    constexpr int KS = HD / 32, DB = HD / 16;           /* k-steps of the score products, dim blocks of the output */
    constexpr int RPI = 512 / HD, NR = 8 / RPI;         /* tile rows per load instruction; instructions per wave and tile */
    extern __shared__ __align__(16) uint16_t lds[];     /* K stages 0, 1, 2 | V stages 0, 1 */

    int qt, split, head;
    if (CAUSAL) {
        /* Workgroups differ in length: query tile qt has 4 (qt + 1) key tiles in front of it, of which range r holds
         * those from r * tiles_per_split on. The hardware deals workgroup b to XCD b % 8 and every XCD starts its own
         * in order, so they are numbered by falling length (causal_pair), heads innermost: neighbours are equally
         * long, which also gives every XCD the same mix. Only pairs that have a key tile get a number. An XCD has been
         * seen to hand its workgroups to its four shader engines in turn and to wait with the next one until the
         * engine whose turn it is has a free CU, so every other group of 32 (8 XCDs x 4 engines) runs backwards: the
         * engine that got the shortest of one group, and is free first, gets the longest of the next. (256 CUs hold
         * eight groups at a time, so it is an odd group that meets an even one there.) */
        const int slot = (blockIdx.x & 32) ? (blockIdx.x & ~31) | (31 - (blockIdx.x & 31)) : blockIdx.x;
        if (slot >= total_work) return;
        int behind;
        causal_pair(slot / heads, tiles_per_split / 4, splits, behind, split);
        head = slot % heads;
        qt = q_tiles - 1 - behind + split * (tiles_per_split / 4);
    } else {
        const int work = (blockIdx.x % XCDS) * work_per_xcd + blockIdx.x / XCDS;
        if (work >= total_work) return;
        const int rest = work / q_tiles;
        qt = work % q_tiles;
        split = rest % splits;
        head = rest / splits;
    }
    const int kvh = head / kv_group;

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lg = lane >> 4;       /* 16x16 block: column li, row group lg */
    const int wq0 = qt * BM + 32 * wave, qrow0 = wq0 + li;

    const uint16_t *kbase = scalar_ptr(k + (size_t)kvh * HD);
    const uint16_t *vbase = scalar_ptr(v + (size_t)kvh * HD);
    int t_begin = split * tiles_per_split;
    /* tiles of this workgroup's range: >= 1 when not causal (the launcher makes no empty range) */
    const int k_end = CAUSAL ? min(seq_k, qt * BM + BM) : seq_k;
    int nt = min((k_end + BN - 1) / BN - t_begin, tiles_per_split);
    if (SPLIT && CAUSAL && nt <= 0) return;          /* the range begins behind the last query: the merge skips it too */
    if (MASK) {
        /* A padding mask: the walk ends with the last tile of the sequence that has a valid key. Every workgroup finds
         * it by itself (at most seven words per thread); a call that is not causal then cuts the tiles up to there
         * into its ranges instead of all tiles, so that the ranges stay equally long. */
        int last = 0;
        for (int i = threadIdx.x; i < (seq_k + BN - 1) / BN; i += THREADS)
            if (mask_words[i]) last = i;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) last = max(last, __shfl_xor(last, off));
        int *share = reinterpret_cast<int *>(lds);
        if ((threadIdx.x & 63) == 0) share[threadIdx.x >> 6] = last;
        lds_barrier();
        last = max(max(share[0], share[1]), max(share[2], share[3]));
        lds_barrier();                               /* before the first tile lands on these words */
        last = __builtin_amdgcn_readfirstlane(last);
        if (CAUSAL) {
            nt = min(nt, last + 1 - t_begin);
        } else {
            const int per = (last + splits) / splits;
            t_begin = split * per;
            nt = min(last + 1 - t_begin, per);
        }
        if (SPLIT && nt <= 0) {                      /* nothing valid in this range: (max, sum) = (-inf, 0), which the merge skips */
            const int row = qt * BM + threadIdx.x;
            if (threadIdx.x < BM && row < seq_q)
                *reinterpret_cast<f32x2 *>(part.ml + 2 * (((size_t)split * heads + head) * seq_q + row)) = f32x2{-INFINITY, 0.0f};
            return;
        }
    }

    /* LDS: K stages 0, 1, 2 | V stages 0, 1 (TILE elements each). Read offsets in elements from the start of the LDS.
     * K operand (key block mb, k-step ks): row 16 mb + li, chunk 4 ks + lg = 16 (ks / 4) + (4 (ks % 4) + lg); the
     * swizzle touches the low four bits of the chunk only, so four registers and immediate offsets do; they run from
     * K stage to K stage with the tiles.
     * V^T operand (dim block db of 16): transposing read of a 4-key x 16-dim block per 16-lane group, row 4 lg + li / 4
     * (+ 16 for the second half of the keys), chunk 2 db + (li % 4) / 2 = 16 (db / 8) + (2 (db % 8) + ..). */
    int k_cur[4], v_rd[8];
#pragma unroll
    for (int i = 0; i < 4; i++) k_cur[i] = li * HD + 8 * ((4 * i + lg) ^ swz(li));
    {
        const int vrow = 4 * lg + (li >> 2);
#pragma unroll
        for (int i = 0; i < 8; i++)
            v_rd[i] = 3 * TILE + vrow * HD + 8 * ((2 * i + ((li & 3) >> 1)) ^ swz(vrow)) + 4 * (li & 1);
    }

    /* 1 KB per instruction, one tile row at head_dim 512: lane i fills slot i of row r = 8 wave + j of the stage, i.e.
     * fetches chunk i ^ swz(r) = i ^ 2 j of global row r (two rows at head_dim 256: lanes 0-31 row 8 wave + 2 j, lanes
     * 32-63 the next, 32 slots each). A wave's rows of a tile differ in the per-lane offset only (row j: j row
     * strides further), kept in NR registers, so that a request is three instructions: M0, a wait state, the load,
     * with one scalar source pointer per tile. A tile never reaches past the last key: the last tile of a
     * sequence whose length is not a multiple of 32 is moved back to end with it, and the keys it then shares
     * with the tile before are masked there; a sequence of fewer than 32 keys is one tile padded with its last key. Tiles past the end of the range repeat its last tile.
     * `stage` counts TILEs from the start of the LDS. */
    uint32_t lane_off[NR];
#pragma unroll
    for (int j = 0; j < NR; j++) {
        const uint32_t row = (uint32_t)(RPI * j + (RPI == 2 ? lane >> 5 : 0)), slot = (uint32_t)(lane & (64 / RPI - 1));
        /* a sequence of fewer than 32 keys is one tile whose last rows repeat its last key (they are masked) */
        const uint32_t in_tile = min(8u * (uint32_t)wave + row, (uint32_t)min(seq_k, BN) - 1u);
        lane_off[j] = 16u * (slot ^ (2u * (row & 7u))) + in_tile * (uint32_t)ldi * 2u;
    }
    const uint32_t lds0 = __builtin_amdgcn_readfirstlane(lds_address(lds)) + (uint32_t)(8 * wave * HD * 2);
    auto tile_rows = [&](const uint16_t *base, int tile) INLINE {          /* the first row of a tile of the range */
        const int k0 = max(min((t_begin + min(tile, nt - 1)) * BN, seq_k - BN), 0);
        return base + (size_t)k0 * ldi;
    };
    auto request_row = [&](const uint16_t *rows, int stage, int j) INLINE {
        const uint32_t dst = lds0 + (uint32_t)(stage * TILE * 2);
        asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3"
                     ::"s"(dst), "n"(j * 1024), "v"(lane_off[j]), "s"(rows) : "memory", "m0", "scc");
    };

    f32x4 o[DB][2];                                  /* O^T: dims 16 db + 4 lg + r of query block nb */
    float m_run[2], neg_m[2], bound[2];
    f32x4 l_acc[2];
#pragma unroll
    for (int nb = 0; nb < 2; nb++) {
#pragma unroll
        for (int db = 0; db < DB; db++) {
            o[db][nb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            asm volatile("" : "+a"(o[db][nb]));
        }
        m_run[nb] = -INFINITY; neg_m[nb] = 0.0f; bound[nb] = -INFINITY;
        l_acc[nb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    const float inv_scale_log2 = 1.0f / scale_log2;
    /* The all-ones A operand of the row-sum product stays in four registers for the whole kernel (the empty asm hides
     * the constant from the compiler): written afresh in front of the product, a move would be followed at once by
     * an asm statement that reads its result, and the compiler places the wait states a matrix instruction needs
     * behind an ordinary one only for matrix instructions it issues itself. */
    u32x4 ones = {0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};
    asm volatile("" : "+v"(ones));

    /* ---- prologue: K of tiles 0, 1, 2 and V of tile 0, then Q ---- */
    {
        const uint16_t *k0r = tile_rows(kbase, 0), *v0r = tile_rows(vbase, 0), *k1r = tile_rows(kbase, 1), *k2r = tile_rows(kbase, 2);
#pragma unroll
        for (int j = 0; j < NR; j++) request_row(k0r, 0, j);
#pragma unroll
        for (int j = 0; j < NR; j++) request_row(v0r, 3, j);
#pragma unroll
        for (int j = 0; j < NR; j++) request_row(k1r, 1, j);
#pragma unroll
        for (int j = 0; j < NR; j++) request_row(k2r, 2, j);
    }

    /* Q^T as B operands: for query block nb and k-step ks the lane holds dims 32 ks + 8 lg .. +7 of query 16 nb + li */
    bf16x8 qb[2][KS];
#pragma unroll
    for (int nb = 0; nb < 2; nb++) {
        const uint16_t *qp = q + (size_t)min(qrow0 + 16 * nb, seq_q - 1) * ldi + (size_t)head * HD + 8 * lg;
#pragma unroll
        for (int ks = 0; ks < KS; ks++)
            qb[nb][ks] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(qp + 32 * ks));
    }
    /* the tile requests are invisible to the compiler's wait-count bookkeeping: complete the loads it knows about
     * here, so that it places no wait for them inside the loop (which would wait for the newest tile requests) */
#pragma unroll
    for (int nb = 0; nb < 2; nb++)
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            u32x4 t = __builtin_bit_cast(u32x4, qb[nb][ks]);
            asm volatile("" : "+v"(t));
            qb[nb][ks] = __builtin_bit_cast(bf16x8, t);
        }
    wait_vmcnt<0>();
    lds_barrier();

    /* ---- S^T = K Q^T of one tile into s: 2 key blocks x 2 query blocks, 16 k-steps of 32 dims (the numbers in these
     * comments are those of head_dim 512; 256 has half the k-steps, dim blocks and requests). A wave that is
     * alone on its SIMD issues in order, and what it issues between two products runs while the matrix core works on
     * the first: one memory instruction per gap is free, more are not. So the two operand reads of k-step ks + KD
     * stand behind the first and the third product of k-step ks, and between(i) behind the i-th of the 64 products
     * is where the caller puts its tile requests. ---- */
    constexpr int KD = 2;
    f32x4 s[2][2];
    auto scores = [&](auto &&between) INLINE {
        u32x4 ka[KD + 1][2];
        auto read_k = [&](int ks, int mb) INLINE {
            ka[ks % (KD + 1)][mb] = *reinterpret_cast<const u32x4 *>(&lds[k_cur[ks & 3] + 128 * (ks >> 2) + 16 * mb * HD]);
        };
#pragma unroll
        for (int ks = 0; ks < KD; ks++) { read_k(ks, 0); read_k(ks, 1); }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
#pragma unroll
            for (int mb = 0; mb < 2; mb++)
#pragma unroll
                for (int nb = 0; nb < 2; nb++) {
                    if (ks == 0) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=&v"(s[mb][nb]) : "v"(ka[0][mb]), "v"(qb[nb][0]));
                    else asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(s[mb][nb]) : "v"(ka[ks % (KD + 1)][mb]), "v"(qb[nb][ks]));
                    if (nb == 0 && ks + KD < KS) read_k(ks + KD, mb);
                    between(4 * ks + 2 * mb + nb);
                    __builtin_amdgcn_sched_barrier(0);
                }
        }
    };

    /* ---- online softmax of the scores in s (tile `tile` of the range) -> P^T as B operands in pw. The lane holds 8
     * of the 32 scores of each of its two queries: keys 16 mb + 4 lg + r. The running max is only raised when some
     * score of the wave exceeds it by more than 2^8; that test needs no cross-lane traffic (the four lanes of a
     * query share the bound). ---- */
    u32x4 pw[2];
    auto softmax = [&](int tile, uint32_t mask_word) INLINE {
        const int k0 = (t_begin + tile) * BN;
        /* valid keys of the tile as a wave-uniform set: the last tile of the sequence is moved back by k0 + 32 - seq_k
         * keys, which belong to the tile before; with a key mask the packed word says all of this already */
        uint32_t valid = ~0u;
        if (k0 + BN > seq_k) valid = seq_k < BN ? ~0u >> (BN - seq_k) : ~0u << (k0 + BN - seq_k);
        if (MASK) valid = mask_word;
        if (valid != ~0u) {
            const unsigned mine = valid >> (4 * lg);
#pragma unroll
            for (int mb = 0; mb < 2; mb++)
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (!((mine >> (16 * mb + r)) & 1u)) {
#pragma unroll
                        for (int nb = 0; nb < 2; nb++) s[mb][nb][r] = -INFINITY;
                    }
        }
        if (CAUSAL) {
            const int first = max(min(k0, seq_k - BN), 0);      /* the key in row 0 of the tile as it was loaded */
            if (first + BN - 1 > wq0) {                          /* wave-uniform: some key lies behind the wave's first query */
                const int lim0 = qrow0 - first - 4 * lg;         /* key offset 16 mb + r is valid iff <= lim0 (+ 16 nb) */
#pragma unroll
                for (int mb = 0; mb < 2; mb++)
#pragma unroll
                    for (int r = 0; r < 4; r++)
#pragma unroll
                        for (int nb = 0; nb < 2; nb++)
                            if (16 * mb + r > lim0 + 16 * nb) s[mb][nb][r] = -INFINITY;
            }
        }
        float lane_max[2];
        bool raise = false;
#pragma unroll
        for (int nb = 0; nb < 2; nb++) {
            const float a = max3(s[0][nb][0], s[0][nb][1], s[0][nb][2]);
            const float b = max3(s[0][nb][3], s[1][nb][0], s[1][nb][1]);
            const float c = max3(s[1][nb][2], s[1][nb][3], a);
            lane_max[nb] = fmaxf(b, c);
            raise = raise || lane_max[nb] > bound[nb];
        }
        if (__any(raise)) {
            /* the accumulators are read by ordinary instructions here, right behind the products of the values: these
             * have to leave the matrix core first (volatile asm statements keep their order, and the empty ones
             * below make every read of an accumulator come after this one) */
            asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
            for (int nb = 0; nb < 2; nb++) {
                const float m_new = fmaxf(m_run[nb], quad_group_max(lane_max[nb]) * scale_log2);
                const float alpha = __builtin_amdgcn_exp2f(m_run[nb] - (m_new == -INFINITY ? 0.0f : m_new));
                m_run[nb] = m_new;
                neg_m[nb] = m_new == -INFINITY ? 0.0f : -m_new;
                bound[nb] = (m_new + RESCALE_THRESHOLD) * inv_scale_log2;
                asm volatile("" : "+v"(l_acc[nb]));
                l_acc[nb] *= alpha;
#pragma unroll
                for (int db = 0; db < DB; db++) {
                    asm volatile("" : "+a"(o[db][nb]));
                    f32x4 t = o[db][nb];
                    t *= alpha;
                    o[db][nb] = t;
                    asm volatile("" : "+a"(o[db][nb]));
                }
            }
        }
#pragma unroll
        for (int nb = 0; nb < 2; nb++) {
            float p[8];
#pragma unroll
            for (int r = 0; r < 4; r++) {
                p[r] = __builtin_amdgcn_exp2f(fmaf(s[0][nb][r], scale_log2, neg_m[nb]));
                p[4 + r] = __builtin_amdgcn_exp2f(fmaf(s[1][nb][r], scale_log2, neg_m[nb]));
            }
            pw[nb] = u32x4{pack_bf16(p[0], p[1]), pack_bf16(p[2], p[3]), pack_bf16(p[4], p[5]), pack_bf16(p[6], p[7])};
        }
    };

    /* ---- O^T += V^T P^T of one tile: one k-step of 32 keys x 32 dim blocks x 2 query blocks, in 16 groups of two
     * dim blocks = four products; the four transposing reads of group g + VD stand one behind each product of
     * group g, between(i) behind the i-th of the 64 products ---- */
    constexpr int VD = 2;
    auto values = [&](int vstage, auto &&between) INLINE {
        const uint16_t *vst = lds + vstage * TILE;            /* v_rd already points into V stage 0 */
        s16x4 lo[VD + 1][2], hi[VD + 1][2];
        auto read_v = [&](int g, int r) INLINE {                /* r: dim block 2 g + r / 2, keys 0-15 or 16-31 of the tile */
            const int db = 2 * g + (r >> 1);
            const uint16_t *vp = &vst[v_rd[db & 7] + 128 * (db >> 3)];
            if (r & 1) hi[g % (VD + 1)][r >> 1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(vp + 16 * HD));
            else lo[g % (VD + 1)][r >> 1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(vp));
        };
#pragma unroll
        for (int g = 0; g < VD; g++)
#pragma unroll
            for (int r = 0; r < 4; r++) read_v(g, r);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int nb = 0; nb < 2; nb++)
            asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(l_acc[nb]) : "v"(ones), "v"(pw[nb]));
#pragma unroll
        for (int g = 0; g < DB / 2; g++) {
#pragma unroll
            for (int d = 0; d < 2; d++) {
                const s16x8 both = __builtin_shufflevector(lo[g % (VD + 1)][d], hi[g % (VD + 1)][d], 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
                for (int nb = 0; nb < 2; nb++) {
                    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(o[2 * g + d][nb]) : "v"(both), "v"(pw[nb]));
                    if (g + VD < DB / 2) read_v(g + VD, 2 * d + nb);
                    between(4 * g + 2 * d + nb);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    };

    /* The scores run one tile ahead of the values: those of tile 0 here. The products are asm statements, which the
     * compiler's hazard bookkeeping does not see: a product's result must have left the matrix core before other
     * instructions read it. In the loop the products of the values stand between the last score product of a tile
     * and the softmax that reads its scores; here idle cycles do. */
    scores([](int) INLINE {});
    asm volatile("s_nop 15\n\ts_nop 15" : "+v"(s[0][0]), "+v"(s[0][1]), "+v"(s[1][0]), "+v"(s[1][1]));
    /* The words of the key mask are read through the scalar cache two turns at a time and waited for on the spot (the
     * empty asm consumes them): a scalar load left pending would turn every wait for an LDS operand into a wait for
     * everything. */
    auto mask_word = [&](int tile) INLINE {
        uint32_t w = 0;
        if (MASK) {
            w = mask_words[t_begin + min(tile, nt - 1)];
            asm volatile("" : "+s"(w));
        }
        return w;
    };
    softmax(0, mask_word(0));
    lds_barrier();                                   /* K stage 0 has no readers any more */
    int kstage = 1;                                  /* where the K operand offsets point: the stage of tile t + 1 */
#pragma unroll
    for (int i = 0; i < 4; i++) k_cur[i] += TILE;

    /* Turn t (par = t % 2): score products of tile t + 1 (K stage (t + 1) % 3), value products of tile t (V stage par,
     * probabilities from the turn before), softmax of tile t + 1. V of tile t + 1 -> V stage par ^ 1 is requested
     * during the score products (its last readers were the value products of turn t - 1), K of tile t + 3 -> K stage
     * t % 3 during the value products (last read by the score products of turn t - 1), one row every eighth
     * product, so that the four waves keep the CU's one load path half busy all the time instead of saturating it
     * for a part of the turn. At the end of the turn everything but the eight newest requests (K of tile t + 3) must
     * have landed. */
    auto turn = [&](int t, int par, uint32_t next_mask_word) INLINE {
        const uint16_t *vrows = tile_rows(vbase, t + 1), *krows = tile_rows(kbase, t + 3);
        scores([&](int i) INLINE {
            if ((i & 7) == 5) request_row(vrows, 3 + (par ^ 1), i >> 3);
        });
        const int kreq = kstage == 0 ? 2 : kstage - 1;       /* t % 3 */
        values(par, [&](int i) INLINE {
            if ((i & 7) == 5) request_row(krows, kreq, i >> 3);
        });
        if (t + 1 < nt) softmax(t + 1, next_mask_word);
        const int step = kstage == 2 ? -2 * TILE : TILE;
        kstage = kstage == 2 ? 0 : kstage + 1;
#pragma unroll
        for (int i = 0; i < 4; i++) k_cur[i] += step;
        wait_vmcnt<NR>();
        lds_barrier();
    };
    for (int t = 0; t < nt; t += 2) {
        const uint32_t w1 = mask_word(t + 1), w2 = mask_word(t + 2);
        turn(t, 0, w1);
        if (t + 1 < nt) turn(t + 1, 1, w2);
    }
    wait_vmcnt<0>();                                  /* nothing may still be on its way into the LDS when it is given back */
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");      /* the last products have left the matrix core */
#pragma unroll
    for (int nb = 0; nb < 2; nb++) {
#pragma unroll
        for (int db = 0; db < DB; db++) asm volatile("" : "+a"(o[db][nb]));
        asm volatile("" : "+v"(l_acc[nb]));
    }

    /* ---- the lane holds dims 16 db + 4 lg + {0..3} of its two queries ---- */
#pragma unroll
    for (int nb = 0; nb < 2; nb++) {
        const float l_tot = l_acc[nb][0];              /* every row of the ones product is the full sum */
        const int qrow = qrow0 + 16 * nb;
        if (qrow >= seq_q) continue;
        if (SPLIT) {
            const size_t prow = ((size_t)split * heads + head) * seq_q + qrow;
            float *po = part.o + prow * HD + 4 * lg;
#pragma unroll
            for (int db = 0; db < DB; db++) *reinterpret_cast<f32x4 *>(po + 16 * db) = o[db][nb];
            if (lg == 0) *reinterpret_cast<f32x2 *>(part.ml + 2 * prow) = f32x2{m_run[nb], l_tot};
        } else {
            const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
            uint16_t *op = out + (size_t)qrow * ldo + (size_t)head * HD + 4 * lg;
#pragma unroll
            for (int db = 0; db < DB; db++) {
                uint2 w;
                w.x = pack_bf16(o[db][nb][0] * inv, o[db][nb][1] * inv);
                w.y = pack_bf16(o[db][nb][2] * inv, o[db][nb][3] * inv);
                *reinterpret_cast<uint2 *>(op + 16 * db) = w;
            }
        }
    }
}

#pragma clang diagnostic pop

/* The key mask as one 32-bit word per key tile, bit j = key j of the tile AS THE KERNEL LOADS IT is valid: the last
 * tile of a sequence whose length is not a multiple of 32 is moved back to end with it, and the keys it shares with
 * the tile before count as invalid there. 256 threads = eight tiles per block, two per wave; `words` has room for a
 * multiple of eight. */
__global__ void __launch_bounds__(256)
k_pack_key_mask(uint32_t *__restrict__ words, const int *__restrict__ key_mask, int seq_k, int tiles) {
    const int pair = 4 * blockIdx.x + (threadIdx.x >> 6);           /* tiles 2 pair, 2 pair + 1: one wave */
    const int tile = 2 * pair + ((threadIdx.x >> 5) & 1), j = threadIdx.x & 31;
    const int first = max(min(tile * BN, seq_k - BN), 0), key = first + j;
    const bool ok = tile < tiles && key >= tile * BN && key < seq_k && key_mask[key] != 0;
    const unsigned long long both = __ballot(ok);
    if ((threadIdx.x & 63) == 0) {
        words[2 * pair] = (uint32_t)both;
        words[2 * pair + 1] = (uint32_t)(both >> 32);
    }
}

/* Combines the key ranges of a query: out = sum_r 2^(m_r - m) o_r / sum_r 2^(m_r - m) l_r with m the largest of the
 * maxima. 64 threads per query row, HD / 64 dims each. */
template <int HD>
__global__ void __launch_bounds__(256)
k_fa_hd512_merge(uint16_t *__restrict__ out, int ldo, Partials part, int seq_q, int heads, int splits, int causal_keys,
                 int tiles_per_split) {
    const size_t rows = (size_t)heads * seq_q;
    const size_t row = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);       /* head * seq_q + query */
    if (row >= rows) return;
    const int t = threadIdx.x & 63;
    const size_t head = row / seq_q, qrow = row - head * seq_q;
    if (causal_keys) {                                /* a causal call of causal_keys keys: ranges behind the query's workgroup were never written */
        const int keys = min(causal_keys, ((int)qrow / BM + 1) * BM);
        splits = min(splits, ((keys + BN - 1) / BN + tiles_per_split - 1) / tiles_per_split);
    }
    float m = -INFINITY;
    for (int r = 0; r < splits; r++) m = fmaxf(m, part.ml[2 * (r * rows + row)]);
    constexpr int PER = HD / 64;                      /* 8 or 4 */
    float l = 0.0f, acc[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    for (int r = 0; r < splits; r++) {
        const f32x2 ml = *reinterpret_cast<const f32x2 *>(part.ml + 2 * (r * rows + row));
        if (ml[0] == -INFINITY) continue;             /* no valid key in this range */
        const float w = __builtin_amdgcn_exp2f(ml[0] - m);
        l += w * ml[1];
        const float *po = part.o + (r * rows + row) * HD + PER * t;
        const f32x4 a = *reinterpret_cast<const f32x4 *>(po);
#pragma unroll
        for (int i = 0; i < 4; i++) acc[i] += w * a[i];
        if (PER == 8) {
            const f32x4 b = *reinterpret_cast<const f32x4 *>(po + 4);
#pragma unroll
            for (int i = 0; i < 4; i++) acc[4 + i] += w * b[i];
        }
    }
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;
    uint16_t *op = out + qrow * ldo + head * HD + PER * t;                /* output rows are 8-byte aligned, not more */
    *reinterpret_cast<uint2 *>(op) = make_uint2(pack_bf16(acc[0] * inv, acc[1] * inv), pack_bf16(acc[2] * inv, acc[3] * inv));
    if (PER == 8)
        *reinterpret_cast<uint2 *>(op + 4) = make_uint2(pack_bf16(acc[4] * inv, acc[5] * inv), pack_bf16(acc[6] * inv, acc[7] * inv));
}

int cu_count() {
    static int n = 0;
    if (n == 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount >= 8)
            n = prop.multiProcessorCount;
        else {
            (void)hipGetLastError();
            n = 256;
        }
    }
    return n;
}

}  // namespace

/* How many key ranges a call is cut into, and the scratch it then needs (partial rows for more than one range, the
 * packed key mask for a masked call; 0 for neither). Host arithmetic only.
 * Fitted at head_dim 512 to every number of ranges at 256 .. 50176 tokens: a turn of 32 keys takes a workgroup 1.6 us
 * when all CUs are busy and 1.3 us when few are (the clock follows the load), a round of workgroups costs its turns
 * plus about 8 us of start and end, and the merge reads and writes the partial rows at about 6 TB/s (they are still
 * in the caches) behind a launch of 4 us and half a microsecond per range. The choice is within 3 % of the best
 * count from 9216 tokens on and within 6 % below (where every count from 4 to 8 is within 10 % of every other).
 * A causal call has workgroups of 4, 8, 12, ... tiles: it takes the longer of its longest workgroup and of all its
 * turns spread over the CUs, and ranges shorten the former; ranges that begin behind a workgroup's last query do
 * not exist, in the kernel and in the merge. Fitted to 1 .. 8 ranges at 1024 .. 30000 tokens: the choice costs 1 %
 * on average against the best count. At head_dim 256 a turn has half the products and costs TURN_256 of the above. */
namespace {
constexpr double TURN_256 = 0.6;
size_t plan_ranges(int hd, int seq_q, int seq_k, int heads, int causal, int masked, int *splits_out) {
    const long cus = cu_count();
    const long tiles = (seq_k + BN - 1) / BN, q_tiles = (seq_q + BM - 1) / BM, wgs = q_tiles * heads;
    const double rows_mb = (double)seq_q * heads * hd * 4 / 1e6;          /* one range's partial O, MB */
    const double turn = hd == 512 ? 1.0 : TURN_256;
    double best = 0.0;
    int best_s = 1;
    for (int s = 1; s <= 8 && s <= tiles; s++) {
        const long per = (tiles + s - 1) / s, ranges = (tiles + per - 1) / per;
        if (ranges != s) continue;
        double us;
        if (causal) {
            long turns = 0, filled = 0;              /* over the query tiles of a head: tiles walked, ranges that are not empty */
            for (long qt = 0; qt < q_tiles; qt++) {
                const long keys = qt * BM + BM < seq_k ? qt * BM + BM : seq_k, mine = (keys + BN - 1) / BN;
                turns += mine;
                filled += (mine + per - 1) / per;
            }
            /* in turns: the longest workgroup when all run at once, else all turns spread over the CUs plus a ragged
             * end; a turn costs 1.2 us on an empty machine and 1.7 us on a full one */
            const double longest = (double)(per < tiles ? per : tiles), spread = (double)turns * heads / cus + 0.2 * longest;
            const double span = filled * heads <= cus || longest > spread ? longest : spread;
            us = span * turn * (1.2 + 0.5 * (double)turns * heads / (cus * span)) + 10.0 * (double)((filled * heads + cus - 1) / cus);
            if (ranges > 1) us += 4.0 + 0.5 * ranges + 2.0 * (double)filled * heads * (BM * hd * 4 / 1e6) / 6.0;
        } else {
            const long full = wgs * ranges / cus, rest = wgs * ranges % cus;
            us = full * (per * turn * 1.6 + 8.0);
            if (rest) us += per * turn * (1.3 + 0.3 * (double)rest / cus) + 8.0;
            if (ranges > 1) us += 4.0 + 0.5 * ranges + 2.0 * ranges * rows_mb / 6.0;          /* MB / (TB/s) = us */
        }
        if (s == 1 || us < best * 0.97) { best = us; best_s = s; }
    }
    *splits_out = best_s;
    const size_t rows = best_s == 1 ? 0 : (size_t)seq_q * heads * best_s;
    const size_t words = masked ? ((size_t)tiles + 7) / 8 * 8 : 0;
    return rows * hd * sizeof(float) + rows * 2 * sizeof(float) + words * sizeof(uint32_t);
}
}  // namespace

extern "C" size_t iris_hip_fa_hd512_plan(int seq_q, int seq_k, int heads, int causal, int masked, int *splits_out) {
    return plan_ranges(512, seq_q, seq_k, heads, causal, masked, splits_out);
}
extern "C" size_t iris_hip_fa_hd256_plan(int seq_q, int seq_k, int heads, int causal, int masked, int *splits_out) {
    return plan_ranges(256, seq_q, seq_k, heads, causal, masked, splits_out);
}

/* The numbering of a causal call's workgroups, for inspection on the host: pair `number` of a call with q_tiles query
 * tiles and ranges of tiles_per_split key tiles -> its query tile and range; returns how many pairs there are. */
extern "C" int iris_hip_fa_hd512_causal_order(int number, int q_tiles, int tiles_per_split, int splits, int *qt, int *range) {
    const int pairs = causal_pairs(q_tiles, tiles_per_split / 4, splits);
    if (number >= 0 && number < pairs) {
        int behind;
        causal_pair(number, tiles_per_split / 4, splits, behind, *range);
        *qt = q_tiles - 1 - behind + *range * (tiles_per_split / 4);
    }
    return pairs;
}

namespace {
template <int HD, bool SPLIT, bool CAUSAL, bool MASK>
int launch_wide(hipStream_t st, uint16_t *out, int ldo, const uint16_t *q, const uint16_t *k, const uint16_t *v, int ldi,
                int seq_q, int seq_k, int heads, int kv_heads, float scale, int splits, int per, Partials part,
                const uint32_t *mask_words) {
    static bool configured = false;
    if (!configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(k_fa_fwd_hd512<HD, SPLIT, CAUSAL, MASK>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes(HD));
        if (e != hipSuccess) return (int)e;
        configured = true;
    }
    const int q_tiles = (seq_q + BM - 1) / BM;
    const int total = (CAUSAL ? causal_pairs(q_tiles, per / 4, splits) : q_tiles * splits) * heads;
    const int per_xcd = CAUSAL ? (total + 31) / 32 * 4 : (total + XCDS - 1) / XCDS;     /* causal: whole groups of 32 */
    hipLaunchKernelGGL((k_fa_fwd_hd512<HD, SPLIT, CAUSAL, MASK>), dim3(per_xcd * XCDS), dim3(THREADS), lds_bytes(HD), st, out, ldo,
                       q, k, v, ldi, seq_q, seq_k, heads, q_tiles, splits, per, total, per_xcd, heads / kv_heads,
                       scale * 1.4426950408889634f, part, mask_words);
    return (int)hipGetLastError();
}

template <int HD>
int fa_wide(hipStream_t st, uint16_t *out, int ldo, const uint16_t *q, const uint16_t *k, const uint16_t *v, int ldi, int seq_q,
            int seq_k, int heads, int kv_heads, float scale, int causal, const int *key_mask, int splits, void *scratch) {
    const int tiles = (seq_k + BN - 1) / BN;
    if (seq_k < 1 || splits < 1 || splits > tiles || ((splits > 1 || key_mask) && !scratch))
        return (int)hipErrorInvalidValue;
    const int per = (tiles + splits - 1) / splits;
    if ((tiles + per - 1) / per != splits) return (int)hipErrorInvalidValue;      /* an empty range */
    const size_t rows = splits == 1 ? 0 : (size_t)seq_q * heads * splits;
    Partials part = {reinterpret_cast<float *>(scratch), reinterpret_cast<float *>(scratch) + rows * HD};
    uint32_t *words = nullptr;
    if (key_mask) {
        words = reinterpret_cast<uint32_t *>(reinterpret_cast<float *>(scratch) + rows * (HD + 2));
        hipLaunchKernelGGL(k_pack_key_mask, dim3((unsigned)((tiles + 7) / 8)), dim3(256), 0, st, words, key_mask, seq_k, tiles);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return (int)e;
    }
#define IRIS_WIDE(S, C, M) launch_wide<HD, S, C, M>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, splits, per, part, words)
    int e;
    if (splits == 1) e = causal ? (key_mask ? IRIS_WIDE(false, true, true) : IRIS_WIDE(false, true, false))
                                : (key_mask ? IRIS_WIDE(false, false, true) : IRIS_WIDE(false, false, false));
    else e = causal ? (key_mask ? IRIS_WIDE(true, true, true) : IRIS_WIDE(true, true, false))
                    : (key_mask ? IRIS_WIDE(true, false, true) : IRIS_WIDE(true, false, false));
#undef IRIS_WIDE
    if (e || splits == 1) return e;
    const size_t merge_rows = (size_t)seq_q * heads;
    hipLaunchKernelGGL(k_fa_hd512_merge<HD>, dim3((unsigned)((merge_rows + 3) / 4)), dim3(256), 0, st, out, ldo, part, seq_q,
                       heads, splits, causal ? seq_k : 0, per);
    return (int)hipGetLastError();
}
}  // namespace

/* head_dim 512 (or 256); rows 16-byte aligned (ldi % 8 == 0, ldo % 4 == 0), seq_k >= 1, scale > 0; key_mask: device
 * int [seq_k] or null. `splits` and `scratch` (16-byte aligned) as the plan function of the same head_dim says for the
 * same sizes and flags; scratch may be null when it says 0 bytes. */
extern "C" int iris_hip_fa_hd512(void *stream, uint16_t *out, int ldo, const uint16_t *q,
                                 const uint16_t *k, const uint16_t *v, int ldi, int seq_q,
                                 int seq_k, int heads, int kv_heads, float scale, int causal, const int *key_mask,
                                 int splits, void *scratch) {
    return fa_wide<512>((hipStream_t)stream, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, causal, key_mask, splits, scratch);
}
extern "C" int iris_hip_fa_hd256(void *stream, uint16_t *out, int ldo, const uint16_t *q,
                                 const uint16_t *k, const uint16_t *v, int ldi, int seq_q,
                                 int seq_k, int heads, int kv_heads, float scale, int causal, const int *key_mask,
                                 int splits, void *scratch) {
    return fa_wide<256>((hipStream_t)stream, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, causal, key_mask, splits, scratch);
}
