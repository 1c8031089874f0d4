/*
 * Flash-attention forward for gfx950 (MI355X), head_dim 128, bf16 inputs,
 * f32 accumulation on the matrix cores (v_mfma_f32_16x16x32_bf16).
 *
 * What it computes (reference iris_dev.h:83-92, iris_cuda.cu:597-682 for the
 * online-softmax recurrence): for every head h and query i
 *     out[i] = softmax_j(scale * q_i . k_j) v_j   over the valid keys j
 * where key j is valid when j < seq_k, (causal ? j <= i : true) and
 * (key_mask ? key_mask[j] != 0 : true). A query without valid keys gives a
 * zero row. P is rounded to bf16 for the P.V product (reference
 * iris_cuda.cu:656-665). The row sum is taken over the same rounded values,
 * on the matrix cores: one more product per tile with an all-ones A operand
 * (+6 % MFMAs) replaces 32 additions per lane and the final cross-lane sum,
 * and the weights of the output rows then add up to exactly one. The
 * reference sums the unrounded f32 values; the two differ by the mean of the
 * bf16 rounding errors of a row, far below one bf16 step of the output.
 *
 * Shape of the computation on CDNA4
 * ---------------------------------
 * One workgroup = WAVES (8, 4, 2 or 1) waves of NB blocks of 16 queries of one
 * head; each wave owns its queries for the whole kernel. 8 waves x 32 queries
 * (NB = 2) = 256 queries is the throughput shape (two waves share a SIMD, one
 * workgroup per CU), 4 x 32 the alternative for the large problems whose
 * rounds over the CUs it fills better. A workgroup walks its key tiles one
 * after the other, so a short sequence is bound by that latency: problems of
 * up to 2048 waves of 16 queries take NB = 1, as many small workgroups as it
 * takes to fill the CUs (or the kernel further down that splits the keys).
 * The waves of a workgroup need not carry the same number of blocks: when the
 * last round of 256-query workgroups would leave CUs idle (432 workgroups on
 * 256 CUs run as 256 + 176), the last queries of every head go to workgroups
 * of 192 queries, four waves of 32 and four of 16, so that the last round
 * uses every CU for about 0.78 of a full round (k_fa_fwd_hd128_two_sizes).
 * Keys/values stream through LDS in tiles of 64 keys, 4 stages (2 below 8
 * waves of 32 queries), and they go there directly: global_load_lds_dwordx4 copies
 * HBM/L2 -> LDS without passing through registers, one group of tiles
 * (two tiles, one with the smaller shapes) ahead of the group in use; one barrier per
 * group. Every wave reads the whole K and V tile,
 * so 256 queries per workgroup mean half the L2 -> LDS traffic per query of
 * 128.
 *
 * Both products are issued transposed so that a query is a COLUMN of every
 * accumulator: S^T = K Q^T (A = K tile from LDS, B = Q^T held in registers)
 * and O^T += V^T P^T (A = V^T from LDS, B = P^T). In the 16x16 accumulator
 * layout lane l holds column l%16 and rows 4(l/16) .. +3, so a lane carries
 * two queries (one per 16-query block), their running max, sum and rescale
 * factor are per-lane scalars, and exp2(S^T) converted to bf16 IS the B
 * operand of the second product -- no LDS round trip; the only cross-lane
 * traffic is one v_permlane16_swap + one v_permlane32_swap per query block
 * and tile to combine the row maxima of the four lanes that share a query.
 *
 * Why 16x16x32 and not 32x32x16: same matrix throughput on paper, but this
 * GPU is power-limited on real data, and a loop of nothing but MFMAs on
 * N(0,1) operands sustains about 1.8 PFLOP/s with the 16x16x32 shape
 * against 1.3 with 32x32x16 (a quarter of the accumulator registers read
 * and written per flop).
 *
 * LDS layout: K and V tiles row-major [64][128] bf16, 256 B rows, unpadded
 * (a direct load writes 64 lanes x 16 B to consecutive addresses, so rows
 * cannot be padded); instead the 16 B chunk c of row r is kept in slot
 * c ^ 2(r mod 8) of its row, the permutation being applied to the SOURCE
 * address of the lane that fills the slot. ds_read_b128 serves 16 lanes per
 * pass, and a pass is not 16 consecutive lanes: lanes 0-3, 12-15, 20-23,
 * 24-27 go together (and the other passes alike), i.e. 16 different rows
 * l%16 with chunk c0 + (0 or 1). Their slots (c0 + e) ^ 2(row mod 8) are 16
 * distinct 16 B bank windows: rows that swizzle alike (r, r+8) sit in
 * different halves of the pass and differ in e, all others differ in the
 * swizzle. The V^T operand comes from the LDS transpose read
 * ds_read_b64_tr_b16, which hands lane i of a 16-lane group column i of a
 * 4-row x 16-column block: four consecutive keys of one head dim, exactly
 * the keys that four consecutive P^T registers of that lane belong to; it
 * serves 32 consecutive lanes (8 rows x 32 B) per pass, and the swizzle
 * sends the eight rows to the eight different 32 B windows (it is even, so
 * the two chunks of a 32 B piece stay adjacent). Hardware counters read zero
 * bank conflicts for both.
 *
 * The running max is only raised when some query of the wave exceeds it by
 * more than 2^8 (the accumulators are then rescaled); otherwise the
 * exponentials are taken against the older max. Softmax is invariant to that
 * shift, and exp2 arguments stay <= 8, far from overflow.
 *
 * Optionally (iris_dev_attention_qnorm, no counterpart in the reference) the per-head RMSNorm
 * and rotary embedding of Q (reference iris_cuda.cu:402-420) are applied to the Q fragments
 * right after they are loaded, with the operations of the stand-alone kernel in the same
 * order, so that the result equals norm-then-attention bit for bit and the separate pass
 * over Q is saved. It is a run-time branch of the prologue, not another instantiation.
 *
 * Workgroups are numbered so that each XCD (own L2) walks a contiguous range
 * of (head, query-tile) pairs: the K/V of a head are then fetched into one
 * L2 instead of eight.
 */
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "iris_kernels_hip.h"
#include "norm_rope_math.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int BN = 64;             /* keys per tile */
constexpr int HD = 128;
constexpr int KS = HD;              /* K and V tile rows are 256 B, unpadded: chunks are swizzled instead */
constexpr int VS = HD;
constexpr int K_TILE = BN * KS;    /* elements */
constexpr int V_TILE = BN * VS;
constexpr int STAGE = K_TILE + V_TILE;      /* 32 KB */
constexpr int XCDS = 8;
constexpr float RESCALE_THRESHOLD = 8.0f;   /* log2 units */

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

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

/* v_maximum3_f32 (a -inf operand is an ordinary value to it). As a builtin, not as inline asm: the
 * compiler may then interleave the independent chains of the two query blocks and place the
 * hazard gaps itself. */
__device__ __forceinline__ float max3(float a, float b, float c) {
    return __builtin_elementwise_maximum(__builtin_elementwise_maximum(a, b), c);
}

/* Max over the four lanes l%16, l%16+16, +32, +48 (one per 16-lane row); every one
 * of them gets the result. v_permlane16_swap(x, x) returns rows {0,0,2,2} and {1,1,3,3} of x,
 * v_permlane32_swap(x, x) rows {0,1,0,1} and {2,3,2,3}. */
__device__ __forceinline__ float quad_group_max(float v) {
    auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    const float t = max3(__uint_as_float(a[0]), __uint_as_float(a[1]), __uint_as_float(a[1]));
    auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(t), __float_as_uint(t), false, false);
    return max3(__uint_as_float(b[0]), __uint_as_float(b[1]), __uint_as_float(b[1]));
}
/* 16 B chunk c of tile row r lives in slot c ^ swz(r) of that row. */
__device__ __forceinline__ int swz(int row) { return 2 * (row & 7); }

/* HBM/L2 -> LDS without passing through registers: one global_load_lds_dwordx4 moves
 * 64 lanes x 16 B into 1 KB of consecutive LDS (lane l at +16 l), i.e. four tile rows.
 * A tile (K then V, 32 KB) is 32 such pieces, NI = ceil(32 / WAVES) per wave; piece g covers
 * rows 4 (g % 16) .. +3 of K (g < 16) or V. The lane that fills slot s of row r fetches
 * chunk s ^ swz(r) of that row: the swizzle is applied on the source side. Rows r and
 * r + 8 swizzle alike, so a lane needs two source offsets in all: lane_off[g % 2], from
 * the first row of the piece.
 *
 * Written as asm, not as __builtin_amdgcn_global_load_lds: the compiler cannot tell which
 * stage a later LDS read touches and would wait for ALL outstanding requests (vmcnt(0))
 * before every operand read, which serialises the pipeline. The waits are placed by hand
 * (wait_vmcnt) where a tile is first needed. M0 carries the LDS address and is named as
 * clobbered by every such statement. */
__device__ __forceinline__ uint32_t lds_address(const uint16_t *p) {
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void *)p;
}

/* a pointer the compiler must keep in scalar registers (it is wave-uniform, but selected at run time) */
__device__ __forceinline__ const uint16_t *scalar_ptr(const uint16_t *p) {
    const uint64_t v = (uint64_t)(uintptr_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (const uint16_t *)(uintptr_t)(((uint64_t)hi << 32) | lo);
}

/* The same for a pointer that an asm load reads right away. v_readfirstlane is a vector instruction, and a memory
 * instruction must not read a scalar register within five wait states of a vector instruction writing it; the
 * compiler places those wait states in front of the memory instructions it issues itself, not in front of an asm
 * statement. (Unsettled, the load could be issued with the register's previous contents: in practice the old high
 * half of the address, i.e. wrong only across a 4 GB boundary.) */
__device__ __forceinline__ const uint16_t *settled_scalar_ptr(const uint16_t *p) {
    p = scalar_ptr(p);
    asm volatile("s_nop 4" : "+s"(p));
    return p;
}

/* The compiler reserves M0 for its own short-lived uses and remarks on seeing it in a clobber list;
 * naming it is still what tells it that a value it placed there does not survive the statement. */
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
template <int NI, int WAVES>
__device__ __forceinline__ void load_tile(uint16_t *stage, const uint16_t *kt, const uint16_t *vt, int ldi,
                                          const uint32_t (&lane_off)[2], int wave) {
    if constexpr (NI <= 8) {
#pragma unroll
        for (int j = 0; j < NI; j++) {
            /* wave-uniform. A wave count that does not divide 32 (12 waves) deals the pieces out
             * round-robin, and the last round is short. */
            const int g = 32 % WAVES == 0 ? wave * NI + j : wave + j * WAVES;
            if (32 % WAVES != 0 && g >= 32) break;
            const uint16_t *src = (g < 16 ? kt : vt) + (size_t)(4 * (g & 15)) * ldi;      /* first row of the piece */
            const uint16_t *dst = stage + (g < 16 ? 0 : K_TILE) + 4 * (g & 15) * KS;
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                         ::"s"(lds_address(dst)), "v"(lane_off[g & 1]), "s"(src) : "memory", "m0");
        }
    } else {
        /* 16 or 32 pieces per wave (2 waves: one takes K, the other V; 1 wave: K then V). Source
         * pointer and LDS address are advanced from piece to piece, and the empty asm hides the
         * running values from the compiler: computed independently, the 32 pointers and addresses
         * become invariants of the tile loop and spill out of the scalar registers. */
#pragma unroll
        for (int part = 0; part < NI / 16; part++) {
            const bool is_v = wave * NI + 16 * part >= 16;
            const uint16_t *src = settled_scalar_ptr(is_v ? vt : kt);
            uint32_t dst = __builtin_amdgcn_readfirstlane(lds_address(stage + (is_v ? K_TILE : 0)));
            const size_t step = 4 * (size_t)ldi;
#pragma unroll
            for (int j = 0; j < 16; j++) {
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                             ::"s"(dst), "v"(lane_off[j & 1]), "s"(src) : "memory", "m0");
                src += step;
                dst += 4 * KS * 2;
                asm volatile("" : "+s"(src), "+s"(dst));
            }
        }
    }
}

/* The same for the last tile of a sequence whose rows run out before the tile does: rows
 * past `last_row` (relative to the tile) are redirected to it. Their scores are masked and
 * their probabilities are exactly zero, so the values never matter; they only must be
 * finite, which any real row is. */
template <int NI, int WAVES>
__device__ __forceinline__ void load_tile_clamped(uint16_t *stage, const uint16_t *kt, const uint16_t *vt, int ldi,
                                                  int last_row, int lane, int wave) {
#pragma unroll
    for (int j = 0; j < NI; j++) {
        const int g = 32 % WAVES == 0 ? wave * NI + j : wave + j * WAVES;
        if (32 % WAVES != 0 && g >= 32) break;
        const int row = 4 * (g & 15) + (lane >> 4);
        const int chunk = (lane & 15) ^ swz(row);
        const uint16_t *src = (g < 16 ? kt : vt) + (size_t)min(row, last_row) * ldi + 8 * chunk;
        const uint16_t *dst = stage + (g < 16 ? 0 : K_TILE) + 4 * (g & 15) * KS;
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                     ::"s"(lds_address(dst)), "v"(src) : "memory", "m0");
    }
}

#pragma clang diagnostic pop

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

/* Optional RMSNorm + rotary embedding of Q while it is loaded (w == nullptr: Q is taken as it
 * is). cos/sin rows belong to the query rows, as in iris_dev_head_norm_rope. */
struct QNorm {
    const float *w, *rope_cos, *rope_sin;
    float eps;
    int split_half;
};

/* Sum over the four lanes l%16, +16, +32, +48, paired (l, l+32) first and then (l, l+16): with
 * the lane in 16-lane row g holding u[g] this is (u[0] + u[2]) + (u[1] + u[3]). */
__device__ __forceinline__ float quad_group_sum_02_13(float v) {
    auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    const float w = __uint_as_float(b[0]) + __uint_as_float(b[1]);
    auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(w), __float_as_uint(w), false, false);
    return __uint_as_float(a[0]) + __uint_as_float(a[1]);
}

/* Normalises and rotates the 32 dims of one query that a lane holds as B operands: chunk
 * c = 4 ks + lg (dims 8c .. 8c+7) in qb[ks], the other chunks of the query in the lanes 16, 32
 * and 48 away. Same operations in the same order as k_norm_rope_hd128 (norm_rope_math.h), so the
 * operand bits equal what that kernel would have stored. */
__device__ __forceinline__ void norm_rope_q_fragment(bf16x8 (&qb)[4], const QNorm &qn, int row, int lg) {
    float e[4][8], p[4];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
        const u32x4 raw = __builtin_bit_cast(u32x4, qb[ks]);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            e[ks][2 * j] = __uint_as_float(raw[j] << 16);
            e[ks][2 * j + 1] = __uint_as_float(raw[j] & 0xffff0000u);
        }
        p[ks] = nr_chunk_sum_squares(e[ks]);
    }
    /* chunks lg, lg+4, lg+8, lg+12: t[lg] = p0 + p2, t[lg+4] = p1 + p3, u[lg] = t[lg] + t[lg+4] */
    const float inv = nr_inv_rms128(quad_group_sum_02_13((p[0] + p[2]) + (p[1] + p[3])), qn.eps);
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
        const float4 w0 = *reinterpret_cast<const float4 *>(qn.w + 32 * ks + 8 * lg);
        const float4 w1 = *reinterpret_cast<const float4 *>(qn.w + 32 * ks + 8 * lg + 4);
        const float w8[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
        for (int i = 0; i < 8; i++) e[ks][i] = nr_scaled(e[ks][i], inv, w8[i]);
    }
    const float *ct = qn.rope_cos + (size_t)row * 64, *st = qn.rope_sin + (size_t)row * 64;
    float o[4][8];
    if (qn.split_half) {
        /* pairs (d, d + 64): chunk c < 8 holds a, chunk c + 8 (k-step ks + 2 of the same lane) holds b;
         * table columns 8c .. 8c+7 */
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
            const int col = 32 * ks + 8 * lg;
            const float4 c0 = *reinterpret_cast<const float4 *>(ct + col), c1 = *reinterpret_cast<const float4 *>(ct + col + 4);
            const float4 s0 = *reinterpret_cast<const float4 *>(st + col), s1 = *reinterpret_cast<const float4 *>(st + col + 4);
            const float cv[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
            const float sv[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
#pragma unroll
            for (int i = 0; i < 8; i++) {
                o[ks][i] = nr_rot_first(e[ks][i], e[ks + 2][i], cv[i], sv[i]);
                o[ks + 2][i] = nr_rot_second(e[ks][i], e[ks + 2][i], cv[i], sv[i]);
            }
        }
    } else {
        /* pairs (2i, 2i+1): four per chunk, table columns 4c .. 4c+3 */
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            const int col = 16 * ks + 4 * lg;
            const float4 c4 = *reinterpret_cast<const float4 *>(ct + col), s4 = *reinterpret_cast<const float4 *>(st + col);
            const float cv[4] = {c4.x, c4.y, c4.z, c4.w}, sv[4] = {s4.x, s4.y, s4.z, s4.w};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                o[ks][2 * j] = nr_rot_first(e[ks][2 * j], e[ks][2 * j + 1], cv[j], sv[j]);
                o[ks][2 * j + 1] = nr_rot_second(e[ks][2 * j], e[ks][2 * j + 1], cv[j], sv[j]);
            }
        }
    }
#pragma unroll
    for (int ks = 0; ks < 4; ks++)
        qb[ks] = __builtin_bit_cast(bf16x8, u32x4{pack_bf16(o[ks][0], o[ks][1]), pack_bf16(o[ks][2], o[ks][3]),
                                                  pack_bf16(o[ks][4], o[ks][5]), pack_bf16(o[ks][6], o[ks][7])});
}


/* The walk of one wave over the key tiles of its workgroup. WAVES and GROUP belong to the workgroup (pieces of a
 * tile per wave, tiles between two barriers, stages); NB, the blocks of 16 queries the wave carries, may differ
 * between the waves of a workgroup as long as every wave passes the same barriers: the tile count depends on the
 * workgroup's queries q0 .. q0 + bm - 1 only. wq0 is the wave's first query. */
template <int WAVES, int NB, int GROUP, bool CAUSAL, bool MASK>
__device__ __forceinline__ void
fa_walk_hd128(uint16_t *__restrict__ lds, uint16_t *__restrict__ out, int ldo, const uint16_t *__restrict__ q,
              const uint16_t *__restrict__ k, const uint16_t *__restrict__ v, int ldi,
              int seq_q, int seq_k, int head, int kvh, int q0, int bm, int wq0,
              float scale_log2, const int *__restrict__ key_mask, const QNorm &qnorm) {
    constexpr int NI = (32 + WAVES - 1) / WAVES;         /* pieces of a tile per wave (the last waves may have one fewer) */
    constexpr int NSTAGE = 2 * GROUP;                    /* the group in use and the group on its way */

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lg = lane >> 4;       /* 16x16 block: column li, row group lg */
    const int qrow0 = wq0 + li;                     /* this lane's queries: qrow0 + 16 nb, one per query block */

    const uint16_t *kbase = k + (size_t)kvh * HD;
    const uint16_t *vbase = v + (size_t)kvh * HD;

    /* row sums on the matrix cores: an all-ones A operand makes every row of the product the
     * column sum of P^T, i.e. the sum of the lane's query over the tile's keys */
    const bf16x8 ones = __builtin_bit_cast(bf16x8, u32x4{0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u});

    int k_end = seq_k;
    if (CAUSAL) k_end = min(seq_k, q0 + bm);       /* keys beyond the last query of the workgroup are never valid */
    const int ntiles = (k_end + BN - 1) / BN;

    /* LDS read addresses (elements, relative to a stage).
     * K operand (key block mb, k-step ks): row = key 16mb + li, 16 B at dims 32ks + 8lg.
     * V^T operand (dim block db, k-step ks): transpose read of a 4-key x 16-dim block per
     * 16-lane group; the lane supplies row 4lg + li/4 (+32ks, +16 for the second half)
     * and columns 4(li%4) (+16db), and receives the four keys of dim 16db + li. */
    int k_rd[4], v_rd[8];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) k_rd[ks] = li * KS + 8 * ((4 * ks + lg) ^ swz(li));
    {
        const int vrow = 4 * lg + (li >> 2);
#pragma unroll
        for (int db = 0; db < 8; db++)
            v_rd[db] = K_TILE + vrow * VS + 8 * ((2 * db + ((li & 3) >> 1)) ^ swz(vrow)) + 4 * (li & 1);
    }

    /* This lane's source offsets inside a piece (bytes): row lane/16 of the piece, chunk by parity of the piece. */
    uint32_t lane_off[2];
#pragma unroll
    for (int par = 0; par < 2; par++)
        lane_off[par] = (uint32_t)((lane >> 4) * ldi + 8 * ((lane & 15) ^ swz(4 * par + (lane >> 4)))) * 2u;
    unsigned long long *mask_words = reinterpret_cast<unsigned long long *>(lds + NSTAGE * STAGE);

    const int last_k0 = (ntiles - 1) * BN;
    auto request = [&](int tile_index, int stage) {      /* tile indices past the end repeat the last tile */
        const int kn = min(tile_index * BN, last_k0);
        const uint16_t *kt = kbase + (size_t)kn * ldi, *vt = vbase + (size_t)kn * ldi;
        if (kn + BN <= seq_k) load_tile<NI, WAVES>(lds + stage * STAGE, kt, vt, ldi, lane_off, wave);
        else load_tile_clamped<NI, WAVES>(lds + stage * STAGE, kt, vt, ldi, seq_k - 1 - kn, lane, wave);
    };

    f32x4 o[8][NB];                                  /* O^T: dims 16db + 4lg + r of query block nb */
    float m_run[NB], neg_m[NB], bound[NB];           /* running max; its negative (0 while it is -inf); (max + margin) / scale */
    f32x4 l_acc[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
#pragma unroll
        for (int db = 0; db < 8; db++) o[db][nb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        m_run[nb] = -INFINITY; neg_m[nb] = 0.0f; bound[nb] = -INFINITY;
        l_acc[nb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    const float inv_scale_log2 = 1.0f / scale_log2;
    /* ---- prologue: the first group of tiles is requested before Q, so that the two fetches overlap ---- */
#pragma unroll
    for (int t = 0; t < GROUP; t++) request(t, t);

    /* Q^T as B operands: for query block nb and k-step ks the lane holds dims 32ks + 8lg .. +7
     * of query 16nb + li. */
    bf16x8 qb[NB][4];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        const uint16_t *qp = q + (size_t)min(qrow0 + 16 * nb, seq_q - 1) * ldi + (size_t)head * HD + 8 * lg;
#pragma unroll
        for (int ks = 0; ks < 4; ks++)
            qb[nb][ks] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(qp + 32 * ks));
    }
    if (qnorm.w) {                                   /* wave-uniform */
#pragma unroll
        for (int nb = 0; nb < NB; nb++) norm_rope_q_fragment(qb[nb], qnorm, min(qrow0 + 16 * nb, seq_q - 1), lg);
    }

    /* The key mask as one 64-bit word per key tile, kept in LDS behind the stages: built once here,
     * so that the loop has no global load of its own (a load there would be waited for with
     * vmcnt(0), i.e. together with the newest tile requests). Keys past seq_k count as masked. Behind the
     * first tile requests and the Q loads, so that its round trips overlap theirs, and several tiles per wave
     * at a time, so that 64 tiles cost a workgroup of 8 waves one round trip and not eight. */
    if (MASK) {
        constexpr int U = GROUP == 2 ? 8 : 2;               /* the small shapes walk few tiles: two per wave at a time */
        for (int t0 = wave; t0 < ntiles; t0 += U * WAVES) {
            int flag[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int key = (t0 + u * WAVES) * BN + lane;
                flag[u] = key < seq_k ? key_mask[key] : 0;         /* tiles past the last one: key >= seq_k */
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                const unsigned long long word = __ballot(flag[u] != 0);
                if (lane == 0 && t0 + u * WAVES < ntiles) mask_words[t0 + u * WAVES] = word;
            }
        }
    }

    /* The tile requests are invisible to the compiler's own wait-count bookkeeping, so every load it
     * does know about (Q, the norm weights and tables) is completed here: the empty asm consumes the
     * registers, which pins the loads and their wait before this point. (Waiting for them also waits
     * for the older tile requests above, which the barrier below needs anyway.) Left to itself the
     * compiler sinks the Q loads to the loop and re-waits for them in every iteration, which in fact
     * waits for the newest tile requests. */
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            u32x4 t = __builtin_bit_cast(u32x4, qb[nb][ks]);
            asm volatile("" : "+v"(t));
            qb[nb][ks] = __builtin_bit_cast(bf16x8, t);
        }

    /* the first group of tiles has landed */
    wait_vmcnt<0>();
    lds_barrier();                                       /* also publishes the key-mask words */

    /* Key tiles behind the last one that holds a valid key change nothing (their probabilities are all
     * zero), so the walk ends there: a prompt of 40 tokens padded to 512 costs one tile, not eight. Every
     * wave reads the same words and gets the same count, which the barriers in the loop rely on. */
    int ntiles_run = ntiles;
    if (MASK) {
        while (ntiles_run > 0) {
            const unsigned long long word = mask_words[ntiles_run - 1];
            const uint32_t any = __builtin_amdgcn_readfirstlane((uint32_t)word | (uint32_t)(word >> 32));
            if (any) break;
            ntiles_run--;
        }
    }

    /* A wave whose queries all lie behind the end of the sequence (the last workgroup of a head when seq_q is not a
     * multiple of the workgroup's queries: 4608 = 10 x 256 + 11 x 192 - 64) multiplies nothing. It still fetches its
     * share of every tile and passes the same barriers as the others: one per group of tiles, as the loop below. */
    if (wq0 >= seq_q) {                                  /* wave-uniform */
        for (int g0 = 0, half = 0; g0 < ntiles_run; g0 += GROUP, half ^= 1) {
#pragma unroll
            for (int t = 0; t < GROUP; t++) request(g0 + GROUP + t, (half ^ 1) * GROUP + t);
            wait_vmcnt<0>();
            lds_barrier();
        }
        return;
    }

    for (int g0 = 0, half = 0; g0 < ntiles_run; g0 += GROUP, half ^= 1) {
#pragma unroll
      for (int h = 0; h < GROUP; h++) {
        const int it = g0 + h;
        if (it >= ntiles_run) break;                     /* wave-uniform */
        const int k0 = it * BN;
        uint16_t *cur = lds + (half * GROUP + h) * STAGE;

        /* validity of the tile's keys: range / key mask as a wave-uniform 64-bit set (read before
         * the tile requests below, so that waiting for it does not wait for them) */
        unsigned long long valid = ~0ull;
        if (k0 + BN > seq_k) valid = (1ull << (seq_k - k0)) - 1ull;
        if (MASK) valid &= mask_words[it];

        /* ---- S^T = K Q^T : 4 key blocks x 2 query blocks of 16x16, 4 k-steps of 32 dims.
         * Software pipeline over the k-steps: the four A operands of step ks+1 are requested from
         * LDS before the eight MFMAs of step ks are issued, so that the LDS serves reads all the
         * time the matrix core works instead of in one burst from all waves that the MFMAs then
         * wait for. Each operand feeds two MFMAs. ---- */
        f32x4 s[4][NB];
        {
            u32x4 ka[2][4];                                /* two k-steps in flight */
            auto read_k = [&](int ks) {
#pragma unroll
                for (int mb = 0; mb < 4; mb++)
                    ka[ks & 1][mb] = *reinterpret_cast<const u32x4 *>(&cur[k_rd[ks] + 16 * mb * KS]);
            };
            read_k(0);
            __builtin_amdgcn_sched_barrier(0);
            const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                if (ks < 3) read_k(ks + 1);
                __builtin_amdgcn_sched_barrier(0);
                
#pragma unroll
                for (int mb = 0; mb < 4; mb++)
#pragma unroll
                    for (int nb = 0; nb < NB; nb++)
                        s[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, ka[ks & 1][mb]), qb[nb][ks],
                                                                            ks == 0 ? zero : s[mb][nb], 0, 0, 0);
                
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        /* The next group: HBM/L2 -> the stages whose last readers passed the barrier that ended the
         * previous group. Requested here, behind the first tile's QK product, and not right after
         * the barrier: there every wave would issue its requests before its first operand read,
         * with the matrix cores of the whole CU idle meanwhile. It still has the rest of the
         * group's time to land. */
        if (h == 0) {
#pragma unroll
            for (int t = 0; t < GROUP; t++) request(g0 + GROUP + t, (half ^ 1) * GROUP + t);
            __builtin_amdgcn_sched_barrier(0);
        }
        /* s[mb][nb][r] is key k0 + 16mb + 4lg + r against query 16nb + li of the wave */

        /* ---- validity: range / key mask (wave-uniform 64-bit set), causal (per lane) ---- */
        if (valid != ~0ull) {
            const unsigned long long mine = valid >> (4 * lg);
#pragma unroll
            for (int mb = 0; mb < 4; mb++)
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (!((mine >> (16 * mb + r)) & 1ull)) {
#pragma unroll
                        for (int nb = 0; nb < NB; nb++) s[mb][nb][r] = -INFINITY;
                    }
        }
        if (CAUSAL && k0 + BN - 1 > wq0) {
            const int lim0 = qrow0 - k0 - 4 * lg;      /* key offset 16mb + r valid iff <= lim */
#pragma unroll
            for (int mb = 0; mb < 4; mb++)
#pragma unroll
                for (int r = 0; r < 4; r++)
#pragma unroll
                    for (int nb = 0; nb < NB; nb++)
                        if (16 * mb + r > lim0 + 16 * nb) s[mb][nb][r] = -INFINITY;
        }

        /* ---- online softmax: the lane holds 16 of the 64 scores of each of its two queries;
         * the other three quarters sit in the lanes 16, 32 and 48 away.
         * The running max is only raised when some score of the wave exceeds it by more than
         * 2^8, and that test needs no cross-lane traffic: "the largest of a query's 64 scores
         * exceeds the bound" is the same as "the largest of the 16 that some lane holds does",
         * because the four lanes of a query share the bound. So the common tile pays for the
         * per-lane maxima and one compare per query block, and only a tile that does raise the
         * max (the first few of a row) combines the four lanes and rescales. The bound is kept
         * in score units (bound[nb] = (m_run[nb] + 2^8 margin) / scale), next to -m_run. ---- */
        float lane_max[NB];
        bool raise = false;
        {
            float t[NB][6];
#pragma unroll
            for (int nb = 0; nb < NB; nb++) {                  /* independent chains, written side by side */
                t[nb][0] = max3(s[0][nb][0], s[0][nb][1], s[0][nb][2]);
                t[nb][1] = max3(s[0][nb][3], s[1][nb][0], s[1][nb][1]);
                t[nb][2] = max3(s[1][nb][2], s[1][nb][3], s[2][nb][0]);
                t[nb][3] = max3(s[2][nb][1], s[2][nb][2], s[2][nb][3]);
                t[nb][4] = max3(s[3][nb][0], s[3][nb][1], s[3][nb][2]);
            }
#pragma unroll
            for (int nb = 0; nb < NB; nb++) {
                t[nb][0] = max3(t[nb][0], t[nb][1], t[nb][2]);
                t[nb][5] = max3(t[nb][3], t[nb][4], s[3][nb][3]);
            }
#pragma unroll
            for (int nb = 0; nb < NB; nb++) {
                lane_max[nb] = fmaxf(t[nb][0], t[nb][5]);
                raise = raise || lane_max[nb] > bound[nb];
            }
        }

        if (__any(raise)) {
#pragma unroll
            for (int nb = 0; nb < NB; nb++) {
                const float m_new = fmaxf(m_run[nb], quad_group_max(lane_max[nb]) * scale_log2);
                const float alpha = __builtin_amdgcn_exp2f(m_run[nb] - (m_new == -INFINITY ? 0.0f : m_new));
                m_run[nb] = m_new;
                neg_m[nb] = m_new == -INFINITY ? 0.0f : -m_new;     /* finite while every key so far is masked */
                bound[nb] = (m_new + RESCALE_THRESHOLD) * inv_scale_log2;
                l_acc[nb] *= alpha;
#pragma unroll
                for (int db = 0; db < 8; db++) o[db][nb] *= alpha;
            }
        }

        /* P^T as B operands: k-step ks covers keys 32ks .. 32ks+31, of which this lane's 8 are
         * 32ks + 4lg + r (key block 2ks) and 32ks + 16 + 4lg + r (key block 2ks+1). */
        u32x4 pw[2][NB];
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
                float p[8];
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    p[r] = __builtin_amdgcn_exp2f(fmaf(s[2 * ks][nb][r], scale_log2, neg_m[nb]));
                    p[4 + r] = __builtin_amdgcn_exp2f(fmaf(s[2 * ks + 1][nb][r], scale_log2, neg_m[nb]));
                }
                pw[ks][nb] = u32x4{pack_bf16(p[0], p[1]), pack_bf16(p[2], p[3]), pack_bf16(p[4], p[5]), pack_bf16(p[6], p[7])};
            }
        }

        /* ---- O^T += V^T P^T : 2 k-steps of 32 keys x 8 dim blocks x 2 query blocks, pipelined the
         * same way in four groups of four dim blocks: the V^T operands of the next group are
         * requested before the MFMAs of this one ---- */
        {
            s16x4 lo[2][4], hi[2][4];                      /* two groups in flight */
            auto read_v = [&](int g) {                     /* group g: k-step g / 2, dim blocks 4 (g % 2) .. +3 */
#pragma unroll
                for (int d = 0; d < 4; d++) {
                    const uint16_t *vp = &cur[v_rd[4 * (g & 1) + d] + 32 * (g >> 1) * VS];
                    lo[g & 1][d] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(vp));
                    hi[g & 1][d] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(vp + 16 * VS));
                }
            };
            read_v(0);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int g = 0; g < 4; g++) {
                if (g < 3) read_v(g + 1);
                __builtin_amdgcn_sched_barrier(0);
                
                const int ks = g >> 1;
                if ((g & 1) == 0) {
#pragma unroll
                    for (int nb = 0; nb < NB; nb++)
                        l_acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, __builtin_bit_cast(bf16x8, pw[ks][nb]), l_acc[nb], 0, 0, 0);
                }
#pragma unroll
                for (int d = 0; d < 4; d++) {
                    const int db = 4 * (g & 1) + d;
                    s16x8 both = __builtin_shufflevector(lo[g & 1][d], hi[g & 1][d], 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
                    for (int nb = 0; nb < NB; nb++)
                        o[db][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, both), __builtin_bit_cast(bf16x8, pw[ks][nb]),
                                                                            o[db][nb], 0, 0, 0);
                }
                
                __builtin_amdgcn_sched_barrier(0);
            }
        }
      }
        /* this wave's pieces of the next group have landed; after the barrier everybody's have, and
         * nobody reads the stages of this group any more */
        wait_vmcnt<0>();
        lds_barrier();
    }

    wait_vmcnt<0>();       /* nothing may still be on its way into the LDS when it is given back (the loop ends with this wait too) */

    /* ---- normalise and store: the lane holds dims 16db + 4lg + {0..3} of its queries ---- */
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        const float l_tot = l_acc[nb][0];              /* every row of the ones product is the full sum */
        const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
        const int qrow = qrow0 + 16 * nb;
        if (qrow < seq_q) {
            uint16_t *op = out + (size_t)qrow * ldo + (size_t)head * HD + 4 * lg;
#pragma unroll
            for (int db = 0; db < 8; db++) {
                uint2 w;
                w.x = pack_bf16(o[db][nb][0] * inv, o[db][nb][1] * inv);
                w.y = pack_bf16(o[db][nb][2] * inv, o[db][nb][3] * inv);
                *reinterpret_cast<uint2 *>(op + 16 * db) = w;
            }
        }
    }
}

/* Workgroups of WAVES waves that all carry NB blocks of 16 queries. */
template <int WAVES, int NB, bool CAUSAL, bool MASK>
__global__ void __launch_bounds__(64 * WAVES, 2)
k_fa_fwd_hd128(uint16_t *__restrict__ out, int ldo, const uint16_t *__restrict__ q,
               const uint16_t *__restrict__ k, const uint16_t *__restrict__ v, int ldi,
               int seq_q, int seq_k, int q_tiles, int total_work, int work_per_xcd,
               int kv_group, float scale_log2, const int *__restrict__ key_mask, QNorm qnorm) {
    extern __shared__ __align__(16) uint16_t lds[];     /* 2 GROUP stages of [K tile | V tile] */
    constexpr int WQ = 16 * NB;                          /* queries per wave */
    constexpr int BM = WQ * WAVES;
    /* Key tiles between two barriers. Two for the 8-wave shape (one workgroup per CU, so the LDS
     * has room for four stages): the waves of a workgroup then only meet every other tile, and
     * the faster ones do not stand at a barrier while the slower ones finish every single tile. */
    constexpr int GROUP = WAVES * NB >= 12 ? 2 : 1;

    /* XCD-aware numbering: hardware deals workgroups round-robin to the 8
     * XCDs, so id%8 is the XCD; give each XCD a contiguous slice of the
     * head-major work list. */
    const int work = (blockIdx.x % XCDS) * work_per_xcd + blockIdx.x / XCDS;
    if (work >= total_work) return;
    const int head = work / q_tiles;
    int qt = work - head * q_tiles;
    if (CAUSAL) qt = q_tiles - 1 - qt;             /* longest rows first */
    const int q0 = qt * BM;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    fa_walk_hd128<WAVES, NB, GROUP, CAUSAL, MASK>(lds, out, ldo, q, k, v, ldi, seq_q, seq_k, head, head / kv_group, q0, BM,
                                                  q0 + wave * WQ, scale_log2, key_mask, qnorm);
}

/* The last, partly filled round of the kernel above leaves CUs idle: 432 workgroups on 256 CUs run as 256 + 176.
 * Here a call is cut into workgroups of two sizes instead, so that its last round uses every CU for a shorter
 * time: per head `full_tiles` workgroups of 256 queries as above, and behind them `tail_tiles` workgroups of 192
 * queries, in which waves 0-3 carry 32 queries and waves 4-7 carry 16 (every SIMD then has three blocks of 16
 * queries instead of four). The 256-query workgroups of all heads are numbered first, so they are dispatched
 * first; each XCD takes its slice of both lists. */
template <bool CAUSAL, bool MASK>
__global__ void __launch_bounds__(512, 2)
k_fa_fwd_hd128_two_sizes(uint16_t *__restrict__ out, int ldo, const uint16_t *__restrict__ q,
                         const uint16_t *__restrict__ k, const uint16_t *__restrict__ v, int ldi,
                         int seq_q, int seq_k, int full_tiles, int total_full, int full_per_xcd,
                         int tail_tiles, int total_tail, int tail_per_xcd,
                         int kv_group, float scale_log2, const int *__restrict__ key_mask, QNorm qnorm) {
    extern __shared__ __align__(16) uint16_t lds[];     /* four stages of [K tile | V tile] */
    const int xcd = blockIdx.x % XCDS, slot = blockIdx.x / XCDS;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int head, q0, bm, wq0;
    bool two_blocks;
    if (slot < full_per_xcd) {
        const int work = xcd * full_per_xcd + slot;
        if (work >= total_full) return;
        head = work / full_tiles;
        q0 = (work - head * full_tiles) * 256; bm = 256;
        wq0 = q0 + 32 * wave; two_blocks = true;
    } else {
        const int work = xcd * tail_per_xcd + slot - full_per_xcd;
        if (work >= total_tail) return;
        head = work / tail_tiles;
        q0 = full_tiles * 256 + (work - head * tail_tiles) * 192; bm = 192;
        two_blocks = wave < 4;
        wq0 = two_blocks ? q0 + 32 * wave : q0 + 128 + 16 * (wave - 4);
    }
    /* Waves 0-3 and 4-7 of a 192-query workgroup run two instantiations of the walk and meet at its barriers.
     * INVARIANT: every barrier of fa_walk_hd128 is passed the same number of times by both, i.e. no barrier may sit
     * under a condition that depends on NB or on the wave's own queries (wq0) -- the tile counts ntiles / ntiles_run
     * depend on the workgroup's q0, bm and the key mask only, and the path of a wave without queries in the sequence
     * passes one barrier per group like the main loop. A violation would hang the GPU, not fail a test. */
    if (two_blocks)
        fa_walk_hd128<8, 2, 2, CAUSAL, MASK>(lds, out, ldo, q, k, v, ldi, seq_q, seq_k, head, head / kv_group, q0, bm, wq0,
                                             scale_log2, key_mask, qnorm);
    else
        fa_walk_hd128<8, 1, 2, CAUSAL, MASK>(lds, out, ldo, q, k, v, ldi, seq_q, seq_k, head, head / kv_group, q0, bm, wq0,
                                             scale_log2, key_mask, qnorm);
}

/* ---- short sequences ----------------------------------------------------------------------------
 * A workgroup of the kernel above walks its key tiles one after the other, about 1.4 us each for a wave
 * that has its SIMD to itself, so a sequence of a few hundred keys is bound by that chain and not by the
 * matrix cores. Here the keys of a block of 32 queries of one head are SPLIT over the S waves of a
 * workgroup instead: wave s takes tiles s, s + S, ... (two at most up to 512 keys with S = 4), and the S
 * partial results (running max, sum, unnormalised O^T) are merged through the LDS at the end.
 * Nothing is shared between the waves before that, so there is no barrier in the loop and no cooperative
 * loading: each wave loads the K tile it works on straight from global memory into the A-operand registers
 * (16 B per lane are 8 consecutive dims of one key, which is the operand layout), and its V tile into a
 * private 16 KB stage of the LDS (only V needs the transposing LDS read). The loads are asm statements with
 * hand-placed waits, because two are in flight at a time and complete in order: the K tile of the next
 * turn is requested behind this turn's QK product and the V tile behind its PV product, so "K has landed"
 * is vmcnt <= 16 (the 16 V pieces may still be on their way) and "V has landed" likewise with the 16
 * K loads of the turn after. Same arithmetic per tile as the kernel above. */
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
template <int S, bool CAUSAL, bool MASK>
__global__ void __launch_bounds__(64 * S, 2)
k_fa_short_hd128(uint16_t *__restrict__ out, int ldo, const uint16_t *__restrict__ q,
                 const uint16_t *__restrict__ k, const uint16_t *__restrict__ v, int ldi,
                 int seq_q, int seq_k, int q_tiles, int kv_group, float scale_log2,
                 const int *__restrict__ key_mask, QNorm qnorm) {
    extern __shared__ __align__(16) uint16_t lds[];     /* S private V stages; afterwards the partial results */
    constexpr int NB = 2, WQ = 16 * NB;
    const int head = blockIdx.x / q_tiles;
    int qt = blockIdx.x - head * q_tiles;
    if (CAUSAL) qt = q_tiles - 1 - qt;             /* longest rows first */
    const int q0 = qt * WQ;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lg = lane >> 4;
    const int kvh = head / kv_group;
    const int qrow0 = q0 + li;
    const uint16_t *kbase = k + (size_t)kvh * HD + 8 * lg;
    const uint16_t *vbase = v + (size_t)kvh * HD;
    uint16_t *stage = lds + wave * V_TILE;

    int k_end = seq_k;
    if (CAUSAL) k_end = min(seq_k, q0 + WQ);
    const int ntiles = (k_end + BN - 1) / BN;

    uint32_t lane_off[2];
#pragma unroll
    for (int par = 0; par < 2; par++)
        lane_off[par] = (uint32_t)((lane >> 4) * ldi + 8 * ((lane & 15) ^ swz(4 * par + (lane >> 4)))) * 2u;

    /* V tile `it` -> this wave's stage: 16 direct loads of 64 lanes x 16 B (four rows each). A tile that the
     * sequence ends in redirects the missing rows to the last one (their probabilities are zero). */
    auto request_v = [&](int it) {
        const int kn = it * BN;
        if (kn + BN <= seq_k) {
            const uint16_t *src = settled_scalar_ptr(vbase + (size_t)kn * ldi);
            uint32_t dst = __builtin_amdgcn_readfirstlane(lds_address(stage));
            const size_t step = 4 * (size_t)ldi;
#pragma unroll
            for (int j = 0; j < 16; j++) {
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                             ::"s"(dst), "v"(lane_off[j & 1]), "s"(src) : "memory", "m0");
                src += step;
                dst += 4 * VS * 2;
                asm volatile("" : "+s"(src), "+s"(dst));
            }
        } else {
#pragma unroll
            for (int j = 0; j < 16; j++) {
                const int row = 4 * j + (lane >> 4);
                const uint16_t *src = vbase + (size_t)min(kn + row, seq_k - 1) * ldi + 8 * ((lane & 15) ^ swz(row));
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                             ::"s"(lds_address(stage + 4 * j * VS)), "v"(src) : "memory", "m0");
            }
        }
    };
    /* K tile `it` as A operands: key block mb, k-step ks -> key 16 mb + li, dims 32 ks + 8 lg .. + 7.
     * The waits further down count on EXACTLY 16 loads per request_k and 16 per request_v, completing in order, and
     * on no other vector-memory load between a request and its wait (wait_vmcnt<16> = "everything but the newest 16").
     * The compiler does not know that ka is pending between request and wait: nothing may read, copy or spill ka
     * there. tests/test_gpu_attention.py::test_keys_split_over_the_waves_of_a_workgroup holds this kernel against
     * the oracle on causal, masked and ragged calls and would catch a toolchain that breaks either assumption. */
    u32x4 ka[4][4];
    auto request_k = [&](int it) {
#pragma unroll
        for (int mb = 0; mb < 4; mb++) {
            const uint16_t *kp = kbase + (size_t)min(it * BN + 16 * mb + li, seq_k - 1) * ldi;
#pragma unroll
            for (int ks = 0; ks < 4; ks++)
                asm volatile("global_load_dwordx4 %0, %1, off offset:%2" : "=v"(ka[ks][mb]) : "v"(kp), "n"(64 * ks) : "memory");
        }
    };
    auto tile_mask = [&](int it) -> unsigned long long {          /* range and key mask of a tile as a 64-bit set */
        const int key = it * BN + lane;
        if (MASK) return __ballot(key < seq_k && key_mask[min(key, seq_k - 1)] != 0);
        return __ballot(key < seq_k);
    };

    const bool busy = wave < ntiles;                 /* wave-uniform */
    if (busy) request_v(wave);
    bf16x8 qb[NB][4];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        const uint16_t *qp = q + (size_t)min(qrow0 + 16 * nb, seq_q - 1) * ldi + (size_t)head * HD + 8 * lg;
#pragma unroll
        for (int ks = 0; ks < 4; ks++)
            qb[nb][ks] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4 *>(qp + 32 * ks));
    }
    if (busy) request_k(wave);
    /* the masks of this wave's first two tiles here, so that the loop has no load of its own to wait for */
    unsigned long long first_masks[2] = {~0ull, ~0ull};
    if (MASK || k_end + BN > seq_k) {
        first_masks[0] = tile_mask(wave);
        first_masks[1] = tile_mask(wave + S);
    }
    if (qnorm.w) {
#pragma unroll
        for (int nb = 0; nb < NB; nb++) norm_rope_q_fragment(qb[nb], qnorm, min(qrow0 + 16 * nb, seq_q - 1), lg);
    }

    int v_rd[8];
    {
        const int vrow = 4 * lg + (li >> 2);
#pragma unroll
        for (int db = 0; db < 8; db++)
            v_rd[db] = vrow * VS + 8 * ((2 * db + ((li & 3) >> 1)) ^ swz(vrow)) + 4 * (li & 1);
    }

    const bf16x8 ones = __builtin_bit_cast(bf16x8, u32x4{0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u});
    f32x4 o[8][NB];
    float m_run[NB], neg_m[NB], bound[NB];
    f32x4 l_acc[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
#pragma unroll
        for (int db = 0; db < 8; db++) o[db][nb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        m_run[nb] = -INFINITY; neg_m[nb] = 0.0f; bound[nb] = -INFINITY;
        l_acc[nb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    const float inv_scale_log2 = 1.0f / scale_log2;

    /* Q is pinned here together with its wait (see the kernel above); the first K and V tiles, requested
     * around it, are waited for explicitly */
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            u32x4 t = __builtin_bit_cast(u32x4, qb[nb][ks]);
            asm volatile("" : "+v"(t));
            qb[nb][ks] = __builtin_bit_cast(bf16x8, t);
        }
    wait_vmcnt<0>();

    for (int it = wave, turn = 0; it < ntiles; it += S, turn++) {
        const int k0 = it * BN;
        const bool more = it + S < ntiles;           /* wave-uniform */
        unsigned long long valid = ~0ull;
        if (MASK || k0 + BN > seq_k) valid = turn < 2 ? first_masks[turn & 1] : tile_mask(it);   /* a load of the compiler's waits for everything in flight */

        /* this turn's K has landed (requested before the V tile that may still be in flight) */
        wait_vmcnt<16>();
#pragma unroll
        for (int ks = 0; ks < 4; ks++)
#pragma unroll
            for (int mb = 0; mb < 4; mb++) asm volatile("" : "+v"(ka[ks][mb]));

        f32x4 s[4][NB];
        const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int ks = 0; ks < 4; ks++)
#pragma unroll
            for (int mb = 0; mb < 4; mb++)
#pragma unroll
                for (int nb = 0; nb < NB; nb++)
                    s[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, ka[ks][mb]), qb[nb][ks],
                                                                        ks == 0 ? zero : s[mb][nb], 0, 0, 0);
        /* the operands have been read once the scores exist; only then may the registers be loaded again */
#pragma unroll
        for (int mb = 0; mb < 4; mb++)
#pragma unroll
            for (int nb = 0; nb < NB; nb++) asm volatile("" : "+v"(s[mb][nb]));
        if (more) request_k(it + S);

        if (valid != ~0ull) {
            const unsigned long long mine = valid >> (4 * lg);
#pragma unroll
            for (int mb = 0; mb < 4; mb++)
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (!((mine >> (16 * mb + r)) & 1ull)) {
#pragma unroll
                        for (int nb = 0; nb < NB; nb++) s[mb][nb][r] = -INFINITY;
                    }
        }
        if (CAUSAL && k0 + BN - 1 > q0) {
            const int lim0 = qrow0 - k0 - 4 * lg;
#pragma unroll
            for (int mb = 0; mb < 4; mb++)
#pragma unroll
                for (int r = 0; r < 4; r++)
#pragma unroll
                    for (int nb = 0; nb < NB; nb++)
                        if (16 * mb + r > lim0 + 16 * nb) s[mb][nb][r] = -INFINITY;
        }

        float lane_max[NB];
        bool raise = false;
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            const float t0 = max3(s[0][nb][0], s[0][nb][1], s[0][nb][2]), t1 = max3(s[0][nb][3], s[1][nb][0], s[1][nb][1]);
            const float t2 = max3(s[1][nb][2], s[1][nb][3], s[2][nb][0]), t3 = max3(s[2][nb][1], s[2][nb][2], s[2][nb][3]);
            const float t4 = max3(s[3][nb][0], s[3][nb][1], s[3][nb][2]);
            lane_max[nb] = fmaxf(max3(t0, t1, t2), max3(t3, t4, s[3][nb][3]));
            raise = raise || lane_max[nb] > bound[nb];
        }
        if (__any(raise)) {
#pragma unroll
            for (int nb = 0; nb < NB; nb++) {
                const float m_new = fmaxf(m_run[nb], quad_group_max(lane_max[nb]) * scale_log2);
                const float alpha = __builtin_amdgcn_exp2f(m_run[nb] - (m_new == -INFINITY ? 0.0f : m_new));
                m_run[nb] = m_new;
                neg_m[nb] = m_new == -INFINITY ? 0.0f : -m_new;
                bound[nb] = (m_new + RESCALE_THRESHOLD) * inv_scale_log2;
                l_acc[nb] *= alpha;
#pragma unroll
                for (int db = 0; db < 8; db++) o[db][nb] *= alpha;
            }
        }

        u32x4 pw[2][NB];
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
#pragma unroll
            for (int ks = 0; ks < 2; ks++) {
                float p[8];
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    p[r] = __builtin_amdgcn_exp2f(fmaf(s[2 * ks][nb][r], scale_log2, neg_m[nb]));
                    p[4 + r] = __builtin_amdgcn_exp2f(fmaf(s[2 * ks + 1][nb][r], scale_log2, neg_m[nb]));
                }
                pw[ks][nb] = u32x4{pack_bf16(p[0], p[1]), pack_bf16(p[2], p[3]), pack_bf16(p[4], p[5]), pack_bf16(p[6], p[7])};
            }

        /* this turn's V has landed (the next K tile, requested after it, may still be in flight) */
        if (more) wait_vmcnt<16>(); else wait_vmcnt<0>();
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
                l_acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, __builtin_bit_cast(bf16x8, pw[ks][nb]), l_acc[nb], 0, 0, 0);
#pragma unroll
            for (int db = 0; db < 8; db++) {
                const uint16_t *vp = &stage[v_rd[db] + 32 * ks * VS];
                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(vp));
                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(vp + 16 * VS));
                const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
                for (int nb = 0; nb < NB; nb++)
                    o[db][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, both), __builtin_bit_cast(bf16x8, pw[ks][nb]),
                                                                        o[db][nb], 0, 0, 0);
            }
        }
        if (more) {
            /* every operand read of the stage has returned before it is written again */
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            request_v(it + S);
        }
    }

    /* ---- merge the S partial results. A wave writes its O^T registers as they are over its own stage
     * (part[wave][db][nb][lane]) and its (max, sum) behind the stages (ml[wave][nb][lane]); after the one barrier
     * wave w merges dim blocks (8 / S) w .. : factor exp2(m_j - max_j m_j) per partial. ---- */
    f32x4 *part = reinterpret_cast<f32x4 *>(lds);
    float2 *ml = reinterpret_cast<float2 *>(lds + S * V_TILE);
#pragma unroll
    for (int db = 0; db < 8; db++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++) part[((wave * 8 + db) * NB + nb) * 64 + lane] = o[db][nb];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) ml[(wave * NB + nb) * 64 + lane] = make_float2(m_run[nb], l_acc[nb][0]);
    lds_barrier();
    constexpr int DBS = 8 / S;
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        float mj[S], lj[S], m_all = -INFINITY;
#pragma unroll
        for (int j = 0; j < S; j++) {
            const float2 t = ml[(j * NB + nb) * 64 + lane];
            mj[j] = t.x; lj[j] = t.y;
            m_all = fmaxf(m_all, t.x);
        }
        float l_tot = 0.0f;
        f32x4 acc[DBS];
#pragma unroll
        for (int d = 0; d < DBS; d++) acc[d] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int j = 0; j < S; j++) {
            const float f = mj[j] == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(mj[j] - m_all);
            l_tot = fmaf(f, lj[j], l_tot);
#pragma unroll
            for (int d = 0; d < DBS; d++) acc[d] += f * part[((j * 8 + DBS * wave + d) * NB + nb) * 64 + lane];
        }
        const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
        const int qrow = qrow0 + 16 * nb;
        if (qrow < seq_q) {
            uint16_t *op = out + (size_t)qrow * ldo + (size_t)head * HD + 4 * lg;
#pragma unroll
            for (int d = 0; d < DBS; d++) {
                uint2 w;
                w.x = pack_bf16(acc[d][0] * inv, acc[d][1] * inv);
                w.y = pack_bf16(acc[d][2] * inv, acc[d][3] * inv);
                *reinterpret_cast<uint2 *>(op + 16 * (DBS * wave + d)) = w;
            }
        }
    }
}
#pragma clang diagnostic pop

template <int W, int NB> constexpr size_t stage_bytes() { return (W * NB >= 12 ? 4 : 2) * STAGE * sizeof(uint16_t); }
constexpr size_t LDS_MAX = 160 * 1024;

/* Compute units of the current device (256 on an MI355X in its single-partition mode); 256 where no device answers,
 * so that the planner can be exercised on a machine without a GPU. The costs further down were fitted on 256 CUs in
 * 8 XCDs: another SKU or partition mode changes the rounds through this count, the cost constants want a re-fit. */
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

template <int W, int NB, bool C, bool M>
int launch(hipStream_t st, uint16_t *out, int ldo, const uint16_t *q, const uint16_t *k,
           const uint16_t *v, int ldi, int seq_q, int seq_k, int heads, int kv_heads,
           float scale, const int *key_mask, const QNorm &qn) {
    static bool configured = false;
    if (!configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(k_fa_fwd_hd128<W, NB, C, M>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_MAX);
        if (e != hipSuccess) return (int)e;
        configured = true;
    }
    const int q_tiles = (seq_q + 16 * NB * W - 1) / (16 * NB * W);
    const int total = q_tiles * heads;
    const int per_xcd = (total + XCDS - 1) / XCDS;
    /* the stages, and for a key mask one 64-bit word per key tile behind them */
    const size_t lds_bytes = stage_bytes<W, NB>() + (M ? 8 * (size_t)((seq_k + BN - 1) / BN) : 0);
    if (lds_bytes > LDS_MAX) return (int)hipErrorInvalidValue;       /* the caller keeps masked seq_k below the limit */
    hipLaunchKernelGGL((k_fa_fwd_hd128<W, NB, C, M>), dim3(per_xcd * XCDS), dim3(64 * W), lds_bytes, st, out, ldo,
                       q, k, v, ldi, seq_q, seq_k, q_tiles, total, per_xcd, heads / kv_heads,
                       scale * 1.4426950408889634f, key_mask, qn);
    return (int)hipGetLastError();
}

template <bool C, bool M>
int launch_two_sizes(hipStream_t st, uint16_t *out, int ldo, const uint16_t *q, const uint16_t *k,
                     const uint16_t *v, int ldi, int seq_q, int seq_k, int heads, int kv_heads,
                     float scale, const int *key_mask, const QNorm &qn, int full_tiles) {
    static bool configured = false;
    if (!configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(k_fa_fwd_hd128_two_sizes<C, M>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_MAX);
        if (e != hipSuccess) return (int)e;
        configured = true;
    }
    const int rest = seq_q - 256 * full_tiles;
    const int tail_tiles = rest > 0 ? (rest + 191) / 192 : 0;
    const int total_full = full_tiles * heads, total_tail = tail_tiles * heads;
    const int full_per_xcd = (total_full + XCDS - 1) / XCDS, tail_per_xcd = (total_tail + XCDS - 1) / XCDS;
    const size_t lds_bytes = stage_bytes<8, 2>() + (M ? 8 * (size_t)((seq_k + BN - 1) / BN) : 0);
    if (lds_bytes > LDS_MAX) return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL((k_fa_fwd_hd128_two_sizes<C, M>), dim3((full_per_xcd + tail_per_xcd) * XCDS), dim3(512), lds_bytes, st,
                       out, ldo, q, k, v, ldi, seq_q, seq_k, full_tiles, total_full, full_per_xcd, tail_tiles, total_tail,
                       tail_per_xcd, heads / kv_heads, scale * 1.4426950408889634f, key_mask, qn);
    return (int)hipGetLastError();
}

template <int W, int NB = 2>
int launch_w(hipStream_t st, uint16_t *out, int ldo, const uint16_t *q, const uint16_t *k,
             const uint16_t *v, int ldi, int seq_q, int seq_k, int heads, int kv_heads, float scale,
             int causal, const int *key_mask, const QNorm &qn) {
    if (causal) {
        if (key_mask) return launch<W, NB, true, true>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, key_mask, qn);
        return launch<W, NB, true, false>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, key_mask, qn);
    }
    if (key_mask) return launch<W, NB, false, true>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, key_mask, qn);
    return launch<W, NB, false, false>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, key_mask, qn);
}

template <int S, bool C, bool M>
int launch_short(hipStream_t st, uint16_t *out, int ldo, const uint16_t *q, const uint16_t *k, const uint16_t *v, int ldi,
                 int seq_q, int seq_k, int heads, int kv_heads, float scale, const int *key_mask, const QNorm &qn) {
    static bool configured = false;
    constexpr size_t lds_bytes = (size_t)S * (V_TILE * sizeof(uint16_t) + 1024);     /* stages / partial O^T, and (max, sum) */
    if (!configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(k_fa_short_hd128<S, C, M>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
        if (e != hipSuccess) return (int)e;
        configured = true;
    }
    const int q_tiles = (seq_q + 31) / 32;
    hipLaunchKernelGGL((k_fa_short_hd128<S, C, M>), dim3(heads * q_tiles), dim3(64 * S), lds_bytes, st, out, ldo,
                       q, k, v, ldi, seq_q, seq_k, q_tiles, heads / kv_heads, scale * 1.4426950408889634f, key_mask, qn);
    return (int)hipGetLastError();
}

template <int S>
int launch_short_cm(hipStream_t st, uint16_t *out, int ldo, const uint16_t *q, const uint16_t *k, const uint16_t *v, int ldi,
                    int seq_q, int seq_k, int heads, int kv_heads, float scale, int causal, const int *key_mask, const QNorm &qn) {
    if (causal) {
        if (key_mask) return launch_short<S, true, true>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, key_mask, qn);
        return launch_short<S, true, false>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, key_mask, qn);
    }
    if (key_mask) return launch_short<S, false, true>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, key_mask, qn);
    return launch_short<S, false, false>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, key_mask, qn);
}

}  // namespace

/* How the hardware deals the workgroups of a grid, as far as timing shows it: workgroup i goes to XCD i % 8, the
 * k-th workgroup of an XCD to its shader engine k % 4, whatever is free elsewhere, and a shader engine hands its
 * workgroups in order to whichever of its 8 CUs is free first. (Measured on the two-size kernel for every number of
 * 256-query workgroups per head on nine shapes: this rule reproduces every step of the curves to 2-3 %, a rule
 * that pools the 256 CUs does not.) So a grid is as fast as its most loaded shader engine.
 *
 * When the last of `n_full` workgroups of cost 100 followed by `n_tail` of cost `tail_cost` ends on the `cus` CUs of a
 * shader engine. The CUs are kept as groups that become free together; a step deals to one whole group. */
static long makespan(long n_full, long n_tail, long tail_cost, long cus) {
    struct Group { long free_at, cus; } g[3] = {{0, cus}};            /* a group splits twice at most */
    int ng = 1;
    long left[2] = {n_full, n_tail}, end = 0;
    const long cost[2] = {100, tail_cost};
    for (int kind = 0; kind < 2; kind++)
        while (left[kind] > 0) {
            int first = 0;
            for (int i = 1; i < ng; i++)
                if (g[i].free_at < g[first].free_at) first = i;
            const long take = g[first].cus < left[kind] ? g[first].cus : left[kind];
            const long done = g[first].free_at + cost[kind];
            left[kind] -= take;
            if (done > end) end = done;
            if (take == g[first].cus) g[first].free_at = done;          /* the whole group moves on */
            else {                                                      /* the last of their kind: the group splits */
                g[first].cus -= take;
                g[ng].free_at = done; g[ng].cus = take; ng++;
            }
        }
    return end;
}

/* The two-size grid (k_fa_fwd_hd128_two_sizes) on its most loaded XCD, the first: workgroups k = 0 .. fx - 1 of the
 * XCD are the 256-query ones, k = fx .. fx + tx - 1 the 192-query ones, and k % 4 is the shader engine. */
static long two_sizes_cost(long n_full, long n_tail) {
    const long fx = (n_full + XCDS - 1) / XCDS, tx = (n_tail + XCDS - 1) / XCDS;
    long worst = 0;
    for (long s = 0; s < 4; s++) {
        const long full = fx > s ? (fx - s + 3) / 4 : 0, both = fx + tx > s ? (fx + tx - s + 3) / 4 : 0;
        const long c = makespan(full, both - full, 78, cu_count() / XCDS / 4);
        if (c > worst) worst = c;
    }
    return worst;
}

/* Which kernel a call takes: kind 0 = k_fa_fwd_hd128<waves, nb>, 1 = k_fa_fwd_hd128_two_sizes with `full` workgroups
 * of 256 queries per head, 2 = k_fa_short_hd128<split>. Host arithmetic only. */
struct FaPlan { int kind, waves, nb, split, full; };

static FaPlan plan_hd128(int seq_q, int seq_k, int heads, int causal) {
    /* Three regimes, by the number of waves of 16 queries the problem makes (heads x ceil(seq_q / 16)).
     *
     * Up to 2048 of them (one wave per SIMD and CU slot, or fewer): a workgroup walks its key tiles one after the
     * other, so a short sequence is bound by that chain, and the chain is shortest when a wave carries ONE block
     * of 16 queries (NB = 1: half the products per tile and wave, twice the waves): 1, 2, 4 or 8 such waves per
     * workgroup so that the workgroups about fill the 256 CUs. Measured, clocks settled, rows in the L2, against
     * 32 queries per wave: 32 heads on 8 x 512 tokens causal + mask 11.9 us against 15.5; 24 heads x 320 tokens
     * 7.7 against 10.5, x 576 11.8 against 15.2, x 768 17.4 against 20.2, x 1280 26.0 against 29.8 (x 1536: 56 against
     * 45, the other way round); same bits either way. About 0.65 us per key tile with up to two waves per
     * workgroup, 0.92 with four, 1.08 with eight.
     * When the (head, 32-query block) pairs are at most one per CU and the sequence has many key tiles, splitting
     * the keys over the waves of a workgroup (k_fa_short_hd128) is shorter still: 1.45 us per turn of
     * ceil(tiles / 4) (S = 4 waves) plus 1.5 for the merge, which pays from seven tiles on. 1 head x 512 tokens
     * 9.0 us against 9.8; 8 heads x 1024 14.9 against 16.9; 4 heads x 2000 + mask 25.4 against 32.5. (With more than one workgroup per CU its private tiles cost
     * what the shorter chain saves: 32 heads x 512 tokens, 512 workgroups, 16.4 us.)
     *
     * Beyond that, 32 queries per wave, and the choice is between 256 queries (8 waves, one workgroup fills a CU,
     * half the K/V traffic from L2 per query) and 128 queries (4 waves, two workgroups per CU), by the cost of
     * their rounds over the 256 CUs, in units of one full round of 256-query workgroups: such a round costs 1
     * however few CUs it uses; a round of 128-query workgroups costs 1.1 when some CU gets two of them and 0.6
     * when none does (one wave per SIMD runs faster than two, not twice as fast). Constants measured on 16 to 48
     * heads, 256 .. 12800 tokens, clocks settled. */
    const long CUS = cu_count();
    const long waves16 = (long)((seq_q + 15) / 16) * heads;
    if (waves16 <= 8 * CUS) {
        const int w = waves16 <= CUS ? 1 : waves16 <= 640 ? 2 : waves16 <= 4 * CUS ? 4 : 8;
        const long q_tiles32 = (seq_q + 31) / 32;
        const long keys = causal ? (seq_k < 32 * q_tiles32 ? seq_k : 32 * q_tiles32) : seq_k;
        const long tiles = (keys + BN - 1) / BN;
        const long cost_chain = tiles * (w <= 2 ? 65 : w == 4 ? 92 : 108);           /* 0.01 us */
        if (q_tiles32 * heads <= CUS && ((tiles + 3) / 4) * 145 + 150 < cost_chain) return {2, 4, 2, 4, 0};   /* from 7 tiles on */
        return {0, w, 1, 0, 0};
    }
    const long wg256 = (long)((seq_q + 255) / 256) * heads, wg128 = (long)((seq_q + 127) / 128) * heads;
    const long cost8 = 100 * ((wg256 + CUS - 1) / CUS);
    const long rest4 = wg128 % (2 * CUS);
    const long cost4 = 110 * (wg128 / (2 * CUS)) + (rest4 == 0 ? 0 : rest4 <= CUS ? 60 : 110);
    if (!causal && cost8 <= 1000) {
        /* Whatever the one-size kernels leave idle in their last round, two sizes may fill (k_fa_fwd_hd128_two_sizes):
         * every number f of 256-query workgroups per head is priced with the dispatch rule above, a 192-query
         * workgroup at 0.78 of a 256-query one, and the best f is taken if it beats both one-size kernels by 3 %.
         * 24 heads x 4608: 224 us (f = 10, then 11 of 192 queries) against 237 and 262 for the 8- and 4-wave
         * kernels; x 3072: 131 (f <= 6) against 160 / 143; x 5632: 351 (f = 4) against 428 / 404; 16 x 4608: 188
         * against 231 / 206; 24 x 12800 gains 1 % and 30 x 4352 nothing (two full rounds). Over 77 shapes (16 to 48
         * heads, 2304 to 8704 tokens) the choice made here is within 2 % of the best of the 4-wave kernel, the 8-wave
         * kernel and every f on 70 of them and within 5 % on all. Beyond ten rounds the last one no longer matters. */
        long best_cost = (cost8 <= cost4 ? cost8 : cost4) * 97 / 100;
        int best_full = -1;
        for (int f = seq_q / 256; f >= 0; f--) {
            const long tails = (seq_q - 256 * f + 191) / 192;
            const long c = two_sizes_cost((long)f * heads, tails * heads);
            if (c < best_cost) { best_cost = c; best_full = f; }
        }
        if (best_full >= 0) return {1, 8, 2, 0, best_full};
    }
    return {0, cost8 <= cost4 ? 8 : 4, 2, 0, 0};
}

static int launch_any_width(hipStream_t st, uint16_t *out, int ldo, const uint16_t *q, const uint16_t *k,
                            const uint16_t *v, int ldi, int seq_q, int seq_k, int heads, int kv_heads, float scale,
                            int causal, const int *key_mask, const QNorm &qn) {
    const FaPlan p = plan_hd128(seq_q, seq_k, heads, causal);
    if (p.kind == 2) return launch_short_cm<4>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, causal, key_mask, qn);
    if (p.kind == 1) {
        if (key_mask) return launch_two_sizes<false, true>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, key_mask, qn, p.full);
        return launch_two_sizes<false, false>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, key_mask, qn, p.full);
    }
    if (p.nb == 1) {
        if (p.waves == 1) return launch_w<1, 1>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, causal, key_mask, qn);
        if (p.waves == 2) return launch_w<2, 1>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, causal, key_mask, qn);
        if (p.waves == 4) return launch_w<4, 1>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, causal, key_mask, qn);
        return launch_w<8, 1>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, causal, key_mask, qn);
    }
    if (p.waves == 8) return launch_w<8>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, causal, key_mask, qn);
    return launch_w<4>(st, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, causal, key_mask, qn);
}

/* The launcher's choice for a head_dim-128 call, without launching anything (no GPU needed): plan[0] = kind (0 one
 * size, 1 two sizes, 2 keys split over the waves), plan[1] = waves per workgroup, plan[2] = blocks of 16 queries per
 * wave, plan[3] = 256-query workgroups per head of the two-size grid, plan[4] = its 192-query workgroups per head. */
extern "C" void iris_hip_fa_hd128_plan(int seq_q, int seq_k, int heads, int causal, int *plan) {
    const FaPlan p = plan_hd128(seq_q, seq_k, heads, causal);
    plan[0] = p.kind; plan[1] = p.waves; plan[2] = p.nb; plan[3] = p.full;
    plan[4] = p.kind == 1 ? (seq_q - 256 * p.full + 191) / 192 : 0;
}

extern "C" int iris_hip_fa_hd128(void *stream, uint16_t *out, int ldo, const uint16_t *q,
                                 const uint16_t *k, const uint16_t *v, int ldi, int seq_q,
                                 int seq_k, int heads, int kv_heads, float scale, int causal,
                                 const int *key_mask) {
    const QNorm none = {nullptr, nullptr, nullptr, 0.0f, 0};
    return launch_any_width((hipStream_t)stream, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, causal,
                            key_mask, none);
}

/* The same with Q normalised and rotated while it is loaded (w, rope_cos, rope_sin 16-byte aligned). */
extern "C" int iris_hip_fa_hd128_qnorm(void *stream, uint16_t *out, int ldo, const uint16_t *q,
                                       const uint16_t *k, const uint16_t *v, int ldi, int seq_q,
                                       int seq_k, int heads, int kv_heads, float scale, int causal,
                                       const int *key_mask, const float *w, const float *rope_cos,
                                       const float *rope_sin, float eps, int split_half) {
    if (!w || !rope_cos || !rope_sin) return (int)hipErrorInvalidValue;
    const QNorm qn = {w, rope_cos, rope_sin, eps, split_half != 0};
    return launch_any_width((hipStream_t)stream, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, causal,
                            key_mask, qn);
}
