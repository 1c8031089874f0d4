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
 * Three kernels. M, N >= 256 with K a multiple of 128 (every linear layer of the models at their
 * sequence lengths) take k_gemm_w4: tiles of 256 rows x 256, 224 or 192 columns on four waves, one per
 * SIMD, staged through registers. Other shapes with M, N >= 256 and K a multiple of 64, and the convolutions, take
 * k_gemm_dma: the same tiles on 8 waves, loaded straight into LDS. Both are described where they are
 * defined and give the same bits. Everything else with K a multiple of 8 takes k_gemm_bf16:
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
 * Convolution with a multiple of 64 input channels (every layer of the VAE but its first) is an
 * implicit GEMM: the image is converted to bf16 once and k_gemm_dma fetches the pixels under each
 * tap itself, so the k x k patches are never written out. Other shapes gather the patches as bf16
 * rows into scratch (what the reference does for all of them, iris_cuda.cu:959-985) and run the
 * plain GEMM on them, chunked by output pixels so the scratch stays bounded.
 */
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "iris_kernels_hip.h"
#include "norm_rope_math.h"

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

/* ---- the large-shape kernel: 256 x TN tiles, 8 waves, tiles straight from HBM/L2 into LDS ----
 *
 * For M >= 256, N >= TN (256 or 128) and K a multiple of 64. A workgroup is 8 waves (two per SIMD,
 * one workgroup per CU). TN = 256: 2 waves along m x 4 along n, each wave owning 128 (m) x 64 (n)
 * outputs = 8 x 4 accumulator blocks, 12 operand reads from LDS per 32 MFMAs. TN = 128: 4 x 2
 * waves of 64 x 64 (8 reads per 16 MFMAs). K advances in tiles of 64; a stage holds the W tile
 * (TN rows of 128 B) and the x tile (256 rows), two stages. The tiles are written by
 * global_load_lds_dwordx4 (64 lanes x 16 B = eight 128 B rows per instruction, no registers, no
 * LDS-write instructions), requested one k tile ahead; one barrier per k tile.
 *
 * Direct loads cannot pad rows, so the 16 B chunk c of tile row r is kept in slot
 * c ^ ((r >> 1) & 7) of its row, the permutation applied to the source address of the lane that
 * fills the slot. A 128-bit LDS read serves 16 lanes per pass: 16 different rows, eight of them
 * with chunk c0 and eight with c0 + 1, and of each parity of row four with either. Two
 * consecutive rows span the 64 banks once, so rows of equal parity must differ in slot: the
 * rows with chunk c0 have (r >> 1) & 7 in {0, 1, 6, 7} (or {2, 3, 4, 5}), those with c0 + 1 the
 * complement, and c0 is a multiple of 2, which makes the eight slots distinct.
 *
 * CONV: the same product with x never materialised ("implicit GEMM"). Row m of x is output pixel
 * p0 + m, column (tap, channel) is the input pixel under that tap: the 128 B a lane group fetches
 * for (row, k tile) are 64 consecutive channels of ONE input pixel (cin is a multiple of 64, so a
 * k tile never straddles taps), found from the pixel's coordinates; taps that fall outside the
 * image read a page of zeros instead. The image is bf16, channels last. The bias is added in the
 * epilogue. */
constexpr int DT = 256;                          /* tile rows of x (m) */

struct ConvGeom {
    int h, w, cin, ksz, stride, pad, ow, p0;     /* input size, kernel, output width, first output pixel of this launch */
    const uint16_t *zeros;                       /* >= 128 B of zeros, 16-byte aligned */
    const float *bias;                           /* [N] or null; 16-byte aligned */
};

__device__ __forceinline__ uint32_t lds_address(const uint16_t *p) {
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void *)p;
}

/* The per-head RMSNorm + rotary embedding of the leading columns of a projection, applied by the GEMM to its
 * own output tile (head_dim 128): columns [0, q_cols) are heads normalised with wq, [q_cols, qk_cols) with wk,
 * the rest is stored as it is. */
struct QkNorm {
    const float *wq, *wk, *rope_cos, *rope_sin;  /* [128], [128], [M, 64], [M, 64] */
    int q_cols, qk_cols;
    float eps;
    int split_half;
};

/* M0 (the LDS address of a direct load) is named as clobbered by the asm statements below; the
 * compiler reserves that register for its own short-lived uses and remarks on it. */
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
template <typename OUT, int TN, bool CONV, bool QKN = false>
__global__ void __launch_bounds__(512, 2)
k_gemm_dma(OUT *__restrict__ y, const uint16_t *__restrict__ x, const uint16_t *__restrict__ W,
           int M, int N, int K, int tiles_m, int total, int per_xcd, ConvGeom geo, QkNorm qn) {
    constexpr int WAVES_N = TN / 64, WAVES_M = 8 / WAVES_N;    /* wave grid */
    constexpr int NB = DT / WAVES_M / 16;                      /* x blocks (16 rows) per wave: 8 or 4 */
    constexpr int HALVES = NB / 4;
    constexpr int W_PIECES = TN / 64, X_PIECES = 4;            /* 8-row pieces per wave and k tile */
    constexpr int STAGE = (TN + DT) * TK;                      /* elements: W tile then x tile */
    extern __shared__ __align__(16) uint16_t dlds[];          /* two stages (and room for the epilogue) */
    /* Each XCD (own L2) walks a contiguous range of the tile list. The list runs through bands of 8 tile rows
     * (m), inside a band m fastest and then n: the 32 workgroups an XCD runs at a time then form an 8 x 4
     * block of tiles that needs 8 x tiles and 4 W tiles per k step, where a whole column of tile rows at a
     * time would need all of x again for every column of W. */
    const int work = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (work >= total) return;
    constexpr int BAND = 8;
    const int tiles_n = total / tiles_m;
    const int band = work / (BAND * tiles_n), in_band = work - band * (BAND * tiles_n);
    const int band_rows = min(tiles_m - band * BAND, BAND);
    const int bm = band * BAND + in_band % band_rows, bn = in_band / band_rows;
    const int m0 = bm * DT, n0 = bn * TN;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lg = lane >> 4;
    const int wm = wave % WAVES_M, wn = wave / WAVES_M;

    /* this wave's share of a stage: W rows 8 W_PIECES wave .. and x rows 32 wave .. +31 */
    const int w_row0 = 8 * W_PIECES * wave, x_row0 = 8 * X_PIECES * wave;
    const int w_left = N - n0 - w_row0, x_left = M - m0 - x_row0;    /* rows of the share that exist (may be <= 0) */
    const uint16_t *w_share = W + (size_t)n0 * K + (size_t)w_row0 * K;
    const uint16_t *x_share = CONV ? x : x + (size_t)m0 * K + (size_t)x_row0 * K;
    /* byte offset of this lane's 16 B inside a piece, from the piece's first row, by parity of the piece:
     * row lane / 8, chunk (lane % 8) ^ swizzle of that row */
    uint32_t lane_off[2];
    int lane_chunk[2];
#pragma unroll
    for (int par = 0; par < 2; par++) {
        lane_chunk[par] = (lane & 7) ^ ((4 * par + (lane >> 4)) & 7);
        lane_off[par] = (uint32_t)((lane >> 3) * K + 8 * lane_chunk[par]) * 2u;
    }
    /* CONV: coordinates of the four output pixels whose rows this lane fetches (piece j: row 8 j + lane / 8) */
    int pix_y[X_PIECES], pix_x[X_PIECES];
    if (CONV) {
#pragma unroll
        for (int j = 0; j < X_PIECES; j++) {
            const int r = x_row0 + 8 * j + (lane >> 3);
            const int p = geo.p0 + min(m0 + r, M - 1);
            const int oy = p / geo.ow;
            pix_y[j] = oy * geo.stride - geo.pad;
            pix_x[j] = (p - oy * geo.ow) * geo.stride - geo.pad;
        }
    }
    auto load16 = [&](uint16_t *dst, const uint16_t *src) {     /* per-lane source address */
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                     ::"s"(lds_address(dst)), "v"(src) : "memory", "m0");
    };
    auto request = [&](int kt, int stage) {
        uint16_t *w_dst = dlds + stage * STAGE + w_row0 * TK;
        uint16_t *x_dst = dlds + stage * STAGE + TN * TK + x_row0 * TK;
        if (w_left >= 8 * W_PIECES) {                           /* wave-uniform */
            const uint16_t *src = w_share + (size_t)kt * TK;
#pragma unroll
            for (int j = 0; j < W_PIECES; j++)
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                             ::"s"(lds_address(w_dst + 8 * j * TK)), "v"(lane_off[j & 1]), "s"(src + (size_t)(8 * j) * K) : "memory", "m0");
        } else {
            /* rows past the end of the matrix are redirected to its last row (their outputs are never stored) */
#pragma unroll
            for (int j = 0; j < W_PIECES; j++) {
                const int rr = min(8 * j + (lane >> 3), w_left - 1);
                load16(w_dst + 8 * j * TK, w_share + (ptrdiff_t)rr * K + (size_t)kt * TK + 8 * lane_chunk[j & 1]);
            }
        }
        if (CONV) {
            const int per_tap = geo.cin / TK;                   /* k tiles per tap */
            const int tap = kt / per_tap, c0 = (kt - tap * per_tap) * TK;
            const int ky = tap / geo.ksz, kx = tap - ky * geo.ksz;
#pragma unroll
            for (int j = 0; j < X_PIECES; j++) {
                const int iy = pix_y[j] + ky, ix = pix_x[j] + kx;
                const bool inside = iy >= 0 && iy < geo.h && ix >= 0 && ix < geo.w;
                const uint16_t *src = inside ? x + ((size_t)iy * geo.w + ix) * geo.cin + c0 + 8 * lane_chunk[j & 1]
                                             : geo.zeros + 8 * (lane & 7);
                load16(x_dst + 8 * j * TK, src);
            }
        } else if (x_left >= 8 * X_PIECES) {
            const uint16_t *src = x_share + (size_t)kt * TK;
#pragma unroll
            for (int j = 0; j < X_PIECES; j++)
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                             ::"s"(lds_address(x_dst + 8 * j * TK)), "v"(lane_off[j & 1]), "s"(src + (size_t)(8 * j) * K) : "memory", "m0");
        } else {
#pragma unroll
            for (int j = 0; j < X_PIECES; j++) {
                const int rr = min(8 * j + (lane >> 3), x_left - 1);
                load16(x_dst + 8 * j * TK, x_share + (ptrdiff_t)rr * K + (size_t)kt * TK + 8 * lane_chunk[j & 1]);
            }
        }
    };

    f32x4 acc[4][NB];
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
        for (int b = 0; b < NB; b++) acc[a][b] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    /* operand addresses inside a stage (elements): W rows n = 64 wn + 16 a + li, x rows m = 16 NB wm + 16 b + li;
     * (row >> 1) & 7 = li >> 1 for both, whatever a or b */
    int a_rd[2], b_rd[2];
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
        const int slot = 8 * ((4 * ks + lg) ^ (li >> 1));
        a_rd[ks] = (64 * wn + li) * TK + slot;
        b_rd[ks] = TN * TK + (16 * NB * wm + li) * TK + slot;
    }
    const int nk = K / TK;

    request(0, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    lds_barrier();

    for (int kt = 0; kt < nk; kt++) {
        const uint16_t *cur = dlds + (kt & 1) * STAGE;
        /* 2 HALVES steps per k tile: k-step ks, x blocks 4 half .. +3. The operands of the next step are
         * requested from LDS before the 16 MFMAs of this one are issued, so that the LDS works while the
         * matrix core does; the W operands of a k-step are read with its first step. */
        u32x4 av[2][4], bv[2][4];
        auto read_step = [&](int step) {
            const int ks = step / HALVES, half = step % HALVES;
            if (half == 0) {
#pragma unroll
                for (int a = 0; a < 4; a++) av[ks][a] = *reinterpret_cast<const u32x4 *>(&cur[a_rd[ks] + 16 * a * TK]);
            }
#pragma unroll
            for (int b = 0; b < 4; b++) bv[step & 1][b] = *reinterpret_cast<const u32x4 *>(&cur[b_rd[ks] + 16 * (4 * half + b) * TK]);
        };
        read_step(0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int step = 0; step < 2 * HALVES; step++) {
            if (step + 1 < 2 * HALVES) read_step(step + 1);
            __builtin_amdgcn_sched_barrier(0);
            const int ks = step / HALVES, half = step % HALVES;
#pragma unroll
            for (int a = 0; a < 4; a++)
#pragma unroll
                for (int b = 0; b < 4; b++)
                    acc[a][4 * half + b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        __builtin_bit_cast(bf16x8, av[ks][a]), __builtin_bit_cast(bf16x8, bv[step & 1][b]), acc[a][4 * half + b], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            /* the next k tile: HBM/L2 -> the other stage, whose last readers passed the barrier that ended
             * tile kt - 1. Requested behind the first step's MFMAs rather than right after the barrier,
             * where every wave would issue its requests before its first operand read. */
            if (step == 0 && kt + 1 < nk) { request(kt + 1, (kt + 1) & 1); __builtin_amdgcn_sched_barrier(0); }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");       /* this wave's share of the next tile has landed */
        lds_barrier();                                          /* everybody's has, and nobody reads this tile any more */
    }

    /* acc[a][b][r] = y[m0 + 16 NB wm + 16 b + li][n0 + 64 wn + 16 a + 4 lg + r].
     * Stored straight from the accumulators a store instruction covers 16 rows x 64 (f32) or 32 (bf16) bytes,
     * and the write path is bound by the number of such pieces, not by bytes. So the wave's block goes
     * through LDS (free after the loop's last barrier; 16 KB per wave, its own region, no workgroup barrier)
     * and leaves as 16 B per lane along the rows: 4 rows x 256 B (f32) or 8 rows x 128 B (bf16) per
     * instruction. 16 B chunk c of row r sits in slot c ^ (r mod 16) (f32, 16 chunks a row) or
     * c ^ (r mod 8) (bf16, 8 chunks), which keeps both the writes and the reads off each other's banks.
     * LDS serves a wave's instructions in order, so the reads see the writes without a barrier. */
    constexpr int PER16 = 16 / (int)sizeof(OUT);               /* outputs per 16 B */
    const int mw = m0 + 16 * NB * wm, nw = n0 + 64 * wn;
    if constexpr (QKN) {
        /* A head (128 columns) spans the blocks of two waves, so a tile with head columns in it is staged as a
         * whole: 256 rows x 512 B fill the 128 KB exactly. 16 B chunk c of row r sits in slot
         * (c & 16) | ((c ^ r) & 15): the 16 rows of a write and the 16 chunks of a head vector both spread over
         * all banks. Then a 16-lane row per (token, head) vector, 32 vectors a pass, through the same function
         * as the stand-alone kernel: the stored bits are those of the plain projection followed by that kernel. */
        static_assert(sizeof(OUT) == 2 && TN == 256 && !CONV, "bf16 projection tiles of 256 x 256 only");
        if (n0 < qn.qk_cols) {                                  /* the same for the whole workgroup */
#pragma unroll
            for (int b = 0; b < NB; b++)
#pragma unroll
                for (int a = 0; a < 4; a++) {
                    const int row = 16 * NB * wm + 16 * b + li, chunk = 8 * wn + 2 * a + (lg >> 1);
                    const int slot = (chunk & 16) | ((chunk ^ li) & 15);
                    *reinterpret_cast<uint2 *>(&dlds[row * 256 + 8 * slot + 4 * (lg & 1)]) =
                        make_uint2(pack_bf16(acc[a][b][0], acc[a][b][1]), pack_bf16(acc[a][b][2], acc[a][b][3]));
                }
            __syncthreads();
            const int sub = tid & 15, head = (tid >> 4) & 1, row_in = tid >> 5;
            const int n_head = n0 + 128 * head, n = n_head + 8 * sub;
            const bool normed = n_head < qn.qk_cols;
            float w8[8] = {};
            if (normed) {
                const float *wsel = (n_head < qn.q_cols ? qn.wq : qn.wk) + 8 * sub;
                const float4 w0 = *reinterpret_cast<const float4 *>(wsel), w1 = *reinterpret_cast<const float4 *>(wsel + 4);
                w8[0] = w0.x; w8[1] = w0.y; w8[2] = w0.z; w8[3] = w0.w; w8[4] = w1.x; w8[5] = w1.y; w8[6] = w1.z; w8[7] = w1.w;
            }
            const int tcol = qn.split_half ? 8 * (sub & 7) : 4 * sub;
            const int chunk = 16 * head + sub;
#pragma unroll 4
            for (int pass = 0; pass < DT / 16; pass++) {
                const int row = 16 * pass + row_in, m = m0 + row;
                if (m >= M || n_head >= N) continue;            /* the same for the 16 lanes of a vector */
                u32x4 v = *reinterpret_cast<const u32x4 *>(&dlds[row * 256 + 8 * ((chunk & 16) | ((chunk ^ row) & 15))]);
                if (normed) {
                    const float *cr = qn.rope_cos + (size_t)m * 64 + tcol, *sr = qn.rope_sin + (size_t)m * 64 + tcol;
                    float cv[8] = {}, sv[8] = {};
                    const float4 c0 = *reinterpret_cast<const float4 *>(cr), s0 = *reinterpret_cast<const float4 *>(sr);
                    cv[0] = c0.x; cv[1] = c0.y; cv[2] = c0.z; cv[3] = c0.w;
                    sv[0] = s0.x; sv[1] = s0.y; sv[2] = s0.z; sv[3] = s0.w;
                    if (qn.split_half) {
                        const float4 c1 = *reinterpret_cast<const float4 *>(cr + 4), s1 = *reinterpret_cast<const float4 *>(sr + 4);
                        cv[4] = c1.x; cv[5] = c1.y; cv[6] = c1.z; cv[7] = c1.w;
                        sv[4] = s1.x; sv[5] = s1.y; sv[6] = s1.z; sv[7] = s1.w;
                        v = nr_vector_hd128<true>(v, w8, cv, sv, qn.eps, sub);
                    } else {
                        v = nr_vector_hd128<false>(v, w8, cv, sv, qn.eps, sub);
                    }
                }
                *reinterpret_cast<u32x4 *>(reinterpret_cast<uint16_t *>(y) + (size_t)m * N + n) = v;
            }
            return;
        }
    }
    const float *bias = CONV ? geo.bias : nullptr;
    const bool staged = N % PER16 == 0 && ((uintptr_t)y & 15) == 0;
    if (staged) {
        uint16_t *mine = dlds + wave * 8192;                    /* 16 KB */
        if constexpr (sizeof(OUT) == 4) {
            float *buf = reinterpret_cast<float *>(mine);       /* 64 rows x 64 f32 at a time */
#pragma unroll
            for (int half = 0; half < HALVES; half++) {
#pragma unroll
                for (int bb = 0; bb < 4; bb++)
#pragma unroll
                    for (int a = 0; a < 4; a++)
                        *reinterpret_cast<f32x4 *>(&buf[(16 * bb + li) * 64 + 4 * ((4 * a + lg) ^ li)]) = acc[a][4 * half + bb];
#pragma unroll
                for (int it = 0; it < 16; it++) {
                    const int row = 4 * it + (lane >> 4), c = lane & 15;
                    f32x4 v = *reinterpret_cast<const f32x4 *>(&buf[row * 64 + 4 * (c ^ (row & 15))]);
                    const int m = mw + 64 * half + row, n = nw + 4 * c;
                    if (m < M && n < N) {
                        if (bias) v += *reinterpret_cast<const f32x4 *>(bias + n);
                        *reinterpret_cast<f32x4 *>(reinterpret_cast<float *>(y) + (size_t)m * N + n) = v;
                    }
                }
            }
        } else {
            uint16_t *buf = mine;                               /* 16 NB rows x 64 bf16 */
#pragma unroll
            for (int b = 0; b < NB; b++)
#pragma unroll
                for (int a = 0; a < 4; a++) {
                    const int chunk = 2 * a + (lg >> 1);
                    *reinterpret_cast<uint2 *>(&buf[(16 * b + li) * 64 + 8 * (chunk ^ (li & 7)) + 4 * (lg & 1)]) =
                        make_uint2(pack_bf16(acc[a][b][0], acc[a][b][1]), pack_bf16(acc[a][b][2], acc[a][b][3]));
                }
#pragma unroll
            for (int it = 0; it < 2 * NB; it++) {
                const int row = 8 * it + (lane >> 3), c = lane & 7;
                const u32x4 v = *reinterpret_cast<const u32x4 *>(&buf[row * 64 + 8 * (c ^ (row & 7))]);
                const int m = mw + row, n = nw + 8 * c;
                if (m < M && n < N) *reinterpret_cast<u32x4 *>(reinterpret_cast<uint16_t *>(y) + (size_t)m * N + n) = v;
            }
        }
        return;
    }
#pragma unroll
    for (int b = 0; b < NB; b++) {
        const int m = mw + 16 * b + li;
        if (m >= M) continue;
#pragma unroll
        for (int a = 0; a < 4; a++) {
            const int n = nw + 16 * a + 4 * lg;
            if (n >= N) continue;
            f32x4 v = acc[a][b];
            if (bias)
                for (int r = 0; r < 4 && n + r < N; r++) v[r] += bias[n + r];
            store4(y + (size_t)m * N + n, v, N - n);
        }
    }
}
/* ---- tiles of 256 rows x 256, 224 or 192 columns x 64 on FOUR waves, one per SIMD with the whole register file ----
 *
 * For M, N >= 256 and K a multiple of 128. Each wave owns 128 rows x 16 NA columns = NA x 8 accumulator
 * blocks, up to 256 registers that live in AGPRs (the products are asm statements, so that they stay there),
 * so an operand read from the LDS feeds NA or eight products: with NA = 8, 32 reads per 128 MFMAs and k tile, two
 * thirds of the LDS traffic of the 8-wave kernel. A wave that is alone on its SIMD has nobody to hide its other instructions behind:
 * it issues in order, and what stands between two products must fit into the 12 cycles the matrix core still
 * works on the first. Hence
 *  - the tiles are staged through registers (a direct HBM -> LDS load blocks the issuing wave for about 100
 *    cycles): NA + 8 loads of 16 B per thread and k tile, two tiles ahead (two register sets), each written to
 *    the LDS as two 8-byte halves (a 16-byte LDS write takes longer to issue than the gap: 1265 -> 1302 TFLOP/s);
 *  - every gap between two products holds at most one memory instruction: odd gaps of steps 0 - 2 the copies
 *    registers -> LDS of tile kt + 1 and the loads of tile kt + 3, even gaps the operand reads of the next step
 *    (all of them bunched at the step boundaries: 1160 TFLOP/s; two and a load per fourth gap: 1230; one per gap:
 *    1253);
 *  - one barrier per k tile, behind the products of step 2.
 * Same LDS layout as above (128 B rows, chunk c of row r in slot c ^ ((r >> 1) & 7)), two stages. Same bits as the
 * 8-wave kernel (same products in the same order per accumulator). Timing-only ablations at 4608 x 3072 -> 27648,
 * 1270 TFLOP/s as it stood then: without the barrier 1262 -> 1305 (+3.5 %), without the global loads 1451, without
 * loads and LDS writes 1711 (what 128 MFMAs and 32 operand reads per k tile run at), with loads that always hit
 * the same cached tile 1396. */
template <typename OUT, int NA, bool QKN>
__global__ void __launch_bounds__(256, 1)
k_gemm_w4(OUT *__restrict__ y, const uint16_t *__restrict__ x, const uint16_t *__restrict__ W,
          int M, int N, int K, int tiles_m, int total, int per_xcd, QkNorm qn, int streaming_out) {
    /* NA blocks of 16 output columns per wave: tiles of 256 rows x TN = 32 NA columns (256, 224 or 192), so that the
     * launcher can pick the width whose grid fills the last round of the 256 CUs best. */
    constexpr int TN = 32 * NA;
    constexpr int STAGE = (TN + DT) * TK;                      /* elements: W tile then x tile */
    constexpr int NCW = NA, NCX = 8, NCH = NCW + NCX;          /* 16 B chunks of W and of x per thread and k tile: rows srow + 32 c */
    extern __shared__ __align__(16) uint16_t dlds[];          /* two stages (and room for the epilogue) */
    const int work = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (work >= total) return;
    constexpr int BAND = 4;                                    /* tile rows per band; 2, 6, 9, 18 measure the same or worse */
    const int tiles_n = total / tiles_m;
    const int band = work / (BAND * tiles_n), in_band = work - band * (BAND * tiles_n);
    const int band_rows = min(tiles_m - band * BAND, BAND);
    const int bm = band * BAND + in_band % band_rows, bn = in_band / band_rows;
    /* The last tile of a row or column of tiles is moved back so that it ends with the matrix: it overlaps its
     * neighbour, and both write the same bits there (an output's products are summed in the same order whatever
     * tile it is in). So no row is ever clamped and no store bounded. */
    const int m0 = min(bm * DT, M - DT), n0 = min(bn * TN, N - TN);
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lg = lane >> 4;
    const int wm = wave & 1, wn = wave >> 1;

    /* staging: chunk tid % 8 of rows tid / 8 + 32 c; (row >> 1) & 7 is the same for all c, and the loads of a
     * thread differ by uniform offsets */
    const int srow = tid >> 3, schunk = tid & 7;
    const int st_off = srow * TK + 8 * (schunk ^ ((srow >> 1) & 7));
    const char *wt = reinterpret_cast<const char *>(W + (size_t)n0 * K), *xt = reinterpret_cast<const char *>(x + (size_t)m0 * K);   /* uniform tile bases */
    const uint32_t lane_b = (uint32_t)(srow * K + 8 * schunk) * 2u;            /* this thread's bytes into a tile row block: never changes */
    uint32_t tile_b = 0;                                                        /* uniform: bytes of the k tile to fetch next */
    const uint32_t cstride = 64u * (uint32_t)K;                                 /* 32 rows, in bytes */
    const int nk = K / TK, nk_tiles = nk;
    u32x4 wreg[2][NCW], xreg[2][NCX];                          /* two tiles on their way at any time */
    int fetched = 0;                                           /* tiles requested so far; tile_b stays on the last tile at the end */
    auto fetch_one = [&](int set, int c) {                     /* c < NCW: chunk c of W, else chunk c - NCW of x */
        if (c < NCW) wreg[set][c] = *reinterpret_cast<const u32x4 *>(wt + (size_t)(tile_b + c * cstride) + lane_b);
        else xreg[set][c - NCW] = *reinterpret_cast<const u32x4 *>(xt + (size_t)(tile_b + (c - NCW) * cstride) + lane_b);
    };
    auto fetched_tile = [&]() { fetched++; tile_b += fetched < nk_tiles ? 2u * TK : 0u; };
    auto store_half = [&](int set, int stage, int c, int hi) {  /* 8 of the 16 bytes of chunk c */
        uint16_t *w_dst = dlds + stage * STAGE + st_off + 4 * hi;
        const u32x4 v = c < NCW ? wreg[set][c] : xreg[set][c - NCW];
        uint16_t *dst = c < NCW ? w_dst + 32 * c * TK : w_dst + TN * TK + 32 * (c - NCW) * TK;
        *reinterpret_cast<uint2 *>(dst) = hi ? make_uint2(v[2], v[3]) : make_uint2(v[0], v[1]);
    };
    auto store_one = [&](int set, int stage, int c) { store_half(set, stage, c, 0); store_half(set, stage, c, 1); };

    f32x4 acc[NA][8];                                          /* [a: 16 columns][b: 16 rows] */
#pragma unroll
    for (int a = 0; a < NA; a++)
#pragma unroll
        for (int b = 0; b < 8; b++) acc[a][b] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    int a_rd[2], b_rd[2];
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
        const int slot = 8 * ((4 * ks + lg) ^ (li >> 1));
        a_rd[ks] = (16 * NA * wn + li) * TK + slot;
        b_rd[ks] = TN * TK + (128 * wm + li) * TK + slot;
    }

    /* Four steps of 4 NA MFMAs per k tile: k-step ks = step / 2, x blocks 4 (step % 2) .. + 3. The operands of a
     * step are requested from the LDS during the step before it, across the tile boundary too. One barrier per
     * tile, behind the products of step 2: by then every wave has written its share of tile kt + 1 and has read
     * the last operands of tile kt, so after it the stage of tile kt + 1 is complete and the stage of tile kt is
     * free for tile kt + 2. The products are asm statements with the accumulators in AGPRs. */
    u32x4 av[2][NA], bv[2][4];
    auto read_a_one = [&](const uint16_t *stage, int ks, int a) {
        av[ks][a] = *reinterpret_cast<const u32x4 *>(&stage[a_rd[ks] + 16 * a * TK]);
    };
    auto read_b_one = [&](const uint16_t *stage, int step, int b) {
        bv[step & 1][b] = *reinterpret_cast<const u32x4 *>(&stage[b_rd[step >> 1] + 16 * (4 * (step & 1) + b) * TK]);
    };
    auto products = [&](int step, auto &&between) {
        const int ks = step >> 1, half = step & 1;
#pragma unroll
        for (int b = 0; b < 4; b++)
#pragma unroll
            for (int a = 0; a < NA; a++) {
                asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[a][4 * half + b]) : "v"(av[ks][a]), "v"(bv[step & 1][b]));
                between(NA * b + a);
            }
    };

#pragma unroll
    for (int c = 0; c < NCH; c++) fetch_one(0, c);             /* tile 0 */
    fetched_tile();
#pragma unroll
    for (int c = 0; c < NCH; c++) store_one(0, 0, c);
#pragma unroll
    for (int c = 0; c < NCH; c++) fetch_one(1, c);             /* tiles 1 and 2 (or the last tile again) wait in the registers */
    fetched_tile();
#pragma unroll
    for (int c = 0; c < NCH; c++) fetch_one(0, c);
    fetched_tile();
    lds_barrier();
#pragma unroll
    for (int a = 0; a < NA; a++) read_a_one(dlds, 0, a);
#pragma unroll
    for (int b = 0; b < 4; b++) read_b_one(dlds, 0, b);

    /* One k tile: `set` holds tile kt + 1 on entry and tile kt + 3 on exit. */
    auto k_tile = [&](int kt, int set) {
        const uint16_t *cur = dlds + (kt & 1) * STAGE, *nxt = dlds + ((kt + 1) & 1) * STAGE;
        const int nstage = (kt + 1) & 1;
        /* At most one memory instruction behind a product: the wave issues in order, and what it issues between
         * two products has to fit into the 12 cycles the matrix core still works on the first. Even gaps: the
         * operands of the next step in the order its products use them (4 x-blocks, and for an odd step the NA
         * W-blocks of its k-step). Odd gaps of steps 0 - 2, 6 NA of them: the 3 NCH staging jobs in order, chunk by
         * chunk two 8-byte copies registers -> LDS of tile kt + 1 and then the load of the same chunk of tile
         * kt + 3 into the registers just freed; the few that do not fit (NA = 7: 45 jobs, 42 odd gaps) take the
         * even gaps of step 2 behind its four reads. */
        constexpr int ODD = 2 * NA;                             /* odd gaps per step */
        auto staging_job = [&](int j) {
            if (j >= 3 * NCH) return;
            const int c = j / 3, part = j - 3 * c;
            if (part < 2) store_half(set, nstage, c, part);
            else fetch_one(set, c);
        };
        auto slot = [&](int step, int i) {
            const int r = i >> 1;
            if (i & 1) {
                if (step < 3) staging_job(ODD * step + r);
            } else {
                if (step == 0 && r < 4) read_b_one(cur, 1, r);
                if (step == 1) { if (r < 4) read_b_one(cur, 2, r); else if (r < 4 + NA) read_a_one(cur, 1, r - 4); }
                if (step == 2) { if (r < 4) read_b_one(cur, 3, r); else staging_job(3 * ODD + r - 4); }
                if (step == 3) { if (r < 4) read_b_one(nxt, 0, r); else if (r < 4 + NA) read_a_one(nxt, 0, r - 4); }
            }
        };
        products(0, [&](int i) { slot(0, i); });
        products(1, [&](int i) { slot(1, i); });
        products(2, [&](int i) { slot(2, i); });
        fetched_tile();
        lds_barrier();
        products(3, [&](int i) { slot(3, i); });
    };
    for (int kt = 0; kt < nk; kt += 2) {                       /* nk is even */
        k_tile(kt, 1);
        k_tile(kt + 1, 0);
    }
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");                /* the last products have left the matrix core before the accumulators are read */
    lds_barrier();                                              /* the LDS is reused by the epilogue */

    /* acc[a][b][r] = y[m0 + 128 wm + 16 b + li][n0 + 16 NA wn + 16 a + 4 lg + r] */
    constexpr int PER16 = 16 / (int)sizeof(OUT);
    const int mw = m0 + 128 * wm, nw = n0 + 16 * NA * wn;
    if constexpr (QKN) {
        /* the whole 256 x 256 bf16 tile in the LDS (128 KB), then a 16-lane row per (token, head) vector: see k_gemm_dma */
        static_assert(sizeof(OUT) == 2 && NA == 8, "bf16 projection, tiles of two whole heads");
        if (n0 < qn.qk_cols) {
#pragma unroll
            for (int b = 0; b < 8; b++)
#pragma unroll
                for (int a = 0; a < 8; a++) {
                    const int row = 128 * wm + 16 * b + li, chunk = 16 * wn + 2 * a + (lg >> 1);
                    const int slot = (chunk & 16) | ((chunk ^ li) & 15);
                    *reinterpret_cast<uint2 *>(&dlds[row * 256 + 8 * slot + 4 * (lg & 1)]) =
                        make_uint2(pack_bf16(acc[a][b][0], acc[a][b][1]), pack_bf16(acc[a][b][2], acc[a][b][3]));
                }
            __syncthreads();
            const int sub = tid & 15, head = (tid >> 4) & 1, row_in = tid >> 5;
            const int n_head = n0 + 128 * head, n = n_head + 8 * sub;
            const bool normed = n_head < qn.qk_cols;
            float w8[8] = {};
            if (normed) {
                const float *wsel = (n_head < qn.q_cols ? qn.wq : qn.wk) + 8 * sub;
                const float4 w0 = *reinterpret_cast<const float4 *>(wsel), w1 = *reinterpret_cast<const float4 *>(wsel + 4);
                w8[0] = w0.x; w8[1] = w0.y; w8[2] = w0.z; w8[3] = w0.w; w8[4] = w1.x; w8[5] = w1.y; w8[6] = w1.z; w8[7] = w1.w;
            }
            const int tcol = qn.split_half ? 8 * (sub & 7) : 4 * sub;
            const int chunk = 16 * head + sub;
            /* whole tiles: no row or head of the tile lies outside y, so the passes are straight-line code and the
             * table loads of eight of them are in flight together (the wave has its SIMD to itself: nothing else
             * hides their latency) */
#pragma unroll 8
            for (int pass = 0; pass < DT / 8; pass++) {
                const int row = 8 * pass + row_in, m = m0 + row;
                u32x4 v = *reinterpret_cast<const u32x4 *>(&dlds[row * 256 + 8 * ((chunk & 16) | ((chunk ^ row) & 15))]);
                if (normed) {
                    const float *cr = qn.rope_cos + (size_t)m * 64 + tcol, *sr = qn.rope_sin + (size_t)m * 64 + tcol;
                    float cv[8] = {}, sv[8] = {};
                    const float4 c0 = *reinterpret_cast<const float4 *>(cr), s0 = *reinterpret_cast<const float4 *>(sr);
                    cv[0] = c0.x; cv[1] = c0.y; cv[2] = c0.z; cv[3] = c0.w;
                    sv[0] = s0.x; sv[1] = s0.y; sv[2] = s0.z; sv[3] = s0.w;
                    if (qn.split_half) {
                        const float4 c1 = *reinterpret_cast<const float4 *>(cr + 4), s1 = *reinterpret_cast<const float4 *>(sr + 4);
                        cv[4] = c1.x; cv[5] = c1.y; cv[6] = c1.z; cv[7] = c1.w;
                        sv[4] = s1.x; sv[5] = s1.y; sv[6] = s1.z; sv[7] = s1.w;
                        v = nr_vector_hd128<true>(v, w8, cv, sv, qn.eps, sub);
                    } else {
                        v = nr_vector_hd128<false>(v, w8, cv, sv, qn.eps, sub);
                    }
                }
                *reinterpret_cast<u32x4 *>(reinterpret_cast<uint16_t *>(y) + (size_t)m * N + n) = v;
            }
            return;
        }
    }
    const bool staged = N % PER16 == 0 && ((uintptr_t)y & 15) == 0;
    if (staged) {
        /* through the LDS (free after the loop's last barrier; 32 KB per wave, its own region, no workgroup barrier), so
         * that the stores leave as 16 B per lane along the rows. LDS serves a wave's instructions in order. */
        uint16_t *mine = dlds + wave * 16384;
        if constexpr (sizeof(OUT) == 4) {
            float *buf = reinterpret_cast<float *>(mine);       /* 64 rows x 128 f32 at a time, chunk c of row r in slot (c & 16) | ((c ^ r) & 15) */
#pragma unroll
            for (int half = 0; half < 2; half++) {
#pragma unroll
                for (int bb = 0; bb < 4; bb++)
#pragma unroll
                    for (int a = 0; a < NA; a++) {
                        const int chunk = 4 * a + lg;
                        *reinterpret_cast<f32x4 *>(&buf[(16 * bb + li) * 128 + 4 * ((chunk & 16) | ((chunk ^ li) & 15))]) = acc[a][4 * half + bb];
                    }
#pragma unroll
                for (int it = 0; it < 32; it++) {
                    const int row = 2 * it + (lane >> 5), c = lane & 31;
                    f32x4 v = *reinterpret_cast<const f32x4 *>(&buf[row * 128 + 4 * ((c & 16) | ((c ^ row) & 15))]);
                    const int m = mw + 64 * half + row, n = nw + 4 * c;
                    if (c < 4 * NA) {
                        f32x4 *dst = reinterpret_cast<f32x4 *>(reinterpret_cast<float *>(y) + (size_t)m * N + n);
                        if (streaming_out) __builtin_nontemporal_store(v, dst);
                        else *dst = v;
                    }
                }
            }
        } else {
            uint16_t *buf = mine;                               /* 128 rows x 128 bf16, chunk c of row r in slot c ^ (r % 16) */
#pragma unroll
            for (int b = 0; b < 8; b++)
#pragma unroll
                for (int a = 0; a < NA; a++) {
                    const int chunk = 2 * a + (lg >> 1);
                    *reinterpret_cast<uint2 *>(&buf[(16 * b + li) * 128 + 8 * (chunk ^ li) + 4 * (lg & 1)]) =
                        make_uint2(pack_bf16(acc[a][b][0], acc[a][b][1]), pack_bf16(acc[a][b][2], acc[a][b][3]));
                }
#pragma unroll
            for (int it = 0; it < 32; it++) {
                const int row = 4 * it + (lane >> 4), c = lane & 15;
                const u32x4 v = *reinterpret_cast<const u32x4 *>(&buf[row * 128 + 8 * (c ^ (row & 15))]);
                const int m = mw + row, n = nw + 8 * c;
                if (c < 2 * NA) {
                    u32x4 *dst = reinterpret_cast<u32x4 *>(reinterpret_cast<uint16_t *>(y) + (size_t)m * N + n);
                    if (streaming_out) __builtin_nontemporal_store(v, dst);
                    else *dst = v;
                }
            }
        }
        return;
    }
#pragma unroll
    for (int b = 0; b < 8; b++) {
        const int m = mw + 16 * b + li;
        if (m >= M) continue;
#pragma unroll
        for (int a = 0; a < NA; a++) {
            const int n = nw + 16 * a + 4 * lg;
            if (n >= N) continue;
            f32x4 v = acc[a][b];
            store4(y + (size_t)m * N + n, v, N - n);
        }
    }
}

#pragma clang diagnostic pop

constexpr int DMA_LDS_BYTES = 128 * 1024;        /* two stages of (256 + 256) x 128 B; also the 8 x 16 KB of the epilogue */

template <typename OUT, int TN, bool CONV, bool QKN = false>
int launch_gemm_dma(hipStream_t st, OUT *y, const uint16_t *x, const uint16_t *W, int M, int N, int K, const ConvGeom &geo,
                    const QkNorm &qn = QkNorm{}) {
    static bool configured = false;
    if (!configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(k_gemm_dma<OUT, TN, CONV, QKN>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, DMA_LDS_BYTES);
        if (e != hipSuccess) return (int)e;
        configured = true;
    }
    const int tiles_m = (M + DT - 1) / DT, tiles_n = (N + TN - 1) / TN, total = tiles_m * tiles_n;
    const int per_xcd = (total + 7) / 8;
    hipLaunchKernelGGL((k_gemm_dma<OUT, TN, CONV, QKN>), dim3((unsigned)per_xcd * 8), dim3(512), DMA_LDS_BYTES, st, y, x, W, M, N, K,
                       tiles_m, total, per_xcd, geo, qn);
    return (int)hipGetLastError();
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

template <typename OUT, int NA, bool QKN = false>
int launch_gemm_w4(hipStream_t st, OUT *y, const uint16_t *x, const uint16_t *W, int M, int N, int K, const QkNorm &qn = QkNorm{}) {
    static bool configured = false;
    if (!configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(k_gemm_w4<OUT, NA, QKN>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, DMA_LDS_BYTES);
        if (e != hipSuccess) return (int)e;
        configured = true;
    }
    const int tiles_m = (M + DT - 1) / DT, tiles_n = (N + 32 * NA - 1) / (32 * NA), total = tiles_m * tiles_n;
    const int per_xcd = (total + 7) / 8;
    /* An output of 192 MB or more cannot stay in the 256 MB Infinity Cache next to the operands: stored with the
     * streaming hint it does not push the weights out on its way (4608 x 3072 -> 27648: f32 output 671 -> 626 us, bf16
     * 594 -> 585; smaller outputs are within 1 % either way and keep the plain stores, which leave them cached for the
     * operator that reads them next). */
    const int streaming_out = (size_t)M * N * sizeof(OUT) >= ((size_t)192 << 20);
    hipLaunchKernelGGL((k_gemm_w4<OUT, NA, QKN>), dim3((unsigned)per_xcd * 8), dim3(256), DMA_LDS_BYTES, st, y, x, W, M, N, K,
                       tiles_m, total, per_xcd, qn, streaming_out);
    return (int)hipGetLastError();
}

/* What the four-wave kernel takes: at least one tile each way (its last tiles are moved back to end with the
 * matrix, so the sizes need not be multiples of the tile), an even number of k tiles, 16-byte stores, and tiles
 * of less than 4 GB. */
static bool four_wave_shape(int M, int N, int K, size_t out_size) {
    return M >= DT && N >= 256 && K % (2 * TK) == 0 && N % (16 / (int)out_size) == 0 &&
           (size_t)K * 2 * (DT + 32) < ((size_t)1 << 32);             /* a thread's byte offsets into a tile are 32-bit */
}

/* The tile width (32 NA columns) whose grid wastes least of its last round of 256 workgroups: time goes with
 * rounds x width. 4608 x 9216 outputs: 648 tiles of 256 columns are 2.53 rounds, 756 of 224 are 2.95. */
static int four_wave_width(int M, int N) {
    const long tiles_m = (M + DT - 1) / DT;
    int best = 8;
    long best_cost = 0;
    for (int na = 8; na >= 6; na--) {
        const long tiles = tiles_m * ((N + 32 * na - 1) / (32 * na));
        const long cost = ((tiles + 255) / 256) * na * (na == 8 ? 100 : 102);      /* the narrower tiles reuse operands a little less */
        if (na == 8 || cost < best_cost) { best = na; best_cost = cost; }
    }
    return best;
}

/* Which kernel a linear layer takes, host arithmetic only: 3 = k_gemm_w4 with tiles of 32 na columns, 2 = k_gemm_dma,
 * 1 = k_gemm_bf16, 0 = k_gemm_scalar. */
struct GemmPlan { int kernel, na; };
static GemmPlan plan_gemm(int M, int N, int K, int out_size, bool operands_aligned16, bool out_aligned16) {
    if (K > 0 && K % TK == 0 && operands_aligned16 && M >= DT && N >= DT && (size_t)K * 2 * 8 < ((size_t)1 << 31)) {
        if (four_wave_shape(M, N, K, (size_t)out_size) && out_aligned16) return {3, four_wave_width(M, N)};
        return {2, 8};
    }
    if (K > 0 && K % 8 == 0 && operands_aligned16) return {1, 0};
    return {0, 0};
}

template <typename OUT>
int gemm(hipStream_t st, OUT *y, const uint16_t *x, const uint16_t *W, int M, int N, int K) {
    if (M <= 0 || N <= 0) return 0;
    const bool aligned16 = ((uintptr_t)x & 15) == 0 && ((uintptr_t)W & 15) == 0;
    const GemmPlan plan = plan_gemm(M, N, K, (int)sizeof(OUT), aligned16, ((uintptr_t)y & 15) == 0);
    if (plan.kernel == 3 || plan.kernel == 2) {
        const ConvGeom none = {};
        int e;
        if (plan.kernel == 3) {
            e = plan.na == 8 ? launch_gemm_w4<OUT, 8>(st, y, x, W, M, N, K)
              : plan.na == 7 ? launch_gemm_w4<OUT, 7>(st, y, x, W, M, N, K) : launch_gemm_w4<OUT, 6>(st, y, x, W, M, N, K);
        } else {
            e = launch_gemm_dma<OUT, 256, false>(st, y, x, W, M, N, K, none);
        }
        if (e) return e;
    } else if (plan.kernel == 1) {
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

__global__ void __launch_bounds__(64)
k_zero_words(uint32_t *__restrict__ p, int n) {
    for (int i = threadIdx.x; i < n; i += 64) p[i] = 0u;
}

__global__ void __launch_bounds__(256)
k_add_bias_rows(float *__restrict__ y, const float *__restrict__ bias, int cols, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) y[i] += bias[i % cols];
}

}  // namespace

extern "C" {

/* The kernel a linear layer of these sizes takes (aligned operands): plan[0] = 3 four waves, 2 eight waves with
 * direct loads, 1 the 128 x 128 kernel, 0 scalar; plan[1] = columns of a tile of the four-wave kernel. No GPU needed. */
void iris_hip_linear_plan(int rows, int in, int out, int out_bytes, int *plan) {
    const GemmPlan p = plan_gemm(rows, out, in, out_bytes, true, true);
    plan[0] = p.kernel; plan[1] = p.kernel == 3 ? 32 * p.na : 0;
}

int iris_hip_linear_f32(void *stream, float *y, const uint16_t *x, const uint16_t *W, int rows, int in, int out) {
    return gemm<float>((hipStream_t)stream, y, x, W, rows, out, in);
}
int iris_hip_linear_bf16(void *stream, uint16_t *y, const uint16_t *x, const uint16_t *W, int rows, int in, int out) {
    return gemm<uint16_t>((hipStream_t)stream, y, x, W, rows, out, in);
}

/* Zeroes the first IRIS_CONV_ZERO_BYTES of a freshly allocated convolution scratch buffer: the page that taps
 * outside the image read. iris_hip_conv2d never writes there. */
/* y = x W^T as bf16 with the per-head RMSNorm + rotary embedding (head_dim 128) of columns [0, q_cols) (weights
 * wq) and [q_cols, q_cols + k_cols) (weights wk) applied in the GEMM's epilogue. Returns -2, with nothing
 * enqueued, for a shape the tiled kernel does not take: the caller then runs the two steps one after the other. */
int iris_hip_linear_bf16_qknorm(void *stream, uint16_t *y, const uint16_t *x, const uint16_t *W, int rows, int in, int out,
                                int q_cols, int k_cols, const float *wq, const float *wk, const float *rope_cos,
                                const float *rope_sin, float eps, int split_half) {
    const int M = rows, N = out, K = in;
    const uintptr_t all = (uintptr_t)x | (uintptr_t)W | (uintptr_t)y | (uintptr_t)wq | (uintptr_t)wk | (uintptr_t)rope_cos |
                          (uintptr_t)rope_sin;
    const bool tiled = K > 0 && K % TK == 0 && (all & 15) == 0 && M >= DT && N >= DT && (size_t)K * 2 * 8 < ((size_t)1 << 31);
    if (!tiled || N % 128 || q_cols < 0 || k_cols < 0 || q_cols % 128 || k_cols % 128 || q_cols + k_cols > N ||
        q_cols + k_cols == 0)
        return -2;
    const ConvGeom none = {};
    const QkNorm qn = {wq, k_cols ? wk : wq, rope_cos, rope_sin, q_cols, q_cols + k_cols, eps, split_half};
    if (M % DT == 0 && N % 256 == 0 && four_wave_shape(M, N, K, 2))   /* whole tiles: a tile holds two whole heads */
        return launch_gemm_w4<uint16_t, 8, true>((hipStream_t)stream, y, x, W, M, N, K, qn);
    return launch_gemm_dma<uint16_t, 256, false, true>((hipStream_t)stream, y, x, W, M, N, K, none, qn);
}

int iris_hip_conv2d_prepare_scratch(void *stream, uint16_t *scratch) {
    hipLaunchKernelGGL(k_zero_words, dim3(1), dim3(64), 0, (hipStream_t)stream, reinterpret_cast<uint32_t *>(scratch),
                       IRIS_CONV_ZERO_BYTES / 4);
    return (int)hipGetLastError();
}

/* scratch: device buffer of scratch_bytes, 16-byte aligned, prepared once by iris_hip_conv2d_prepare_scratch: the
 * page of zeros, then room for the bf16 image rows of a chunk or (gathered shapes) at least one patch row */
int iris_hip_conv2d(void *stream, uint16_t *scratch, size_t scratch_bytes, float *out, const float *in,
                    const uint16_t *w, const float *bias, int h, int width, int cin, int cout, int k,
                    int stride, int pad_before, int pad_after) {
    hipStream_t st = (hipStream_t)stream;
    const int oh = (h + pad_before + pad_after - k) / stride + 1;
    const int ow = (width + pad_before + pad_after - k) / stride + 1;
    if (oh <= 0 || ow <= 0) return 0;
    const int ohw = oh * ow, row_len = k * k * cin;

    /* Implicit GEMM: the image once as bf16 (the rows a chunk of output rows needs), then k_gemm_dma in its
     * convolution mode straight on it; no patch matrix. Needs cin % 64 == 0 (a k tile inside one tap). */
    if (scratch_bytes <= IRIS_CONV_ZERO_BYTES) return (int)hipErrorInvalidValue;
    const uint16_t *zeros = scratch;
    scratch += IRIS_CONV_ZERO_BYTES / sizeof(uint16_t);
    scratch_bytes -= IRIS_CONV_ZERO_BYTES;
    const size_t in_row_bytes = (size_t)width * cin * sizeof(uint16_t);
    if (cin % TK == 0 && cout >= 128 && ((uintptr_t)w & 15) == 0 && ((uintptr_t)in & 15) == 0 && ((uintptr_t)scratch & 15) == 0 &&
        scratch_bytes / in_row_bytes >= (size_t)k) {
        const long max_in_rows = (long)(scratch_bytes / in_row_bytes);
        const long rows_out = (max_in_rows - k) / stride + 1;          /* (rows_out - 1) * stride + k <= max_in_rows */
        uint16_t *img = scratch;
        const bool bias_fused = bias && ((uintptr_t)bias & 15) == 0;
        for (long r0 = 0; r0 < oh; r0 += rows_out) {
            const long r1 = r0 + rows_out < oh ? r0 + rows_out : oh;
            const long y_lo = r0 * stride - pad_before > 0 ? r0 * stride - pad_before : 0;
            const long y_hi = (r1 - 1) * stride - pad_before + k < h ? (r1 - 1) * stride - pad_before + k : h;
            if (y_hi > y_lo) {
                int e = iris_hip_f32_to_bf16(stream, img, in + (size_t)y_lo * width * cin, (size_t)(y_hi - y_lo) * width * cin);
                if (e) return e;
            }
            const ConvGeom geo = {h, width, cin, k, stride, pad_before, ow, (int)(r0 * ow), zeros, bias_fused ? bias : nullptr};
            const uint16_t *virtual_image = img - (size_t)y_lo * width * cin;     /* row y of the image at + y * width * cin */
            float *dst = out + (size_t)r0 * ow * cout;
            const int m = (int)((r1 - r0) * ow);
            const int e = cout >= 256 ? launch_gemm_dma<float, 256, true>(st, dst, virtual_image, w, m, cout, row_len, geo)
                                      : launch_gemm_dma<float, 128, true>(st, dst, virtual_image, w, m, cout, row_len, geo);
            if (e) return e;
        }
        if (bias && !bias_fused) {
            const size_t n = (size_t)ohw * cout;
            hipLaunchKernelGGL(k_add_bias_rows, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, out, bias, cout, n);
        }
        return (int)hipGetLastError();
    }

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
