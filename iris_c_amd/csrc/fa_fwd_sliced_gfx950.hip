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
 * g's queries. For every tile of 32 keys each wave multiplies its slice,
 *     S_part^T = K[:, slice] Q[:, slice]^T        (8 MFMAs 32x32x16),
 * the NS partial score blocks are exchanged through LDS and added in slice
 * order, so every wave of the group holds bit-identical scores and runs the
 * same online softmax redundantly; then O[:, slice]^T += V[:, slice]^T P^T
 * (8 MFMAs). As in the 128 kernel both products are transposed, a lane owns
 * one query, and exp2(S^T) in bf16 is directly the B operand.
 *
 * Workgroup = 8 waves = 8/NS query groups (64 queries at 512, 128 at 256).
 * One LDS stage [K tile 32 x (HD+8) | V tile 32 x (HD+32)] plus the exchange
 * area; the next tile waits in registers while the current one is used.
 * Three barriers per tile: scores exchanged / tile consumed / next tile
 * stored.
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

__device__ __forceinline__ float max3(float a, float b, float c) {
    float d;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
    return d;
}

__device__ __forceinline__ float half_swap_max(float v) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float half_swap_sum(float v) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

template <int NS, bool CAUSAL, bool MASK>
__global__ void __launch_bounds__(THREADS, 2)
k_fa_fwd_sliced(uint16_t *__restrict__ out, int ldo, const uint16_t *__restrict__ q,
                const uint16_t *__restrict__ k, const uint16_t *__restrict__ v, int ldi,
                int seq_q, int seq_k, int q_tiles, int total_work, int work_per_xcd,
                int kv_group, float scale_log2, const int *__restrict__ key_mask) {
    constexpr int HD = 128 * NS;
    constexpr int QG = 8 / NS;             /* query groups per workgroup */
    constexpr int BM = 32 * QG;
    constexpr int KS = HD + 8;             /* K tile row stride in elements: 16 B x odd */
    constexpr int VS = HD + 32;            /* V tile row stride: 64 B x odd */
    constexpr int K_TILE = BN * KS, V_TILE = BN * VS;
    constexpr int CPR = HD / 8;            /* 16 B chunks per row */
    constexpr int NP = BN * CPR / THREADS; /* chunks of K (and of V) per thread and tile = NS */
    constexpr int RSTEP = THREADS / CPR;   /* rows between a thread's chunks */

    extern __shared__ __align__(16) uint16_t lds[];     /* [K tile | V tile | score exchange] */
    f32x4 *xch = reinterpret_cast<f32x4 *>(lds + K_TILE + V_TILE);   /* [QG][NS][4][64] */

    const int work = (blockIdx.x % XCDS) * work_per_xcd + blockIdx.x / XCDS;
    if (work >= total_work) return;
    const int head = work / q_tiles;
    int qt = work - head * q_tiles;
    if (CAUSAL) qt = q_tiles - 1 - qt;
    const int kvh = head / kv_group;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int sl = wave % NS, grp = wave / NS;
    const int col = lane & 31, hh = lane >> 5;
    const int q0 = qt * BM, wq0 = q0 + grp * 32, qrow = wq0 + col;

    const uint16_t *kbase = k + (size_t)kvh * HD;
    const uint16_t *vbase = v + (size_t)kvh * HD;

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
    float m_run = -INFINITY, l_run = 0.0f;

    int k_end = seq_k;
    if (CAUSAL) k_end = min(seq_k, q0 + BM);
    const int ntiles = (k_end + BN - 1) / BN;
    const int last_k0 = (ntiles - 1) * BN;

    /* LDS read addresses (elements): K operand row = key `col`, 16 B at dims 128 sl + 16t + 8hh;
     * V^T operand through the transpose read, rows 4hh + (lane%16)/4 (+16t, +8),
     * columns 128 sl + 16 ((lane/16)%2) + 4 (lane%4) (+32 db). */
    const int k_rd = col * KS + 128 * sl + 8 * hh;
    const int v_rd = K_TILE + (4 * hh + ((lane & 15) >> 2)) * VS + 128 * sl + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

    /* This thread's chunks of a tile: rows row0 + RSTEP c, 16 B at element column ccol. */
    const int row0 = tid / CPR, ccol = (tid % CPR) * 8;
    u32x4 tk[NP], tv[NP];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int c = 0; c < NP; c++) {
            const int r = min(k0 + row0 + RSTEP * c, seq_k - 1);     /* rows past the end: masked later */
            const size_t off = (size_t)r * ldi + ccol;
            tk[c] = *reinterpret_cast<const u32x4 *>(kbase + off);
            tv[c] = *reinterpret_cast<const u32x4 *>(vbase + off);
        }
    };
    auto store = [&]() {
#pragma unroll
        for (int c = 0; c < NP; c++) {
            const int r = row0 + RSTEP * c;
            *reinterpret_cast<u32x4 *>(&lds[r * KS + ccol]) = tk[c];
            *reinterpret_cast<u32x4 *>(&lds[K_TILE + r * VS + ccol]) = tv[c];
        }
    };

    fetch(0);
    store();
    fetch(min(BN, last_k0));
    __syncthreads();

    for (int it = 0; it < ntiles; it++) {
        const int k0 = it * BN;

        /* ---- partial scores over this wave's 128 dims ---- */
        f32x16 s;
        {
            u32x4 ka[8];
#pragma unroll
            for (int t = 0; t < 8; t++) ka[t] = *reinterpret_cast<const u32x4 *>(&lds[k_rd + 16 * t]);
            const f32x16 zero = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
            s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ka[0]), qb[0], zero, 0, 0, 0);
#pragma unroll
            for (int t = 1; t < 8; t++)
                s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ka[t]), qb[t], s, 0, 0, 0);
        }
        /* ---- exchange: every wave of the group adds the NS parts in slice order ---- */
        {
            f32x4 *mine = xch + ((grp * NS + sl) * 4) * 64 + lane;
#pragma unroll
            for (int g = 0; g < 4; g++) mine[g * 64] = f32x4{s[4 * g], s[4 * g + 1], s[4 * g + 2], s[4 * g + 3]};
            lds_barrier();
            const f32x4 *all = xch + (grp * NS * 4) * 64 + lane;
#pragma unroll
            for (int g = 0; g < 4; g++) {
                f32x4 a = all[g * 64];
#pragma unroll
                for (int p = 1; p < NS; p++) a += all[(p * 4 + g) * 64];
                s[4 * g] = a.x; s[4 * g + 1] = a.y; s[4 * g + 2] = a.z; s[4 * g + 3] = a.w;
            }
        }
        /* register r holds key k0 + 8(r/4) + 4hh + r%4 for query qrow */

        /* ---- validity ---- */
        unsigned valid = ~0u;
        if (k0 + BN > seq_k) valid = (1u << (seq_k - k0)) - 1u;
        if (MASK) {
            const unsigned long long b = __ballot(lane < BN && (k0 + lane < seq_k) && key_mask[min(k0 + lane, seq_k - 1)] != 0);
            valid &= (unsigned)b;
        }
        if (valid != ~0u) {
            const unsigned mine = valid >> (4 * hh);
#pragma unroll
            for (int r = 0; r < 16; r++)
                if (!((mine >> (8 * (r >> 2) + (r & 3))) & 1u)) s[r] = -INFINITY;
        }
        if (CAUSAL && k0 + BN - 1 > wq0) {
            const int lim = qrow - k0 - 4 * hh;
#pragma unroll
            for (int r = 0; r < 16; r++)
                if (8 * (r >> 2) + (r & 3) > lim) s[r] = -INFINITY;
        }

        /* ---- online softmax, one query per lane ---- */
        float mx = max3(s[0], s[1], s[2]);
#pragma unroll
        for (int r = 3; r < 15; r += 2) mx = max3(mx, s[r], s[r + 1]);
        mx = fmaxf(mx, s[15]);
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
        const float neg_m = m_run == -INFINITY ? 0.0f : -m_run;
        float psum = 0.0f;
        uint32_t pw[8];                            /* pw[4t + j]: k-step t, elements 2j, 2j+1 */
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
            const float p0 = __builtin_amdgcn_exp2f(fmaf(s[r], scale_log2, neg_m));
            const float p1 = __builtin_amdgcn_exp2f(fmaf(s[r + 1], scale_log2, neg_m));
            psum += p0 + p1;
            pw[r >> 1] = pack_bf16(p0, p1);
        }
        l_run += psum;

        /* ---- O[:, slice]^T += V[:, slice]^T P^T ---- */
        {
            s16x4 lo[2][4], hi[2][4];
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int db = 0; db < 4; db++) {
                    const uint16_t *vp = &lds[v_rd + 16 * t * VS + 32 * db];
                    lo[t][db] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(vp));
                    hi[t][db] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(vp + 8 * VS));
                }
#pragma unroll
            for (int t = 0; t < 2; t++) {
                uint4 praw = make_uint4(pw[4 * t], pw[4 * t + 1], pw[4 * t + 2], pw[4 * t + 3]);
                bf16x8 pb = __builtin_bit_cast(bf16x8, praw);
#pragma unroll
                for (int db = 0; db < 4; db++) {
                    s16x8 both = __builtin_shufflevector(lo[t][db], hi[t][db], 0, 1, 2, 3, 4, 5, 6, 7);
                    o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, both), pb, o[db], 0, 0, 0);
                }
            }
        }
        lds_barrier();                              /* tile and exchange area consumed by every wave */
        store();                                    /* tile it+1 */
        fetch(min(k0 + 2 * BN, last_k0));           /* tile it+2 */
        lds_barrier();
    }

    /* ---- normalise and store this wave's 128 dims: lane holds dims 32db + 8g + 4hh + {0..3} ---- */
    const float l_tot = half_swap_sum(l_run);
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
    constexpr size_t LDS_BYTES = (size_t)(BN * (HD + 8) + BN * (HD + 32)) * sizeof(uint16_t) + 8 * 4 * 64 * sizeof(f32x4);
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
