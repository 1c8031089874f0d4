/*
 * Elementwise and normalisation operators of the device API for gfx950
 * (reference iris_dev.h:45-107, 123-129; kernels iris_cuda.cu:271-400, 943-946,
 * 1018-1087). All of them are HBM-bound: one pass over the data with 16-byte
 * accesses per lane where the pointers and sizes allow it, a scalar form of
 * the same kernel otherwise.
 *
 * Row normalisations use one wave per row (four rows per workgroup, no LDS,
 * no barrier) and keep the row in registers between the statistics and the
 * write (rows up to 4096 floats; longer rows are read again, from cache).
 * Statistics follow the reference: LayerNorm takes the mean first and the
 * variance about it. Group norm takes its statistics in ONE pass over the
 * image (coalesced per-pixel reads, per-workgroup partial moments of every
 * group, merged in double by a small second kernel) and normalises in a
 * second pass; the partial moments and the final statistics live in a
 * scratch buffer the caller of the launcher provides.
 */
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "iris_kernels_hip.h"

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

namespace {

constexpr int EW_THREADS = 256;
constexpr int ROW_THREADS = 256;

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    f32x2 p = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(p, bf16x2));
}
__device__ __forceinline__ uint16_t to_bf16(float v) { return (uint16_t)(pack_bf16(v, 0.0f) & 0xffffu); }
__device__ __forceinline__ float bf_lo(uint32_t u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float bf_hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }
__device__ __forceinline__ float silu(float v) { return v / (1.0f + __expf(-v)); }

inline unsigned blocks_for(size_t n, int per_block) { return (unsigned)((n + per_block - 1) / per_block); }

/* ---------------------------------------------------------------- elementwise */

enum EwOp { OP_SILU, OP_ADD, OP_ADD_ROW, OP_MULADD_ROW, OP_FILL_ROW };

/* x[i] = f(x[i], a[i] or row[i % dim]); VEC = floats per thread (4: all pointers 16-byte
 * aligned and n, dim multiples of 4; 1 otherwise). */
template <int OP, int VEC>
__global__ void __launch_bounds__(EW_THREADS)
k_ew(float *__restrict__ x, const float *__restrict__ a, const float *__restrict__ row, int dim, size_t n) {
    const size_t i = ((size_t)blockIdx.x * EW_THREADS + threadIdx.x) * VEC;
    if (i >= n) return;
    float xv[VEC], av[VEC], rv[VEC];
    if (VEC == 4) {
        if (OP != OP_FILL_ROW) *reinterpret_cast<float4 *>(xv) = *reinterpret_cast<const float4 *>(x + i);
        if (OP == OP_ADD || OP == OP_MULADD_ROW) *reinterpret_cast<float4 *>(av) = *reinterpret_cast<const float4 *>(a + i);
        if (OP == OP_ADD_ROW || OP == OP_MULADD_ROW || OP == OP_FILL_ROW)
            *reinterpret_cast<float4 *>(rv) = *reinterpret_cast<const float4 *>(row + i % dim);
    } else {
        if (OP != OP_FILL_ROW) xv[0] = x[i];
        if (OP == OP_ADD || OP == OP_MULADD_ROW) av[0] = a[i];
        if (OP == OP_ADD_ROW || OP == OP_MULADD_ROW || OP == OP_FILL_ROW) rv[0] = row[i % dim];
    }
#pragma unroll
    for (int j = 0; j < VEC; j++) {
        if (OP == OP_SILU) xv[j] = silu(xv[j]);
        if (OP == OP_ADD) xv[j] += av[j];
        if (OP == OP_ADD_ROW) xv[j] += rv[j];
        if (OP == OP_MULADD_ROW) xv[j] = fmaf(rv[j], av[j], xv[j]);
        if (OP == OP_FILL_ROW) xv[j] = rv[j];
    }
    if (VEC == 4) *reinterpret_cast<float4 *>(x + i) = *reinterpret_cast<float4 *>(xv);
    else x[i] = xv[0];
}

inline bool al16(const void *p) { return p == nullptr || ((uintptr_t)p & 15) == 0; }

template <int OP>
int launch_ew(hipStream_t st, float *x, const float *a, const float *row, int dim, size_t n) {
    if (!n) return 0;
    const bool vec = al16(x) && al16(a) && al16(row) && n % 4 == 0 && (dim <= 0 || dim % 4 == 0);
    if (vec) hipLaunchKernelGGL((k_ew<OP, 4>), dim3(blocks_for(n, EW_THREADS * 4)), dim3(EW_THREADS), 0, st, x, a, row, dim > 0 ? dim : 4, n);
    else hipLaunchKernelGGL((k_ew<OP, 1>), dim3(blocks_for(n, EW_THREADS)), dim3(EW_THREADS), 0, st, x, a, row, dim > 0 ? dim : 1, n);
    return (int)hipGetLastError();
}

template <int VEC>
__global__ void __launch_bounds__(EW_THREADS)
k_f32_to_bf16(uint16_t *__restrict__ dst, const float *__restrict__ src, size_t n) {
    const size_t i = ((size_t)blockIdx.x * EW_THREADS + threadIdx.x) * VEC;
    if (i >= n) return;
    if (VEC == 8) {
        const float4 a = *reinterpret_cast<const float4 *>(src + i), b = *reinterpret_cast<const float4 *>(src + i + 4);
        *reinterpret_cast<uint4 *>(dst + i) = make_uint4(pack_bf16(a.x, a.y), pack_bf16(a.z, a.w), pack_bf16(b.x, b.y), pack_bf16(b.z, b.w));
    } else {
        dst[i] = to_bf16(src[i]);
    }
}

/* out[r, c] = silu(gate[r, c]) * up[r, c] on bf16 rows with strides */
template <int VEC>
__global__ void __launch_bounds__(EW_THREADS)
k_swiglu(uint16_t *__restrict__ out, int ldo, const uint16_t *__restrict__ gate, const uint16_t *__restrict__ up,
         int ldi, int cols, size_t n) {
    const size_t i = ((size_t)blockIdx.x * EW_THREADS + threadIdx.x) * VEC;
    if (i >= n) return;
    const size_t r = i / cols, c = i % cols;
    if (VEC == 8) {
        const uint4 g = *reinterpret_cast<const uint4 *>(gate + r * ldi + c), u = *reinterpret_cast<const uint4 *>(up + r * ldi + c);
        const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w};
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 4; j++) o[j] = pack_bf16(silu(bf_lo(gw[j])) * bf_lo(uw[j]), silu(bf_hi(gw[j])) * bf_hi(uw[j]));
        *reinterpret_cast<uint4 *>(out + r * ldo + c) = make_uint4(o[0], o[1], o[2], o[3]);
    } else {
        const float g = bf_lo(gate[r * ldi + c]);
        out[r * ldo + c] = to_bf16(silu(g) * bf_lo(up[r * ldi + c]));
    }
}

/* nearest-neighbour 2x upsampling of a channels-last image */
template <int VEC>
__global__ void __launch_bounds__(EW_THREADS)
k_upsample2x(float *__restrict__ out, const float *__restrict__ in, int w, int c, size_t n) {
    const size_t i = ((size_t)blockIdx.x * EW_THREADS + threadIdx.x) * VEC;
    if (i >= n) return;
    const int ch = (int)(i % c);
    const size_t p = i / c;
    const int x = (int)(p % (2 * (size_t)w)), y = (int)(p / (2 * (size_t)w));
    const float *src = in + ((size_t)(y / 2) * w + x / 2) * c + ch;
    if (VEC == 4) *reinterpret_cast<float4 *>(out + i) = *reinterpret_cast<const float4 *>(src);
    else out[i] = *src;
}

/* ---------------------------------------------------------------- row normalisations */

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

__device__ __forceinline__ float block_sum(float v, float *sh) {
    v = wave_sum(v);
    const int wave = threadIdx.x >> 6;
    __syncthreads();                                  /* sh may still be read from the previous reduction */
    if ((threadIdx.x & 63) == 0) sh[wave] = v;
    __syncthreads();
    return sh[0] + sh[1] + sh[2] + sh[3];
}

enum NormKind { LAYER_NORM_MOD, RMS_NORM_MOD, RMS_NORM_RESIDUAL };
constexpr int ROW_VECS = 16;          /* float4 per lane kept in registers: rows up to 4096 floats */

/* One WAVE per row, four rows per workgroup: no LDS, no barrier. CACHE: dim % 4 == 0,
 * dim <= 4096, 16-byte aligned rows -> the row stays in registers between the statistics
 * and the write; otherwise it is read again. p0/p1 are (shift, scale) for LayerNorm,
 * (w, scale) for RMSNorm, (w, gate) for the residual form; out_bf is unused by the latter. */
template <int KIND, bool CACHE>
__global__ void __launch_bounds__(ROW_THREADS)
k_row_norm(uint16_t *__restrict__ out_bf, float *__restrict__ xres, const float *__restrict__ src,
           const float *__restrict__ p0, const float *__restrict__ p1, int rows, int dim, float eps) {
    const int row = blockIdx.x * (ROW_THREADS / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int lane = threadIdx.x & 63;
    const float *xr = src + (size_t)row * dim;
    float4 keep[ROW_VECS];
    const int nvec = dim >> 2;

    float s = 0.0f;
    if (CACHE) {
#pragma unroll
        for (int j = 0; j < ROW_VECS; j++) {
            const int v = lane + j * 64;
            keep[j] = v < nvec ? *reinterpret_cast<const float4 *>(xr + 4 * v) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (KIND == LAYER_NORM_MOD) s += (keep[j].x + keep[j].y) + (keep[j].z + keep[j].w);
            else s += (keep[j].x * keep[j].x + keep[j].y * keep[j].y) + (keep[j].z * keep[j].z + keep[j].w * keep[j].w);
        }
    } else {
        for (int i = lane; i < dim; i += 64) s += KIND == LAYER_NORM_MOD ? xr[i] : xr[i] * xr[i];
    }
    s = wave_sum(s);
    float mean = 0.0f, inv;
    if (KIND == LAYER_NORM_MOD) {
        mean = s / (float)dim;
        float v = 0.0f;
        if (CACHE) {
#pragma unroll
            for (int j = 0; j < ROW_VECS; j++)
                if (lane + j * 64 < nvec) {
                    const float a = keep[j].x - mean, b = keep[j].y - mean, c = keep[j].z - mean, d = keep[j].w - mean;
                    v += (a * a + b * b) + (c * c + d * d);
                }
        } else {
            for (int i = lane; i < dim; i += 64) { const float d = xr[i] - mean; v += d * d; }
        }
        inv = 1.0f / sqrtf(wave_sum(v) / (float)dim + eps);
    } else {
        inv = 1.0f / sqrtf(s / (float)dim + eps);
    }

    const size_t row_off = (size_t)row * dim;
    if (CACHE) {
#pragma unroll
        for (int j = 0; j < ROW_VECS; j++) {
            const int v = lane + j * 64;
            if (v >= nvec) continue;
            const float xin[4] = {keep[j].x, keep[j].y, keep[j].z, keep[j].w};
            float4 a = *reinterpret_cast<const float4 *>(KIND == LAYER_NORM_MOD ? (p1 ? p1 : xr) + 4 * v : p0 + 4 * v);   /* scale | w */
            float4 b = *reinterpret_cast<const float4 *>((KIND == LAYER_NORM_MOD ? (p0 ? p0 : xr) : (p1 ? p1 : xr)) + 4 * v);   /* shift | scale/gate */
            const float av[4] = {a.x, a.y, a.z, a.w}, bv[4] = {b.x, b.y, b.z, b.w};
            float r[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                if (KIND == LAYER_NORM_MOD) {
                    float n = (xin[e] - mean) * inv;
                    if (p1) n *= 1.0f + av[e];
                    if (p0) n += bv[e];
                    r[e] = n;
                } else {
                    float t = xin[e] * inv * av[e];
                    if (KIND == RMS_NORM_MOD) { if (p1) t *= 1.0f + bv[e]; }
                    else t *= p1 ? tanhf(bv[e]) : 1.0f;
                    r[e] = t;
                }
            }
            if (KIND == RMS_NORM_RESIDUAL) {
                float4 t = *reinterpret_cast<float4 *>(xres + row_off + 4 * v);
                t.x += r[0]; t.y += r[1]; t.z += r[2]; t.w += r[3];
                *reinterpret_cast<float4 *>(xres + row_off + 4 * v) = t;
            } else {
                *reinterpret_cast<uint2 *>(out_bf + row_off + 4 * v) = make_uint2(pack_bf16(r[0], r[1]), pack_bf16(r[2], r[3]));
            }
        }
    } else {
        for (int i = lane; i < dim; i += 64) {
            float r;
            if (KIND == LAYER_NORM_MOD) {
                r = (xr[i] - mean) * inv;
                if (p1) r *= 1.0f + p1[i];
                if (p0) r += p0[i];
            } else {
                r = xr[i] * inv * p0[i];
                if (KIND == RMS_NORM_MOD) { if (p1) r *= 1.0f + p1[i]; }
                else r *= p1 ? tanhf(p1[i]) : 1.0f;
            }
            if (KIND == RMS_NORM_RESIDUAL) xres[row_off + i] += r;
            else out_bf[row_off + i] = to_bf16(r);
        }
    }
}

template <int KIND>
int launch_row_norm(hipStream_t st, uint16_t *out_bf, float *xres, const float *src, const float *p0,
                    const float *p1, int rows, int dim, float eps) {
    if (rows <= 0 || dim <= 0) return 0;
    const bool cache = dim % 4 == 0 && dim <= 4 * 64 * ROW_VECS && al16(src) && al16(xres) && al16(p0) && al16(p1) &&
                       ((uintptr_t)out_bf & 7) == 0;
    const unsigned blocks = (unsigned)((rows + ROW_THREADS / 64 - 1) / (ROW_THREADS / 64));
    if (cache) hipLaunchKernelGGL((k_row_norm<KIND, true>), dim3(blocks), dim3(ROW_THREADS), 0, st, out_bf, xres, src, p0, p1, rows, dim, eps);
    else hipLaunchKernelGGL((k_row_norm<KIND, false>), dim3(blocks), dim3(ROW_THREADS), 0, st, out_bf, xres, src, p0, p1, rows, dim, eps);
    return (int)hipGetLastError();
}

/* ---------------------------------------------------------------- group norm
 *
 * Two passes over the image in all: one for the statistics, one that normalises.
 *
 * Statistics in ONE pass: a thread sums (x - K) and (x - K)^2 over its share of a group, K being
 * the first value it reads. K is a sample of the data, so the sums stay of the size of the
 * spread and the cancellation that plain sum / sum-of-squares formulas suffer does not arise.
 * Each thread's (count, mean, M2) is then merged with the others' by the pairwise update of the
 * parallel variance algorithm: inside the workgroup in f32, across workgroups in double.
 * (The reference reads the image twice for the statistics, mean first and then the squared
 * deviations, iris_cuda.cu:1069-1074; the merged single pass gives the same moments to f32
 * rounding.) */

constexpr int GN_MAX_BLOCKS = 1024;      /* partial moments per group */

struct Moments { float n, mean, m2; };

__device__ __forceinline__ void merge(Moments &a, const Moments b) {
    if (b.n == 0.0f) return;
    const float n = a.n + b.n, d = b.mean - a.mean;
    a.mean += d * (b.n / n);
    a.m2 += b.m2 + d * d * (a.n * b.n / n);
    a.n = n;
}

/* from sums shifted by k */
__device__ __forceinline__ Moments from_shifted(float n, float k, float s, float ss) {
    Moments m = {n, 0.0f, 0.0f};
    if (n > 0.0f) { m.mean = k + s / n; m.m2 = fmaxf(ss - s * s / n, 0.0f); }
    return m;
}

/* part[(g * nblocks + b)] = moments of group g over the pixels of block b. Coalesced form: needs
 * c % 4 == 0, cg % 4 == 0 and (c / 4) dividing 256; a thread keeps one quad of channels (inside
 * one group), the workgroup walks 256 / (c / 4) pixels per step with 16-byte loads. */
__global__ void __launch_bounds__(ROW_THREADS)
k_gn_moments_quads(Moments *__restrict__ part, const float *__restrict__ in, int hw, int c, int cg, int per_block) {
    __shared__ Moments sh[ROW_THREADS];
    const int quads = c >> 2, ppi = ROW_THREADS / quads;      /* pixels per iteration */
    const int q = threadIdx.x % quads, sub = threadIdx.x / quads;
    const int start = blockIdx.x * per_block, end = min(start + per_block, hw);
    float n = 0.0f, k = 0.0f, s = 0.0f, ss = 0.0f;
    int p = start + sub;
    if (p < end) k = in[(size_t)p * c + 4 * q];
    for (; p < end; p += ppi) {
        const float4 v = *reinterpret_cast<const float4 *>(in + (size_t)p * c + 4 * q);
        const float a0 = v.x - k, a1 = v.y - k, a2 = v.z - k, a3 = v.w - k;
        s += (a0 + a1) + (a2 + a3);
        ss += (a0 * a0 + a1 * a1) + (a2 * a2 + a3 * a3);
        n += 4.0f;
    }
    sh[threadIdx.x] = from_shifted(n, k, s, ss);
    __syncthreads();
    const int groups = c / cg, qpg = cg >> 2;
    if ((int)threadIdx.x < groups) {
        Moments t = {0.0f, 0.0f, 0.0f};
        for (int sb = 0; sb < ppi; sb++)
            for (int j = 0; j < qpg; j++) merge(t, sh[sb * quads + threadIdx.x * qpg + j]);
        part[(size_t)threadIdx.x * gridDim.x + blockIdx.x] = t;
    }
}

/* Any shape: one workgroup per (group, block), scalar strided reads. */
__global__ void __launch_bounds__(ROW_THREADS)
k_gn_moments_any(Moments *__restrict__ part, const float *__restrict__ in, int hw, int c, int cg) {
    __shared__ Moments sh[ROW_THREADS];
    const int g = blockIdx.x, b = blockIdx.y;
    const size_t total = (size_t)hw * cg;
    const size_t per_block = (total + gridDim.y - 1) / gridDim.y;
    const size_t start = (size_t)b * per_block, end = start + per_block < total ? start + per_block : total;
    float n = 0.0f, k = 0.0f, s = 0.0f, ss = 0.0f;
    for (size_t i = start + threadIdx.x; i < end; i += ROW_THREADS) {
        const float v = in[(i / cg) * c + (size_t)g * cg + i % cg];
        if (n == 0.0f) k = v;
        const float a = v - k;
        s += a; ss += a * a; n += 1.0f;
    }
    sh[threadIdx.x] = from_shifted(n, k, s, ss);
    __syncthreads();
    for (int half = ROW_THREADS / 2; half > 0; half >>= 1) {
        if ((int)threadIdx.x < half) merge(sh[threadIdx.x], sh[threadIdx.x + half]);
        __syncthreads();
    }
    if (threadIdx.x == 0) part[(size_t)g * gridDim.y + b] = sh[0];
}

/* stats[g] = mean, stats[groups + g] = 1 / sqrt(var + eps) from the workgroups' partial moments, in double, one
 * workgroup per group: the mean is the count-weighted mean of the partial means, the sum of squared deviations is
 * the sum of the partial ones plus count x (partial mean - mean)^2 -- the same combination as the pairwise
 * merge, written so that it takes two sums over the partials and a single division. */
__device__ __forceinline__ double wave_sum64(double v) {
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

/* one workgroup of 256 threads per group; a thread holds up to GN_MAX_BLOCKS / 256 partials, loaded together */
__device__ __forceinline__ double block_sum64(double v, double *sh) {
    v = wave_sum64(v);
    __syncthreads();                                   /* sh may still be read from the previous call */
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = v;
    __syncthreads();
    return (sh[0] + sh[1]) + (sh[2] + sh[3]);
}

__global__ void __launch_bounds__(256)
k_gn_finish(float *__restrict__ stats, const Moments *__restrict__ part, int groups, int nblocks, float eps) {
    __shared__ double sh[4];
    constexpr int PER = GN_MAX_BLOCKS / 256;
    const int g = blockIdx.x;
    Moments m[PER];
#pragma unroll
    for (int i = 0; i < PER; i++) {
        const int b = threadIdx.x + 256 * i;
        m[i] = b < nblocks ? part[(size_t)g * nblocks + b] : Moments{0.0f, 0.0f, 0.0f};
    }
    double n = 0.0, weighted = 0.0;
#pragma unroll
    for (int i = 0; i < PER; i++) { n += (double)m[i].n; weighted += (double)m[i].n * (double)m[i].mean; }
    n = block_sum64(n, sh);
    const double mean = n > 0.0 ? block_sum64(weighted, sh) / n : 0.0;
    double m2 = 0.0;
#pragma unroll
    for (int i = 0; i < PER; i++) {
        const double d = (double)m[i].mean - mean;
        m2 += (double)m[i].m2 + (double)m[i].n * d * d;
    }
    m2 = block_sum64(m2, sh);
    if (threadIdx.x == 0) {
        stats[g] = (float)mean;
        stats[groups + g] = (float)(1.0 / sqrt((n > 0.0 ? m2 / n : 0.0) + (double)eps));
    }
}

/* out = (x - mean[g]) * rstd[g] * gamma[ch] + beta[ch], optionally through SiLU. VEC = 4: a thread's four
 * channels are one aligned quad, which lies inside one group (c % 4 == 0 and cg % 4 == 0) or, when
 * cg % 4 != 0, is looked up channel by channel. */
template <int VEC>
__global__ void __launch_bounds__(EW_THREADS)
k_gn_normalize(float *__restrict__ out, const float *__restrict__ in, const float *__restrict__ stats,
               const float *__restrict__ gamma, const float *__restrict__ beta, int c, int cg, int groups,
               int do_silu, size_t n) {
    const size_t i = ((size_t)blockIdx.x * EW_THREADS + threadIdx.x) * VEC;
    if (i >= n) return;
    const int ch0 = (int)(i % (size_t)c);
    float v[VEC], ga[VEC], be[VEC];
    if (VEC == 4) {
        *reinterpret_cast<float4 *>(v) = *reinterpret_cast<const float4 *>(in + i);
        *reinterpret_cast<float4 *>(ga) = *reinterpret_cast<const float4 *>(gamma + ch0);
        *reinterpret_cast<float4 *>(be) = *reinterpret_cast<const float4 *>(beta + ch0);
    } else {
        v[0] = in[i]; ga[0] = gamma[ch0]; be[0] = beta[ch0];
    }
    const bool one_group = VEC == 1 || cg % 4 == 0;
    const int g0 = ch0 / cg;
    const float mean0 = stats[g0], rstd0 = stats[groups + g0];
#pragma unroll
    for (int j = 0; j < VEC; j++) {
        float mean = mean0, rstd = rstd0;
        if (!one_group) { const int g = (ch0 + j) / cg; mean = stats[g]; rstd = stats[groups + g]; }
        const float y = (v[j] - mean) * rstd * ga[j] + be[j];
        v[j] = do_silu ? silu(y) : y;
    }
    if (VEC == 4) *reinterpret_cast<float4 *>(out + i) = *reinterpret_cast<float4 *>(v);
    else out[i] = v[0];
}

}  // namespace

extern "C" {

int iris_hip_f32_to_bf16(void *stream, uint16_t *dst, const float *src, size_t n) {
    if (!n) return 0;
    hipStream_t st = (hipStream_t)stream;
    if (al16(dst) && al16(src) && n % 8 == 0)
        hipLaunchKernelGGL(k_f32_to_bf16<8>, dim3(blocks_for(n, EW_THREADS * 8)), dim3(EW_THREADS), 0, st, dst, src, n);
    else
        hipLaunchKernelGGL(k_f32_to_bf16<1>, dim3(blocks_for(n, EW_THREADS)), dim3(EW_THREADS), 0, st, dst, src, n);
    return (int)hipGetLastError();
}

int iris_hip_silu(void *stream, float *x, size_t n) { return launch_ew<OP_SILU>((hipStream_t)stream, x, nullptr, nullptr, 0, n); }
int iris_hip_add(void *stream, float *x, const float *a, size_t n) { return launch_ew<OP_ADD>((hipStream_t)stream, x, a, nullptr, 0, n); }
int iris_hip_add_bias(void *stream, float *y, const float *bias, int rows, int cols) {
    return launch_ew<OP_ADD_ROW>((hipStream_t)stream, y, nullptr, bias, cols, (size_t)rows * cols);
}
int iris_hip_fill_rows(void *stream, float *out, const float *row, int rows, int dim) {
    return launch_ew<OP_FILL_ROW>((hipStream_t)stream, out, nullptr, row, dim, (size_t)rows * dim);
}
/* x[r, c] += gate[c] * a[r, c], gate may be NULL */
int iris_hip_residual(void *stream, float *x, const float *a, const float *gate, int rows, int dim) {
    if (!gate) return launch_ew<OP_ADD>((hipStream_t)stream, x, a, nullptr, 0, (size_t)rows * dim);
    return launch_ew<OP_MULADD_ROW>((hipStream_t)stream, x, a, gate, dim, (size_t)rows * dim);
}

int iris_hip_swiglu(void *stream, uint16_t *out, int ldo, const uint16_t *gate, const uint16_t *up, int ldi,
                    int rows, int cols) {
    const size_t n = (size_t)rows * cols;
    if (!n) return 0;
    hipStream_t st = (hipStream_t)stream;
    if (al16(out) && al16(gate) && al16(up) && cols % 8 == 0 && ldi % 8 == 0 && ldo % 8 == 0)
        hipLaunchKernelGGL(k_swiglu<8>, dim3(blocks_for(n, EW_THREADS * 8)), dim3(EW_THREADS), 0, st, out, ldo, gate, up, ldi, cols, n);
    else
        hipLaunchKernelGGL(k_swiglu<1>, dim3(blocks_for(n, EW_THREADS)), dim3(EW_THREADS), 0, st, out, ldo, gate, up, ldi, cols, n);
    return (int)hipGetLastError();
}

int iris_hip_upsample2x(void *stream, float *out, const float *in, int h, int width, int c) {
    const size_t n = (size_t)4 * h * width * c;
    if (!n) return 0;
    hipStream_t st = (hipStream_t)stream;
    if (al16(out) && al16(in) && c % 4 == 0)
        hipLaunchKernelGGL(k_upsample2x<4>, dim3(blocks_for(n, EW_THREADS * 4)), dim3(EW_THREADS), 0, st, out, in, width, c, n);
    else
        hipLaunchKernelGGL(k_upsample2x<1>, dim3(blocks_for(n, EW_THREADS)), dim3(EW_THREADS), 0, st, out, in, width, c, n);
    return (int)hipGetLastError();
}

int iris_hip_layer_norm_mod(void *stream, uint16_t *out, const float *x, const float *shift, const float *scale,
                            int rows, int dim, float eps) {
    return launch_row_norm<LAYER_NORM_MOD>((hipStream_t)stream, out, nullptr, x, shift, scale, rows, dim, eps);
}
int iris_hip_rms_norm_mod(void *stream, uint16_t *out, const float *x, const float *w, const float *scale,
                          int rows, int dim, float eps) {
    return launch_row_norm<RMS_NORM_MOD>((hipStream_t)stream, out, nullptr, x, w, scale, rows, dim, eps);
}
int iris_hip_rms_norm_residual(void *stream, float *x, const float *a, const float *w, const float *gate,
                               int rows, int dim, float eps) {
    return launch_row_norm<RMS_NORM_RESIDUAL>((hipStream_t)stream, nullptr, x, a, w, gate, rows, dim, eps);
}

size_t iris_hip_group_norm_scratch_floats(int groups) { return 3 * (size_t)groups * GN_MAX_BLOCKS + 2 * (size_t)groups; }

/* scratch: iris_hip_group_norm_scratch_floats(groups) floats of device memory. Every slot a call
 * reads (partial moments [group][workgroup], statistics [2][group]) is written by that call first. */
int iris_hip_group_norm(void *stream, float *scratch, float *out, const float *in, const float *gamma,
                        const float *beta, int hw, int c, int groups, float eps, int do_silu) {
    if (hw <= 0 || c <= 0) return 0;
    hipStream_t st = (hipStream_t)stream;
    Moments *part = reinterpret_cast<Moments *>(scratch);
    float *stats = scratch + 3 * (size_t)groups * GN_MAX_BLOCKS;
    const int cg = c / groups;
    const bool quads_form = c % 4 == 0 && cg % 4 == 0 && c / 4 <= ROW_THREADS && ROW_THREADS % (c / 4) == 0 && al16(in);
    int nblocks;
    if (quads_form) {
        const int ppi = ROW_THREADS / (c / 4);
        nblocks = (hw + ppi - 1) / ppi;                         /* at least one step of the workgroup per block */
        if (nblocks > GN_MAX_BLOCKS) nblocks = GN_MAX_BLOCKS;
        const int per_block = (hw + nblocks - 1) / nblocks;
        nblocks = (hw + per_block - 1) / per_block;
        hipLaunchKernelGGL(k_gn_moments_quads, dim3(nblocks), dim3(ROW_THREADS), 0, st, part, in, hw, c, cg, per_block);
    } else {
        const size_t total = (size_t)hw * cg;
        nblocks = (int)((total + 4 * ROW_THREADS - 1) / (4 * ROW_THREADS));
        if (nblocks > GN_MAX_BLOCKS) nblocks = GN_MAX_BLOCKS;
        hipLaunchKernelGGL(k_gn_moments_any, dim3(groups, nblocks), dim3(ROW_THREADS), 0, st, part, in, hw, c, cg);
    }
    hipLaunchKernelGGL(k_gn_finish, dim3(groups), dim3(256), 0, st, stats, part, groups, nblocks, eps);
    const size_t n = (size_t)hw * c;
    if (al16(out) && al16(in) && al16(gamma) && al16(beta) && c % 4 == 0)
        hipLaunchKernelGGL(k_gn_normalize<4>, dim3(blocks_for(n, EW_THREADS * 4)), dim3(EW_THREADS), 0, st, out, in, stats, gamma, beta, c, cg, groups, do_silu, n);
    else
        hipLaunchKernelGGL(k_gn_normalize<1>, dim3(blocks_for(n, EW_THREADS)), dim3(EW_THREADS), 0, st, out, in, stats, gamma, beta, c, cg, groups, do_silu, n);
    return (int)hipGetLastError();
}

}  // extern "C"

/* ---- group norm for callers that cannot allocate -------------------------------------------
 * The same kernels with their scratch in a device array that is part of the library image, so the
 * call needs no hipMalloc: each GPU holds its own copy of the array, at its own address, until the
 * process ends. In host code the array's name is only a handle for hipGetSymbolAddress; kernels
 * get the address that call returned, kept per device. Calls on one GPU share the array: they must
 * not overlap (the library issues everything on one stream, which orders them). */
constexpr int GN_STATIC_MAX_GROUPS = 64;
constexpr size_t GN_STATIC_FLOATS = 3 * (size_t)GN_STATIC_MAX_GROUPS * GN_MAX_BLOCKS + 2 * (size_t)GN_STATIC_MAX_GROUPS;
static __device__ __align__(256) float scratch[GN_STATIC_FLOATS];          /* 786,944 B */

constexpr int GN_STATIC_MAX_DEVICES = 64;
static float *scratch_address[GN_STATIC_MAX_DEVICES];                        /* per device; null = not looked up yet */

extern "C" {

int iris_hip_group_norm_static_max_groups(void) { return GN_STATIC_MAX_GROUPS; }

/* Looks up the address of the current device's copy of the array (once per device). */
int iris_hip_group_norm_static_setup(void) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= GN_STATIC_MAX_DEVICES) return (int)hipErrorInvalidDevice;
    if (scratch_address[dev]) return 0;
    float *p = nullptr;
    e = hipGetSymbolAddress(reinterpret_cast<void **>(&p), HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!p) return (int)hipErrorInvalidSymbol;
    scratch_address[dev] = p;
    return 0;
}

/* groups <= iris_hip_group_norm_static_max_groups(), checked by the caller too */
int iris_hip_group_norm_static(void *stream, float *out, const float *in, const float *gamma,
                               const float *beta, int hw, int c, int groups, float eps, int do_silu) {
    if (groups <= 0 || groups > GN_STATIC_MAX_GROUPS) return (int)hipErrorInvalidValue;
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= GN_STATIC_MAX_DEVICES) return (int)hipErrorInvalidDevice;
    if (!scratch_address[dev]) {                         /* first call on a device the set-up call did not see */
        const int rc = iris_hip_group_norm_static_setup();
        if (rc) return rc;
    }
    return iris_hip_group_norm(stream, scratch_address[dev], out, in, gamma, beta, hw, c, groups, eps, do_silu);
}

}  // extern "C"
