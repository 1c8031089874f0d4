/*
 * The arithmetic of the per-head RMSNorm + rotary embedding for head_dim 128
 * (reference iris_cuda.cu:402-420), one operation per function. The
 * stand-alone kernel (qknorm_rope.hip) and the attention kernel's Q load
 * (fa_fwd_gfx950.hip) both go through these, with explicit fused
 * multiply-adds, so that the two produce the same bits: a vector is handled in
 * 16 chunks of 8 consecutive dims; the sum of squares of chunk c is a chain of
 * fused multiply-adds from 0, and the chunk sums p[c] are added as
 *     t[c] = p[c] + p[c+8],  u[c] = t[c] + t[c+4],  w[c] = u[c] + u[c+2],
 *     total = w[0] + w[1]
 * (the rotate-and-add tree over a 16-lane row; every addition is commutative,
 * so the order of the two operands is free).
 */
#ifndef IRIS_NORM_ROPE_MATH_H
#define IRIS_NORM_ROPE_MATH_H

__device__ __forceinline__ float nr_chunk_sum_squares(const float (&e)[8]) {
    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; i++) ss = fmaf(e[i], e[i], ss);
    return ss;
}

__device__ __forceinline__ float nr_inv_rms128(float sum_squares, float eps) {
    return 1.0f / sqrtf(fmaf(sum_squares, 1.0f / 128.0f, eps));
}

/* x * r * w with the two factors of the row combined first */
__device__ __forceinline__ float nr_scaled(float x, float inv, float w) { return x * (inv * w); }

/* the pair (a, b) rotated by (c, s): a*c - b*s and b*c + a*s */
__device__ __forceinline__ float nr_rot_first(float a, float b, float c, float s) { return fmaf(-b, s, a * c); }
__device__ __forceinline__ float nr_rot_second(float a, float b, float c, float s) { return fmaf(a, s, b * c); }

/* ---- one (token, head) vector held by the 16 lanes of a DPP row, 16 B (8 dims) per lane ----
 * Shared by the stand-alone kernel and by the projection that normalises its own output tile, so that
 * the two store the same bits. */
typedef unsigned int nr_u32x4 __attribute__((ext_vector_type(4)));
typedef float nr_f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 nr_bf16x2 __attribute__((ext_vector_type(2)));

/* Two f32 -> packed bf16x2, round to nearest even (v_cvt_pk_bf16_f32; equals the integer form
 * u += 0x7fff + ((u >> 16) & 1) for every finite input). */
__device__ __forceinline__ unsigned int nr_pack_bf16(float lo, float hi) {
    nr_f32x2 p = {lo, hi};
    return __builtin_bit_cast(unsigned int, __builtin_convertvector(p, nr_bf16x2));
}

/* Sum over the 16 lanes of a DPP row; every lane gets the total. */
__device__ __forceinline__ float nr_row16_sum(float v) {
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xf, 0xf, false));
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124, 0xf, 0xf, false));
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x122, 0xf, 0xf, false));
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x121, 0xf, 0xf, false));
    return v;
}

/* The value held by the lane 8 places away in the same 16-lane row. */
__device__ __forceinline__ float nr_row16_partner8(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xf, 0xf, false));
}

/* raw: this lane's 8 bf16 (dims 8 sub .. 8 sub + 7); w8: the norm weights of those dims; cv / sv: the
 * table entries this lane needs -- consecutive pairs: columns 4 sub .. 4 sub + 3 in cv[0..3]; split halves:
 * columns 8 (sub % 8) .. + 7 in cv[0..7] (shared with the partner lane 8 away). All 16 lanes of the row
 * must be active. Returns the normalised, rotated 8 bf16. */
template <bool SPLIT>
__device__ __forceinline__ nr_u32x4 nr_vector_hd128(nr_u32x4 raw, const float (&w8)[8], const float (&cv)[8],
                                                    const float (&sv)[8], float eps, int sub) {
    float e[8] = {__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u), __uint_as_float(raw.y << 16),
                  __uint_as_float(raw.y & 0xffff0000u), __uint_as_float(raw.z << 16), __uint_as_float(raw.z & 0xffff0000u),
                  __uint_as_float(raw.w << 16), __uint_as_float(raw.w & 0xffff0000u)};
    const float ss = nr_row16_sum(nr_chunk_sum_squares(e));
    const float inv = nr_inv_rms128(ss, eps);
#pragma unroll
    for (int i = 0; i < 8; i++) e[i] = nr_scaled(e[i], inv, w8[i]);
    float o[8];
    if (SPLIT) {
        /* lanes 0-7 hold a (first half), lanes 8-15 hold b: a*c - b*s / b*c + a*s, i.e. nr_rot_first(e, other)
         * on the a lanes and nr_rot_second(other, e) on the b lanes as one expression: the sign flip is exact */
        const float sgn = sub < 8 ? -1.0f : 1.0f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const float other = nr_row16_partner8(e[i]);
            o[i] = fmaf(sgn * other, sv[i], e[i] * cv[i]);
        }
    } else {
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const float a = e[2 * p], b = e[2 * p + 1];
            o[2 * p] = nr_rot_first(a, b, cv[p], sv[p]);
            o[2 * p + 1] = nr_rot_second(a, b, cv[p], sv[p]);
        }
    }
    nr_u32x4 out;
    out.x = nr_pack_bf16(o[0], o[1]);
    out.y = nr_pack_bf16(o[2], o[3]);
    out.z = nr_pack_bf16(o[4], o[5]);
    out.w = nr_pack_bf16(o[6], o[7]);
    return out;
}

#endif
