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

#endif
