/*
 * C-callable launchers of the HIP kernels (defined in the .hip files, called
 * from iris_rocm.c). Each enqueues on `stream` and returns the hipError_t of
 * the launch as an int (0 = success). Shapes are checked by the caller:
 * launchers assume what their comment states.
 */
#ifndef IRIS_KERNELS_HIP_H
#define IRIS_KERNELS_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Fused per-head RMSNorm + RoPE, head_dim 128, on one or two tensors that
 * share rows. Requires: xq (and xk if k_heads > 0) 16-byte aligned,
 * ld % 8 == 0, w / cos / sin 16-byte aligned, seq * (q_heads + k_heads) < 2^24. */
int iris_hip_norm_rope_hd128(void *stream, uint16_t *xq, uint16_t *xk, int ld,
                             const float *wq, const float *wk,
                             const float *rope_cos, const float *rope_sin,
                             int seq, int q_heads, int k_heads, float eps, int split_half);

/* Any even head_dim <= 1024, any alignment. One wave per (token, head). */
int iris_hip_norm_rope_generic(void *stream, uint16_t *x, int ld, const float *w,
                               const float *rope_cos, const float *rope_sin,
                               int seq, int heads, int head_dim, float eps, int split_half);

/* Flash attention forward, head_dim 128, bf16 MFMA. Requires: q/k/v 16-byte
 * aligned, ldi % 8 == 0, out 8-byte aligned, ldo % 4 == 0, scale > 0,
 * heads % kv_heads == 0, seq_q > 0, seq_k > 0. */
int iris_hip_fa_hd128(void *stream, uint16_t *out, int ldo, const uint16_t *q,
                      const uint16_t *k, const uint16_t *v, int ldi, int seq_q, int seq_k,
                      int heads, int kv_heads, float scale, int causal, const int *key_mask);

/* head_dim 256 or 512 (the VAE's single 512-wide head): the head dim is cut into slices of
 * 128 that a group of waves shares; same argument conditions as iris_hip_fa_hd128. */
int iris_hip_fa_sliced(void *stream, uint16_t *out, int ldo, const uint16_t *q,
                       const uint16_t *k, const uint16_t *v, int ldi, int seq_q, int seq_k,
                       int heads, int kv_heads, int head_dim, float scale, int causal,
                       const int *key_mask);

/* Any head_dim <= 512, any stride / alignment / scale. Correctness path. */
int iris_hip_attention_generic(void *stream, uint16_t *out, int ldo, const uint16_t *q,
                               const uint16_t *k, const uint16_t *v, int ldi, int seq_q,
                               int seq_k, int heads, int kv_heads, int head_dim, float scale,
                               int causal, const int *key_mask);

#ifdef __cplusplus
}
#endif
#endif
