/*
 * C-callable launchers of the HIP kernels (defined in the .hip files, called
 * from iris_rocm.c). Each enqueues on `stream` and returns the hipError_t of
 * the launch as an int (0 = success). Shapes are checked by the caller:
 * launchers assume what their comment states.
 */
#ifndef IRIS_KERNELS_HIP_H
#define IRIS_KERNELS_HIP_H

#include <stddef.h>
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

/* The same with a second weight pair (wq_b, wk_b) for the rows from rows_a on (wq_b NULL: one pair for all rows).
 * Calls that touch 128 MB of rows or more store with the streaming hint (iris_norm_rope_streaming_stores). */
int iris_hip_norm_rope_hd128_streams(void *stream, uint16_t *xq, uint16_t *xk, int ld,
                                     const float *wq, const float *wk, const float *wq_b, const float *wk_b,
                                     int rows_a, const float *rope_cos, const float *rope_sin,
                                     int seq, int q_heads, int k_heads, float eps, int split_half);
int iris_norm_rope_streaming_stores(int seq, int heads_total);

/* The multiplier the kernel above divides by heads_total with (0 for one head, which needs
 * none). Exported for the host-side test of the division. */
uint32_t iris_norm_rope_magic(int heads_total);

/* Any even head_dim <= 1024, any alignment. One wave per (token, head). */
int iris_hip_norm_rope_generic(void *stream, uint16_t *x, int ld, const float *w,
                               const float *rope_cos, const float *rope_sin,
                               int seq, int heads, int head_dim, float eps, int split_half);

/* Flash attention forward, head_dim 128, bf16 MFMA. Requires: q/k/v 16-byte
 * aligned, ldi % 8 == 0, out 8-byte aligned, ldo % 4 == 0, scale > 0,
 * heads % kv_heads == 0, seq_q > 0, seq_k > 0, and with a key mask
 * seq_k <= IRIS_FA_MAX_MASKED_KEYS (the mask is kept in LDS as one bit per key). */
#define IRIS_FA_MAX_MASKED_KEYS 250000
int iris_hip_fa_hd128(void *stream, uint16_t *out, int ldo, const uint16_t *q,
                      const uint16_t *k, const uint16_t *v, int ldi, int seq_q, int seq_k,
                      int heads, int kv_heads, float scale, int causal, const int *key_mask);

/* The same with the per-head RMSNorm + rotary embedding of Q (weights w[128], tables
 * [seq_q, 64], all 16-byte aligned) applied while Q is loaded; q itself is only read. The Q
 * operand has the bits that iris_hip_norm_rope_hd128 would have stored. */
int iris_hip_fa_hd128_qnorm(void *stream, uint16_t *out, int ldo, const uint16_t *q,
                            const uint16_t *k, const uint16_t *v, int ldi, int seq_q, int seq_k,
                            int heads, int kv_heads, float scale, int causal, const int *key_mask,
                            const float *w, const float *rope_cos, const float *rope_sin, float eps,
                            int split_half);

/* What iris_hip_fa_hd128 would launch for these sizes, host arithmetic only (no GPU needed): plan[0] = 0 one size
 * of workgroup, 1 two sizes (256 queries, then 192), 2 keys split over the waves of a workgroup; plan[1] = waves per
 * workgroup; plan[2] = blocks of 16 queries per wave; plan[3], plan[4] = 256- and 192-query workgroups per head of
 * the two-size grid. */
void iris_hip_fa_hd128_plan(int seq_q, int seq_k, int heads, int causal, int *plan);

/* head_dim 512 (the VAE's call; key mask and causal limit as options): one wave per SIMD owns 32 queries and all 512
 * output dims; the keys may be cut into ranges that a second launch merges. iris_hip_fa_hd512_plan says how many ranges a call of these sizes takes and returns the bytes of scratch
 * it then needs: partial rows of the ranges, and the packed key mask of a masked call (0 for one range without mask;
 * host arithmetic, no GPU needed). iris_hip_fa_hd512 wants exactly that `splits` and a scratch of that size, 16-byte
 * aligned. Same argument conditions as iris_hip_fa_hd128 otherwise. */
size_t iris_hip_fa_hd512_plan(int seq_q, int seq_k, int heads, int causal, int masked, int *splits);
/* host arithmetic: workgroup `number` of a causal call -> (query tile, key range); returns the count of workgroups */
int iris_hip_fa_hd512_causal_order(int number, int q_tiles, int tiles_per_split, int splits, int *qt, int *range);
int iris_hip_fa_hd512(void *stream, uint16_t *out, int ldo, const uint16_t *q, const uint16_t *k,
                      const uint16_t *v, int ldi, int seq_q, int seq_k, int heads, int kv_heads,
                      float scale, int causal, const int *key_mask, int splits, void *scratch);
/* the same kernel at head_dim 256 (half the products per tile of 32 keys), with its own plan */
size_t iris_hip_fa_hd256_plan(int seq_q, int seq_k, int heads, int causal, int masked, int *splits);
int iris_hip_fa_hd256(void *stream, uint16_t *out, int ldo, const uint16_t *q, const uint16_t *k,
                      const uint16_t *v, int ldi, int seq_q, int seq_k, int heads, int kv_heads,
                      float scale, int causal, const int *key_mask, int splits, void *scratch);

/* Any head_dim (up to IRIS_ATTENTION_Q_IN_LDS_MAX_HEAD_DIM the 8 queries of a workgroup are kept in LDS as f32,
 * beyond it they are read from global memory), any stride / alignment / scale; the rows of q may have a stride
 * (ldq) of their own. Correctness path. */
#define IRIS_ATTENTION_Q_IN_LDS_MAX_HEAD_DIM 2048
int iris_hip_attention_generic(void *stream, uint16_t *out, int ldo, const uint16_t *q, int ldq,
                               const uint16_t *k, const uint16_t *v, int ldi, int seq_q,
                               int seq_k, int heads, int kv_heads, int head_dim, float scale,
                               int causal, const int *key_mask);

/* Padded, aligned copy of q, k, v for the matrix-core kernels: dst is one fused row buffer
 * [max(seq_q, seq_k)][(heads + 2 kv_heads) * hdp] (q | k | v), 16-byte aligned, every head's hd
 * elements followed by hdp - hd zeros (hdp a multiple of 8, >= hd); rows a tensor does not have are
 * zero. Sources: any stride and alignment. unpack copies the first hd of every hdp output columns
 * back into rows of any stride and alignment. */
int iris_hip_pack_heads(void *stream, uint16_t *dst, const uint16_t *q, int ldq, int seq_q,
                        const uint16_t *k, const uint16_t *v, int ldkv, int seq_k,
                        int heads, int kv_heads, int hd, int hdp);
int iris_hip_unpack_heads(void *stream, uint16_t *out, int ldo, const uint16_t *src, int ld_src,
                          int rows, int heads, int hd, int hdp);

/* ---- elementwise and normalisation operators (ew_norm_ops.hip): any size and alignment,
 * 16-byte accesses when the pointers and sizes allow ---- */
int iris_hip_f32_to_bf16(void *stream, uint16_t *dst, const float *src, size_t n);
int iris_hip_silu(void *stream, float *x, size_t n);
int iris_hip_add(void *stream, float *x, const float *a, size_t n);
int iris_hip_add_bias(void *stream, float *y, const float *bias, int rows, int cols);
int iris_hip_fill_rows(void *stream, float *out, const float *row, int rows, int dim);
int iris_hip_residual(void *stream, float *x, const float *a, const float *gate, int rows, int dim);
int iris_hip_swiglu(void *stream, uint16_t *out, int ldo, const uint16_t *gate, const uint16_t *up,
                    int ldi, int rows, int cols);
int iris_hip_upsample2x(void *stream, float *out, const float *in, int h, int width, int c);
int iris_hip_layer_norm_mod(void *stream, uint16_t *out, const float *x, const float *shift,
                            const float *scale, int rows, int dim, float eps);
int iris_hip_rms_norm_mod(void *stream, uint16_t *out, const float *x, const float *w,
                          const float *scale, int rows, int dim, float eps);
int iris_hip_rms_norm_residual(void *stream, float *x, const float *a, const float *w,
                               const float *gate, int rows, int dim, float eps);
/* group norm needs iris_hip_group_norm_scratch_floats(groups) floats of device scratch;
 * requires c % groups == 0 */
size_t iris_hip_group_norm_scratch_floats(int groups);
int iris_hip_group_norm(void *stream, float *scratch, float *out, const float *in, const float *gamma,
                        const float *beta, int hw, int c, int groups, float eps, int do_silu);

/* The same with the scratch in a device array inside the library (no allocation anywhere):
 * groups <= iris_hip_group_norm_static_max_groups(). The set-up call looks up the array's address
 * on the current device, once per device; the launcher does it itself on a device it has not seen. */
int iris_hip_group_norm_static_max_groups(void);
int iris_hip_group_norm_static_setup(void);
int iris_hip_group_norm_static(void *stream, float *out, const float *in, const float *gamma,
                               const float *beta, int hw, int c, int groups, float eps, int do_silu);

/* ---- linear layers and convolution (gemm_conv_gfx950.hip) ---- */
/* y[rows, out] = x[rows, in] @ W[out, in]^T, contiguous; MFMA kernel when in % 8 == 0 and
 * x, W are 16-byte aligned, scalar kernel otherwise */
int iris_hip_linear_f32(void *stream, float *y, const uint16_t *x, const uint16_t *W, int rows, int in, int out);
int iris_hip_linear_bf16(void *stream, uint16_t *y, const uint16_t *x, const uint16_t *W, int rows, int in, int out);
/* -2 = shape not taken, nothing enqueued */
/* Which kernel a linear layer of these sizes takes with aligned operands, host arithmetic only: plan[0] = 3 the
 * four-wave 256-row tiles, 2 the eight-wave ones, 1 the 128 x 128 kernel, 0 the scalar kernel; plan[1] = the tile width
 * of the four-wave kernel (256, 224 or 192 columns). */
void iris_hip_linear_plan(int rows, int in, int out, int out_bytes, int *plan);

int iris_hip_linear_bf16_qknorm(void *stream, uint16_t *y, const uint16_t *x, const uint16_t *W, int rows, int in, int out,
                                int q_cols, int k_cols, const float *wq, const float *wk, const float *rope_cos,
                                const float *rope_sin, float eps, int split_half);
/* Convolution. `scratch` is a private device buffer, 16-byte aligned, whose first IRIS_CONV_ZERO_BYTES are zeroed
 * once by iris_hip_conv2d_prepare_scratch and never written again (the page that taps outside the image read);
 * the rest holds the image as bf16 (or the bf16 patches of the shapes that are gathered: >= 2 * k * k * cin bytes). */
#define IRIS_CONV_ZERO_BYTES 256
int iris_hip_conv2d_prepare_scratch(void *stream, uint16_t *scratch);
int iris_hip_conv2d(void *stream, uint16_t *scratch, size_t scratch_bytes, float *out, const float *in,
                    const uint16_t *w, const float *bias, int h, int width, int cin, int cout, int k,
                    int stride, int pad_before, int pad_after);

/* Linear layer through hipBLASLt (linear_hipblaslt.cpp; the library is opened with dlopen at the
 * first call). Returns 0 when the product was enqueued, 1 when the caller must use its own
 * kernel: library absent, or no algorithm for this problem. Operands contiguous as above. */
int iris_lt_linear(void *stream, void *y, int out_bf16, const uint16_t *x, const uint16_t *W,
                   int rows, int in, int out);
int iris_lt_available(void);
void iris_lt_release(void);

/* Rotary tables [seq, half] gathered from a dictionary of (axis, position) rows: entry
 * (s, col) with columns[col] = (axis a, column j inside the axis, columns n of the axis, unused) is
 * values[index[s * naxes + a] + j] for the cosine and ... + n + j for the sine. All pointers
 * are device memory; columns is 16-byte aligned, index and values 4-byte aligned. */
int iris_hip_rope_gather(void *stream, float *cos_t, float *sin_t, const float *values,
                         const uint32_t *index, const void *columns, int seq, int half, int naxes);

#ifdef __cplusplus
}
#endif
#endif
