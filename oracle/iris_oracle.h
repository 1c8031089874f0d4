/*
 * CPU oracle for the attention hot path (TEST INFRASTRUCTURE, not product).
 *
 * A plain-C, fp32 restatement of the reference's CPU algorithms for
 *   - seeded inputs (SplitMix64 + xoshiro256** + Box-Muller),
 *   - bf16 round-to-nearest-even conversion,
 *   - per-head RMSNorm and rotary embedding (both pairings),
 *   - RoPE table / position-id / mask construction of the four model families,
 *   - softmax, naive attention, online-softmax ("flash") attention,
 *   - strided attention with causal limit, key mask and grouped kv heads.
 *
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
 * link or load this library, and only as the checker. The product library
 * never calls into it and has no CPU fallback.
 *
 * Every function names the reference file:line it follows (paths relative
 * to the reference tree).
 *
 * Pin status (what each function has been checked against, see
 * tests/test_oracle_*.py):
 *   orc_rng_*, orc_randn        bit-exact vs compiled reference + published
 *                               SplitMix64/xoshiro256** vectors
 *   orc_f2bf / orc_bf2f         exhaustive closed form + torch.bfloat16
 *   orc_fast_expf               vs libm exp, vs compiled reference softmax
 *   orc_softmax_rows            compiled reference iris_softmax_cpu
 *   orc_rms_norm_rows           compiled reference iris_rms_norm, numpy
 *   orc_rope_*                  compiled reference (public + static via the
 *                               include harness), complex-multiply identity
 *   orc_*_tables / positions    bit-exact vs compiled reference statics,
 *                               closed form in double
 *   orc_attention_naive/flash   compiled reference iris_attention /
 *                               iris_flash_attention (both branches),
 *                               float64 brute force, torch SDPA
 *   orc_attention_strided       float64 brute force, torch SDPA (mask,
 *                               causal, GQA), compiled zi_attention core
 *   orc_head_norm_rope_bf16     composition of the pinned pieces; device
 *                               semantics iris_cuda.cu:402-420
 *   orc_dev_*                   the other device operators: see the list
 *                               at the top of iris_oracle_ops.c
 */
#ifndef IRIS_ORACLE_H
#define IRIS_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- seeded inputs (iris_kernels.c:47-98) ---- */
typedef struct { uint64_t s[4]; } orc_rng_t;
void orc_rng_seed(orc_rng_t *g, uint64_t seed);
uint64_t orc_rng_next(orc_rng_t *g);
float orc_rng_uniform(orc_rng_t *g);
float orc_rng_normal(orc_rng_t *g);
void orc_randn(orc_rng_t *g, float *out, size_t n);

/* ---- bf16 (iris_cuda.cu:236-245) ---- */
uint16_t orc_f2bf(float f);
float orc_bf2f(uint16_t v);
void orc_f2bf_n(uint16_t *dst, const float *src, size_t n);
void orc_bf2f_n(float *dst, const uint16_t *src, size_t n);

/* ---- exp / softmax (iris_kernels.h:21-32, iris_kernels.c:611-634) ---- */
float orc_fast_expf(float x);
void orc_softmax_rows(float *x, int rows, int cols);

/* ---- norms (iris_kernels.c:479-508; per-head twins listed in the .c) ---- */
void orc_rms_norm_rows(float *out, const float *x, const float *w,
                       int rows, int hidden, float eps);
void orc_head_rms_norm(float *x, const float *w, int seq, int heads,
                       int head_dim, float eps);

/* ---- rotary embedding application ---- */
/* consecutive pairs, table [seq, head_dim/2] (iris_transformer_flux3.c:185-200) */
void orc_rope_pairs(float *x, const float *cos_t, const float *sin_t,
                    int seq, int heads, int head_dim);
/* consecutive pairs, duplicated table [seq, head_dim] (iris_transformer_flux.c:952-974) */
void orc_rope_pairs_dup(float *x, const float *cos_t, const float *sin_t,
                        int seq, int heads, int head_dim);
/* split-half, table [seq, head_dim/2] (iris_qwen3.c:317-360) */
void orc_rope_split(float *x, const float *cos_t, const float *sin_t,
                    int seq, int heads, int head_dim);
/* split-half, interleaved (cos,sin) table (iris_kernels.c:998-1024) */
void orc_rope_split_interleaved(float *x, const float *freqs, int batch,
                                int seq, int heads, int head_dim);
void orc_rope_freqs_interleaved(float *freqs, const int *pos, int seq,
                                int dim, float theta);   /* iris_kernels.c:1026-1038 */

/* ---- device-semantics op on bf16 storage (iris_cuda.cu:402-420) ---- */
void orc_head_norm_rope_bf16(uint16_t *x, int ld, const float *w,
                             const float *cos_t, const float *sin_t,
                             int seq, int heads, int head_dim, float eps,
                             int split_half);
/* same op, f32 storage and no final rounding (CPU twins a9 + a10) */
void orc_head_norm_rope_f32(float *x, int ld, const float *w,
                            const float *cos_t, const float *sin_t,
                            int seq, int heads, int head_dim, float eps,
                            int split_half);

/* ---- RoPE tables ---- */
/* FLUX.2: duplicated [seq,128] tables (iris_transformer_flux.c:823-881, 887-944, 981-1013) */
void orc_flux2_rope_text(float *cos_o, float *sin_o, int txt_seq, int axis_dim, float theta);
void orc_flux2_rope_image(float *cos_o, float *sin_o, int ph, int pw, int axis_dim,
                          float theta, int t_offset);
/* keep even entries: [seq,hd] -> [seq,hd/2] in place (iris_transformer_flux.c:3754-3757) */
void orc_flux2_compact(float *t, size_t seq, int head_dim);
/* full joint table [TEXT | IMAGE | REF0 ..] compacted to [seq,64]
 * (iris_transformer_flux.c:3738-3757; refs at T = 10*(i+1), iris.c:1911) */
void orc_flux2_joint_tables(float *cos_o, float *sin_o, int txt_seq, int img_h, int img_w,
                            const int *ref_h, const int *ref_w, int num_refs,
                            int axis_dim, float theta);

/* Z-Image (iris_transformer_zimage.c:604-622, 1924-1938, 1983-1994) */
void orc_zimage_axis_table(float *cos_o, float *sin_o, int axis_dim, int max_pos, float theta);
void orc_zimage_positions(int *pos, int *mask, int img_seq, int wt, int cap_seq,
                          int *ip_out, int *cp_out);
void orc_zimage_gather(float *cos_o, float *sin_o, const int *pos, int seq,
                       const int axes_dims[3], const int axes_lens[3], float theta);

/* FLUX.3 (iris_transformer_flux3.c:282-333) */
void orc_flux3_rope_rows(float *cos_o, float *sin_o, const float *pos4, int seq,
                         const int axes_dim[4], float theta);
void orc_flux3_joint_positions(float *pos4, int txt_seq, int img_h, int img_w,
                               const int *ref_h, const int *ref_w, int num_refs);

/* Qwen3 (iris_qwen3.c:277-291) */
void orc_qwen3_rope_table(float *cos_o, float *sin_o, const int *attention_mask,
                          int seq, int head_dim, float theta, int pad_at_one);

/* ---- attention ---- */
/* [b,h,s,d] contiguous, materialised scores (iris_kernels.c:656-697) */
void orc_attention_naive(float *out, const float *Q, const float *K, const float *V,
                         int batch, int heads, int seq_q, int seq_k, int head_dim, float scale);
/* [seq, heads*hd] contiguous, online softmax (iris_kernels.c:722-991) */
void orc_attention_flash(float *out, const float *Q, const float *K, const float *V,
                         int seq_q, int seq_k, int heads, int head_dim, float scale);
/* Strided rows, optional causal limit / key mask / grouped kv heads.
 * Masked scores become -1e9 after scaling, then the fast_expf softmax
 * (iris_transformer_zimage.c:698-772, iris_qwen3.c:415-491). */
void orc_attention_strided(float *out, int ldo, const float *q, const float *k, const float *v,
                           int ldq, int ldkv, int seq_q, int seq_k, int heads, int kv_heads,
                           int head_dim, float scale, int causal, const int *key_mask);
/* Same on bf16 storage with an f32 result (inputs widened exactly). */
void orc_attention_bf16(float *out, int ldo, const uint16_t *q, const uint16_t *k,
                        const uint16_t *v, int ldi, int seq_q, int seq_k, int heads,
                        int kv_heads, int head_dim, float scale, int causal,
                        const int *key_mask);

/* Selected query rows (absolute indices) against all keys; out [nrows, heads*hd]. */
void orc_attention_bf16_rows(float *out, const uint16_t *q, const uint16_t *k,
                             const uint16_t *v, int ldi, const int *rows, int nrows, int seq_k,
                             int heads, int kv_heads, int head_dim, float scale, int causal,
                             const int *key_mask);

/* ---- the remaining device operators (iris_oracle_ops.c; reference iris_dev.h:45-127) ---- */
void orc_dev_linear(float *y, const uint16_t *x, const uint16_t *W, int rows, int in, int out);
void orc_dev_layer_norm_mod(uint16_t *out, const float *x, const float *shift, const float *scale,
                            int rows, int dim, float eps);
void orc_dev_rms_norm_mod(uint16_t *out, const float *x, const float *w, const float *scale,
                          int rows, int dim, float eps);
void orc_dev_rms_norm_residual(float *x, const float *a, const float *w, const float *gate,
                               int rows, int dim, float eps);
void orc_dev_swiglu(uint16_t *out, int ldo, const uint16_t *gate, const uint16_t *up, int ldi,
                    int rows, int cols);
void orc_dev_residual(float *x, const float *a, const float *gate, int rows, int dim);
void orc_dev_silu(float *x, size_t n);
void orc_dev_add(float *x, const float *a, size_t n);
void orc_dev_add_bias(float *y, const float *bias, int rows, int cols);
void orc_dev_fill_rows(float *out, const float *row, int rows, int dim);
void orc_dev_conv2d(float *out, const float *in, const uint16_t *w, const float *bias, int h, int width,
                    int cin, int cout, int k, int stride, int pad_before, int pad_after);
void orc_dev_group_norm(float *out, const float *in, const float *gamma, const float *beta, int hw, int c,
                        int groups, float eps, int silu);
void orc_dev_upsample2x(float *out, const float *in, int h, int width, int c);

#ifdef __cplusplus
}
#endif
#endif
