/*
 * Device (GPU) compute API, MI355X (gfx950) backend: the attention hot path and
 * the other operators of the reference's device header.
 *
 * This is the C ABI of libiris_dev.so. Every declaration below that cites
 * the reference header keeps that header's name, argument order, units and
 * meaning, so host C code written against the reference's iris_dev.h
 * (FLUX.2 / FLUX.3 / Z-Image transformers, Qwen3 encoder) links against
 * this library for these calls without change.
 *
 * Conventions (reference iris_dev.h:7-15):
 *  - tensors are plain device pointers from iris_dev_alloc(); bf16 values are
 *    stored as uint16_t; matrices are row-major; strides count elements;
 *  - operations are enqueued in order on one stream owned by the library;
 *    results are visible to later operations, and to the host after
 *    iris_dev_download() or iris_dev_sync();
 *  - compute entries return void: on failure a line prefixed "iris_dev:"
 *    goes to stderr, the output is left undefined and the process goes on
 *    (reference iris_cuda.cu:108-111). There is no CPU fallback here.
 *  - one caller thread, device 0.
 */
#ifndef IRIS_DEV_H
#define IRIS_DEV_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- setup (reference iris_dev.h:27-31, iris_cuda.cu:117-173) ---- */
int iris_dev_init(void);            /* 1 if a usable gfx950 GPU was found */
int iris_dev_available(void);
const char *iris_dev_name(void);
void iris_dev_cleanup(void);

/* ---- memory (reference iris_dev.h:33-43, iris_cuda.cu:175-230) ---- */
void *iris_dev_alloc(size_t bytes);                 /* NULL on failure; 0 bytes allocates 1 */
void iris_dev_free(void *p);                        /* waits for pending work first */
void iris_dev_upload(void *dst, const void *src, size_t bytes);     /* returns after the copy */
void iris_dev_download(void *dst, const void *src, size_t bytes);   /* returns after the copy */
void iris_dev_upload_2d(void *dst, size_t dst_stride, const void *src, size_t src_stride,
                        size_t row_bytes, size_t rows);             /* strides in bytes */
void iris_dev_sync(void);

/* ---- the hot path ---- */

/* reference iris_dev.h:74-81 (kernel iris_cuda.cu:402-420, launcher :445-453).
 * In place on the bf16 heads x[s, h * head_dim + d] (row stride ld): per-head
 * RMSNorm with weight w [head_dim], then rotation by the angles of row s
 * (rope_cos/sin: [seq, head_dim / 2]). Pairs are consecutive (2i, 2i + 1),
 * or (i, i + head_dim / 2) when split_half is set. */
void iris_dev_head_norm_rope(uint16_t *x, int ld, const float *w,
                             const float *rope_cos, const float *rope_sin,
                             int seq, int heads, int head_dim, float eps,
                             int split_half);

/* reference iris_dev.h:83-92 (dispatcher iris_cuda.cu:878-937).
 * Scaled dot-product attention over bf16 [seq, heads * head_dim] tensors.
 * q, k, v share the row stride ldi, out has row stride ldo. With fewer kv
 * heads (GQA), query head h uses kv head h / (heads / kv_heads).
 * causal: query i ignores keys j > i. key_mask: device int [seq_k],
 * 0 = ignored key, or NULL. A query with no valid key gives a zero row
 * (reference iris_cuda.cu:531, 650, 676).
 * Every combination of heads / kv_heads / head_dim / stride / alignment is answered, as in the
 * reference (its fallback is two GEMMs, iris_cuda.cu:897-936, with no limit on head_dim). head_dim 128, 256
 * and 512 on 16-byte aligned rows run on the matrix cores directly, any other head_dim <= 512 or
 * alignment through a padded, aligned private copy of q, k, v; the rest (head_dim > 512,
 * scale <= 0, more than 250000 masked keys) on a scalar kernel. head_dim 512 with at least 32 keys
 * (the VAE's call, reference iris_vae.c:1112-1124) and head_dim 256 may cut the keys into ranges
 * whose partial results pass through private scratch (67 MB at 16384 tokens x 512), and keep a
 * packed copy of the key mask there (4 bytes per 32 keys); every other directly taken layout
 * allocates nothing.
 * Numerics: P = exp(s - max) is rounded to bf16 for the P V product, as in the reference's GPU
 * kernels (iris_cuda.cu:656-665), and the row sum in the denominator is taken over those ROUNDED
 * values (on the matrix cores), where the reference sums the unrounded f32 values (:659-665): the
 * output weights then add up to exactly one; the two differ by the mean bf16 rounding error of a
 * row, far inside the tolerance against the fp32 CPU attention. */
void iris_dev_attention(uint16_t *out, int ldo,
                        const uint16_t *q, const uint16_t *k, const uint16_t *v,
                        int ldi, int seq_q, int seq_k, int heads, int kv_heads,
                        int head_dim, float scale, int causal,
                        const int *key_mask);

/* ---- the other operators of the device API (reference iris_dev.h:45-72, 94-127) ----
 * Same names, arguments and meaning as the reference; each one enqueues on the
 * library's stream. */

/* dst[i] = bf16(src[i]) (reference iris_dev.h:45-46) */
void iris_dev_f32_to_bf16(uint16_t *dst, const float *src, size_t n);

/* y[rows, out] = x[rows, in] @ W[out, in]^T: bf16 inputs, f32 accumulation, f32 or bf16
 * output; all matrices contiguous (reference iris_dev.h:48-53) */
void iris_dev_linear_f32(float *y, const uint16_t *x, const uint16_t *W, int rows, int in, int out);
void iris_dev_linear_bf16(uint16_t *y, const uint16_t *x, const uint16_t *W, int rows, int in, int out);

/* out = LayerNorm(x) * (1 + scale) + shift, no affine parameters; shift / scale [dim],
 * either may be NULL (reference iris_dev.h:55-59) */
void iris_dev_layer_norm_mod(uint16_t *out, const float *x, const float *shift, const float *scale,
                             int rows, int dim, float eps);
/* out = RMSNorm(x) * w (reference iris_dev.h:61-63) */
void iris_dev_rms_norm(uint16_t *out, const float *x, const float *w, int rows, int dim, float eps);
/* out = RMSNorm(x) * w * (1 + scale), scale optional (reference iris_dev.h:65-68) */
void iris_dev_rms_norm_mod(uint16_t *out, const float *x, const float *w, const float *scale,
                           int rows, int dim, float eps);
/* x += tanh(gate) * RMSNorm(a) * w in f32; gate [dim] may be NULL (reference iris_dev.h:70-73) */
void iris_dev_rms_norm_residual(float *x, const float *a, const float *w, const float *gate,
                                int rows, int dim, float eps);

/* out[r, c] = silu(gate[r, c]) * up[r, c]; gate / up row stride ldi, out row stride ldo
 * (reference iris_dev.h:94-97) */
void iris_dev_swiglu(uint16_t *out, int ldo, const uint16_t *gate, const uint16_t *up, int ldi,
                     int rows, int cols);
/* x[r, c] += gate[c] * a[r, c], or x += a when gate is NULL (reference iris_dev.h:99-101) */
void iris_dev_residual(float *x, const float *a, const float *gate, int rows, int dim);

/* elementwise helpers on f32 vectors (reference iris_dev.h:103-107) */
void iris_dev_silu(float *x, size_t n);
void iris_dev_add(float *x, const float *a, size_t n);                    /* x += a */
void iris_dev_add_bias(float *y, const float *bias, int rows, int cols);  /* y[r, c] += bias[c] */
void iris_dev_fill_rows(float *out, const float *row, int rows, int dim); /* out[r, c] = row[c] */

/* k x k convolution of a channels-last f32 image [h * width, cin] into [oh * ow, cout] with
 * zero padding of pad_before / pad_after pixels on each axis,
 *   oh = (h + pad_before + pad_after - k) / stride + 1 (same for ow),
 * w: bf16 [cout, k * k * cin] in (ky, kx, c) order, bias may be NULL (reference iris_dev.h:111-121) */
void iris_dev_conv2d(float *out, const float *in, const uint16_t *w, const float *bias,
                     int h, int width, int cin, int cout, int k, int stride,
                     int pad_before, int pad_after);
/* GroupNorm over [hw, c] with affine gamma / beta [c], optionally followed by SiLU
 * (reference iris_dev.h:123-126) */
void iris_dev_group_norm(float *out, const float *in, const float *gamma, const float *beta,
                         int hw, int c, int groups, float eps, int silu);
/* No counterpart in the reference. The same operator for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc):
 * same arguments, same kernels and the same bits as iris_dev_group_norm, but its scratch (partial
 * moments and statistics, 787 KB) is an array inside the library instead of memory allocated at
 * the first call, so this entry calls no hipMalloc / hipFree at all. groups <= 64; more is refused
 * with an error (use iris_dev_group_norm). All calls on a GPU share that one array: calls that
 * overlap in time would race, so keep them on the library's stream, which orders them. */
void iris_dev_group_norm_noalloc(float *out, const float *in, const float *gamma, const float *beta,
                                 int hw, int c, int groups, float eps, int silu);
/* nearest-neighbour 2x upsampling of [h * w, c] into [2h * 2w, c] (reference iris_dev.h:128-129) */
void iris_dev_upsample2x(float *out, const float *in, int h, int width, int c);

/* ---- additions (no counterpart in the reference header) ---- */

/* The Q and K calls that every reference call site issues back to back
 * (e.g. iris_transformer_flux.c:3834-3837, iris_qwen3.c:1590-1593) as ONE
 * launch: xq has q_heads heads normalised with wq, xk has k_heads heads
 * normalised with wk; both share ld, the tables, eps and the pairing.
 * Same result as the two iris_dev_head_norm_rope calls. */
void iris_dev_head_norm_rope_qk(uint16_t *xq, uint16_t *xk, int ld,
                                const float *wq, const float *wk,
                                const float *rope_cos, const float *rope_sin,
                                int seq, int q_heads, int k_heads, int head_dim,
                                float eps, int split_half);

/* The FOUR calls of a double-stream block (iris_transformer_flux.c:3796-3803: text rows and image rows of the joint
 * q | k | v buffer, Q and K each, every stream with its own weight pair, tables offset to the stream's first row)
 * as ONE launch over the joint rows: rows [0, rows_a) of xq / xk take (wq_a, wk_a), rows [rows_a, seq) take
 * (wq_b, wk_b); row s of the tables belongs to row s of the joint sequence. Same result as
 *     iris_dev_head_norm_rope(xq, ld, wq_a, cos, sin, rows_a, q_heads, ...);   ..(xk, ld, wk_a, ...)
 *     iris_dev_head_norm_rope(xq + rows_a * ld, ld, wq_b, cos + rows_a * head_dim / 2, sin + ..., seq - rows_a, ...);
 *     ..(xk + rows_a * ld, ld, wk_b, ...)
 * bit for bit. The 512-row text calls alone are launch-bound (6.5 MB each). */
void iris_dev_head_norm_rope_qk_streams(uint16_t *xq, uint16_t *xk, int ld,
                                        const float *wq_a, const float *wk_a, const float *wq_b, const float *wk_b,
                                        int rows_a, const float *rope_cos, const float *rope_sin,
                                        int seq, int q_heads, int k_heads, int head_dim, float eps, int split_half);

/* iris_dev_attention with the Q half of the normalisation folded in: the result is what
 *     iris_dev_head_norm_rope(q, ldi, wq, rope_cos, rope_sin, seq_q, heads, head_dim, eps, split_half);
 *     iris_dev_attention(out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, head_dim, scale, causal, key_mask);
 * gives, bit for bit, but q is only read: the rows in memory stay as they were, and the pass
 * that reads and rewrites them is saved. k must already be normalised (the single
 * iris_dev_head_norm_rope call on K stays). For the call sites that use Q for nothing else
 * after the attention, which is all of them (iris_transformer_flux.c:3834-3839,
 * iris_transformer_flux3.c:693-696, iris_transformer_zimage.c:1948-1951, iris_qwen3.c:1590-1596).
 * Row s of the tables belongs to query row s. Every argument combination is answered: those the
 * matrix-core kernel does not take go through a normalised copy of Q in private scratch. */
void iris_dev_attention_qnorm(uint16_t *out, int ldo,
                              const uint16_t *q, const uint16_t *k, const uint16_t *v,
                              int ldi, int seq_q, int seq_k, int heads, int kv_heads,
                              int head_dim, float scale, int causal, const int *key_mask,
                              const float *wq, const float *rope_cos, const float *rope_sin,
                              float eps, int split_half);

/* The projection and the normalisation of its output as one launch: the result is what
 *     iris_dev_linear_bf16(y, x, W, rows, in, out);
 *     iris_dev_head_norm_rope_qk(y, y + q_heads * head_dim, out, wq, wk, rope_cos, rope_sin,
 *                                rows, q_heads, k_heads, head_dim, eps, split_half);
 * gives: the leading q_heads * head_dim columns of y are Q heads, the next k_heads * head_dim columns K heads,
 * the rest (V, and the MLP columns of the fused single-block projection) is stored as the projection leaves
 * it. This is the layout of every fused QKV projection of the reference's device paths
 * (iris_transformer_flux.c:3795-3800 and 3833-3837, iris_transformer_flux3.c:692-694,
 * iris_transformer_zimage.c:1947-1949, iris_qwen3.c:1589-1593), which all issue exactly these three calls. The
 * library's own GEMM can normalise each 256 x 256 output tile while it still sits in the LDS, which saves the
 * pass that reads and rewrites the Q and K rows: that one-launch kernel runs unless the vendor GEMM is selected
 * (iris_dev_linear_backend(2)) and present, for head_dim 128, rows >= 256, out >= 256 and
 * a multiple of 128, in a multiple of 64 and 16-byte aligned operands; its bits are those of the two calls
 * above on the own GEMM. Otherwise the entry issues the two calls itself (the vendor GEMM followed by the norm
 * kernel is the faster pair where that library is present). */
void iris_dev_linear_bf16_qknorm(uint16_t *y, const uint16_t *x, const uint16_t *W, int rows, int in, int out,
                                 int q_heads, int k_heads, int head_dim, const float *wq, const float *wk,
                                 const float *rope_cos, const float *rope_sin, float eps, int split_half);

/* The library's stream as a hipStream_t, for callers that time kernels with
 * HIP events or order their own work after the library's. */
void *iris_dev_stream(void);

/* 0 when the most recent compute / memory entry succeeded, else a HIP error
 * code or -1 for a rejected argument; reading it clears it. Lets a test see
 * the failures that the void entries only report on stderr. */
int iris_dev_last_error(void);

/* Which kernel the most recent iris_dev_attention / iris_dev_head_norm_rope
 * call used: a static string such as "fa_hd128" or "generic". */
const char *iris_dev_last_kernel(void);

/* Which GEMM runs the linear layers. 0 (default) and 1: this library's own MFMA kernels. 2: the vendor
 * library hipBLASLt where it can be opened at run time and takes the problem (the reference's backend calls
 * cuBLAS / hipBLAS for them, iris_cuda.cu:456-505), the own kernels otherwise: the yardstick the benchmark
 * measures the own kernels against, not a production path. No counterpart in the reference. */
void iris_dev_linear_backend(int which);

#ifdef __cplusplus
}
#endif
#endif /* IRIS_DEV_H */
