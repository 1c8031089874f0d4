/*
 * Rotary-position tables for the callers of iris_dev_head_norm_rope.
 *
 * The reference's models build these tables on the host at the start of every
 * forward pass, each with its own private routine, and upload them. This
 * header gives the same tables from one small library, in two forms:
 *
 *   iris_rope_*      host builders, plain C + libm, bit-identical to the
 *                    reference's routines (same float / double arithmetic,
 *                    same libm calls on the same arguments);
 *   iris_dev_rope_*  the same tables written straight into device memory, with the
 *                    same bits: the host evaluates each DISTINCT (axis,
 *                    position) of the sequence once, with those same libm
 *                    calls (an h x w image has h + w distinct positions per
 *                    axis, not h * w), uploads that dictionary plus one
 *                    32-bit offset per (token, axis) -- 16 bytes a token for
 *                    four axes instead of the 512 bytes of its two table
 *                    rows -- and a kernel expands it. Nothing is evaluated on
 *                    the device, so nothing can round differently there.
 *
 * All tables are [seq, half] floats, half = sum of axis_dim / 2, one (cos, sin)
 * per rotated pair: the layout iris_dev_head_norm_rope takes. Column blocks
 * follow the axes in order; inside axis a, column j has frequency
 * theta^(-2j / axis_dim[a]).
 *
 * Row order of the joint sequences (text / image / reference images) is the
 * models' own: FLUX.2 and FLUX.3 [text | image | refs], Z-Image
 * [image padded to x32 | caption padded to x32].
 */
#ifndef IRIS_ROPE_H
#define IRIS_ROPE_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- generic expansion ------------------------------------------------------------------ */

/* Integer positions pos[seq][naxes], float arithmetic: angle = (float)p * (1.0f / powf(theta,
 * (float)(2j) / (float)dim)). axis_lens (may be NULL) bounds each axis: a position outside
 * [0, len) leaves that axis unrotated (cos 1, sin 0), the rule of the Z-Image gather
 * (iris_transformer_zimage.c:1924-1938). Returns 0, or -1 on a bad argument or failed allocation
 * (outputs untouched). */
int iris_rope_expand_i32(float *cos_t, float *sin_t, const int *pos, int seq, int naxes,
                         const int *axis_dims, const int *axis_lens, float theta);

/* Float positions pos[seq][naxes] (integers and half-integers, possibly negative), double
 * arithmetic rounded to float at the end (iris_transformer_flux3.c:282-294). */
int iris_rope_expand_f64(float *cos_t, float *sin_t, const float *pos, int seq, int naxes,
                         const int *axis_dims, float theta);

/* ---- FLUX.2: 4 axes (T, H, W, L) of axis_dim each --------------------------------------- */

/* rows of [text | image | refs] */
int iris_rope_joint_rows(int txt_seq, int img_h, int img_w, const int *ref_h, const int *ref_w, int num_refs);

/* pos[rows][4]: text row t -> (0, 0, 0, t); image cell (y, x) -> (0, y, x, 0); cell of reference
 * image i -> (ref_t[i], y, x, 0). ref_t NULL = 10, 20, 30, ... (iris.c:1911).
 * Replaces compute_rope_text / compute_rope_2d / compute_rope_2d_with_t_offset
 * (iris_transformer_flux.c:981-1013, 823-881, 887-944). */
void iris_rope_flux2_positions(int *pos4, int txt_seq, int img_h, int img_w,
                               const int *ref_h, const int *ref_w, const int *ref_t, int num_refs);

/* The compacted [rows, 2 * axis_dim] tables that forward_dev_flux uploads
 * (iris_transformer_flux.c:3738-3757). */
int iris_rope_flux2_tables(float *cos_t, float *sin_t, int txt_seq, int img_h, int img_w,
                           const int *ref_h, const int *ref_w, const int *ref_t, int num_refs,
                           int axis_dim, float theta);

/* ---- FLUX.3: 4 axes, half-integer grid coordinates, double math ------------------------- */

/* pos[rows][4]: text row s -> (0, 0, 0, s); image cell (r, c) -> (0, r/2, c/2, 0); cell of
 * reference image i -> (0, r/2, c/2, -(i+1)) (iris_transformer_flux3.c:296-333). */
void iris_rope_flux3_positions(float *pos4, int txt_seq, int img_h, int img_w,
                               const int *ref_h, const int *ref_w, int num_refs);

int iris_rope_flux3_tables(float *cos_t, float *sin_t, int txt_seq, int img_h, int img_w,
                           const int *ref_h, const int *ref_w, int num_refs,
                           const int axes_dim[4], float theta);

/* ---- Z-Image: 3 axes, bounded per-axis tables ------------------------------------------- */

/* pos[rows][3] and mask[rows] for [image padded to a multiple of 32 | caption padded likewise];
 * rows = *img_pad + *cap_pad (either may be NULL). Image token s -> (cap_pad + 1, s / wt, s % wt),
 * image padding -> (0, 0, 0) masked; caption slot s -> (1 + s, 0, 0), masked beyond cap_seq
 * (iris_transformer_zimage.c:1965-1994). */
void iris_rope_zimage_positions(int *pos3, int *mask, int img_seq, int wt, int cap_seq,
                                int *img_pad, int *cap_pad);

int iris_rope_zimage_tables(float *cos_t, float *sin_t, const int *pos3, int seq,
                            const int axes_dims[3], const int axes_lens[3], float theta);

/* ---- Qwen3 text encoder: one axis over the whole head ----------------------------------- */

/* Row s rotates by position s; with pad_at_one, rows whose attention_mask is 0 use position 1
 * (iris_qwen3.c:277-291). attention_mask may be NULL. Table [seq, head_dim / 2] for the
 * split-half pairing. */
int iris_rope_qwen3_tables(float *cos_t, float *sin_t, const int *attention_mask, int seq,
                           int head_dim, float theta, int pad_at_one);

/* ---- device-side generation (needs iris_dev_init) --------------------------------------- */

/* Same arguments, meaning and resulting bits as the host builders above; d_cos / d_sin are device
 * pointers from iris_dev_alloc with room for rows * half floats. The work is enqueued on the backend's stream
 * like every other operator; pos / mask arguments are HOST arrays, read before the call returns.
 * Failures are reported as for the other iris_dev_* entries (one line on stderr,
 * iris_dev_last_error() non-zero). */
void iris_dev_rope_expand_i32(float *d_cos, float *d_sin, const int *pos, int seq, int naxes,
                              const int *axis_dims, const int *axis_lens, float theta);
void iris_dev_rope_expand_f64(float *d_cos, float *d_sin, const float *pos, int seq, int naxes,
                              const int *axis_dims, float theta);
void iris_dev_rope_flux2_tables(float *d_cos, float *d_sin, int txt_seq, int img_h, int img_w,
                                const int *ref_h, const int *ref_w, const int *ref_t, int num_refs,
                                int axis_dim, float theta);
void iris_dev_rope_flux3_tables(float *d_cos, float *d_sin, int txt_seq, int img_h, int img_w,
                                const int *ref_h, const int *ref_w, int num_refs,
                                const int axes_dim[4], float theta);
void iris_dev_rope_zimage_tables(float *d_cos, float *d_sin, const int *pos3, int seq,
                                 const int axes_dims[3], const int axes_lens[3], float theta);
void iris_dev_rope_qwen3_tables(float *d_cos, float *d_sin, const int *attention_mask, int seq,
                                int head_dim, float theta, int pad_at_one);

#ifdef __cplusplus
}
#endif

#endif /* IRIS_ROPE_H */
