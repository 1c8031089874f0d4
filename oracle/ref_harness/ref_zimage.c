/*
 * Include harness for static functions of the reference's Z-Image
 * transformer (see ref_flux2.c for the rules this follows).
 */
#include "iris_transformer_zimage.c"

static void zi_setup(zi_transformer_t *tf, int n_heads, int head_dim, const int *axes_dims,
                     const int *axes_lens, float theta) {
    memset(tf, 0, sizeof(*tf));
    tf->n_heads = n_heads;
    tf->head_dim = head_dim;
    tf->dim = n_heads * head_dim;
    tf->rope_theta = theta;
    for (int i = 0; i < 3; i++) { tf->axes_dims[i] = axes_dims[i]; tf->axes_lens[i] = axes_lens[i]; }
    zi_precompute_rope(tf);
}
static void zi_teardown(zi_transformer_t *tf) {
    for (int i = 0; i < 3; i++) { free(tf->rope_cos[i]); free(tf->rope_sin[i]); }
}

/* Per-axis table of zi_precompute_rope: [axes_lens[ax], axes_dims[ax]/2]. */
void ref_zi_axis_table(float *cos_o, float *sin_o, int ax, const int *axes_dims,
                       const int *axes_lens, float theta) {
    zi_transformer_t tf;
    zi_setup(&tf, 1, axes_dims[0] + axes_dims[1] + axes_dims[2], axes_dims, axes_lens, theta);
    size_t n = (size_t)axes_lens[ax] * (axes_dims[ax] / 2);
    memcpy(cos_o, tf.rope_cos[ax], n * sizeof(float));
    memcpy(sin_o, tf.rope_sin[ax], n * sizeof(float));
    zi_teardown(&tf);
}

#ifdef IRIS_DEV  /* only when built with the device path, which needs a device backend */
void ref_zi_dev_rope(float *cos_o, float *sin_o, const int *pos, int seq, const int *axes_dims,
                     const int *axes_lens, float theta) {
    zi_transformer_t tf;
    zi_setup(&tf, 1, axes_dims[0] + axes_dims[1] + axes_dims[2], axes_dims, axes_lens, theta);
    zi_dev_rope(cos_o, sin_o, pos, seq, &tf);
    zi_teardown(&tf);
}
#endif

void ref_zi_apply_rope(float *x, const int *pos, int seq, int n_heads, const int *axes_dims,
                       const int *axes_lens, float theta) {
    zi_transformer_t tf;
    zi_setup(&tf, n_heads, axes_dims[0] + axes_dims[1] + axes_dims[2], axes_dims, axes_lens, theta);
    zi_apply_rope(x, pos, seq, n_heads, &tf);
    zi_teardown(&tf);
}

void ref_zi_qk_norm(float *x, const float *w, int seq, int n_heads, int head_dim, float eps) {
    zi_qk_norm(x, w, seq, n_heads, head_dim, eps);
}

/* The whole CPU attention of one block: projections with the given
 * [dim,dim] weights, QK norm, RoPE from pos ids, masked softmax, P.V and
 * output projection. x: [seq, dim]. */
void ref_zi_attention(float *out, const float *x, float *wq, float *wk, float *wv, float *wo,
                      float *norm_q, float *norm_k, const int *pos, const int *mask, int seq,
                      int n_heads, const int *axes_dims, const int *axes_lens, float theta) {
    zi_transformer_t tf;
    int hd = axes_dims[0] + axes_dims[1] + axes_dims[2];
    zi_setup(&tf, n_heads, hd, axes_dims, axes_lens, theta);
    zi_block_t b;
    memset(&b, 0, sizeof(b));
    b.attn_q_weight = wq; b.attn_k_weight = wk; b.attn_v_weight = wv; b.attn_out_weight = wo;
    b.attn_norm_q = norm_q; b.attn_norm_k = norm_k;
    tf.work_qkv = malloc((size_t)3 * seq * tf.dim * sizeof(float));
    tf.work_attn = malloc((size_t)seq * seq * sizeof(float));
    zi_attention(out, x, &b, pos, mask, seq, &tf);
    free(tf.work_qkv); free(tf.work_attn);
    zi_teardown(&tf);
}
