/*
 * Include harness for static functions of the reference's FLUX.3
 * transformer (see ref_flux2.c for the rules this follows).
 */
#include "iris_transformer_flux3.c"

void ref_flux3_head_rms_norm(float *x, const float *w, int seq, int heads, int hd, float eps) {
    head_rms_norm(x, w, seq, heads, hd, eps);
}
void ref_flux3_apply_rope(float *x, const float *c, const float *s, int seq, int heads, int hd) {
    apply_rope(x, c, s, seq, heads, hd);
}
void ref_flux3_attention(float *out, const float *q, const float *k, const float *v,
                         int seq, int heads, int hd) {
    int nq = seq < F3_ATTN_QCHUNK ? seq : F3_ATTN_QCHUNK;
    float *scores = malloc((size_t)nq * seq * sizeof(float));
    attention(out, q, k, v, scores, seq, heads, hd);
    free(scores);
}
/* Joint tables for [TXT | IMG | REFS]; returns the number of rows written. */
int ref_flux3_joint_rope(float *cos_o, float *sin_o, int head_dim, float theta,
                         int txt_seq, int img_h, int img_w,
                         const int *ref_h, const int *ref_w, int num_refs) {
    iris_transformer_flux3_t tf;
    memset(&tf, 0, sizeof(tf));
    tf.head_dim = head_dim;
    tf.rope_theta = theta;
    for (int i = 0; i < F3_ROPE_AXES; i++) tf.axes_dim[i] = head_dim / F3_ROPE_AXES;
    float *c = NULL, *s = NULL;
    joint_rope(&tf, txt_seq, img_h, img_w, ref_h, ref_w, num_refs, &c, &s);
    int total = txt_seq + img_h * img_w;
    for (int i = 0; i < num_refs; i++) total += ref_h[i] * ref_w[i];
    size_t n = (size_t)total * (head_dim / 2);
    memcpy(cos_o, c, n * sizeof(float));
    memcpy(sin_o, s, n * sizeof(float));
    free(c); free(s);
    return total;
}
