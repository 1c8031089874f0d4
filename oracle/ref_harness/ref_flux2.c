/*
 * Include harness: exposes static functions of the reference's FLUX.2
 * transformer (compiled from the reference tree where it lies; nothing is
 * copied) so tests can pin the oracle against them. Built only when the
 * reference tree is present; output goes to oracle/_ref/.
 */
#include "iris_transformer_flux.c"

void ref_flux2_rope_text(float *c, float *s, int txt_seq, int axis_dim, float theta) {
    compute_rope_text(c, s, txt_seq, axis_dim, theta);
}
void ref_flux2_rope_2d(float *c, float *s, int ph, int pw, int axis_dim, float theta) {
    compute_rope_2d(c, s, ph, pw, axis_dim, theta);
}
void ref_flux2_rope_2d_t(float *c, float *s, int ph, int pw, int axis_dim, float theta, int t) {
    compute_rope_2d_with_t_offset(c, s, ph, pw, axis_dim, theta, t);
}
void ref_flux2_apply_rope_2d(float *x, const float *c, const float *s, int seq, int heads,
                             int head_dim, int axis_dim) {
    apply_rope_2d(x, c, s, seq, heads, head_dim, axis_dim);
}
void ref_flux2_apply_qk_norm(float *q, float *k, const float *qw, const float *kw, int seq,
                             int heads, int head_dim, float eps) {
    apply_qk_norm(q, k, qw, kw, seq, heads, head_dim, eps);
}
