/*
 * Include harness for static functions of the reference's Qwen3 encoder
 * (see ref_flux2.c for the rules this follows).
 */
#include "iris_qwen3.c"

void ref_qwen3_rope_table(float *cos_o, float *sin_o, const int *mask, int seq, int head_dim,
                          float theta, int flux3_mode) {
    qwen3_model_t m;
    memset(&m, 0, sizeof(m));
    m.head_dim = head_dim;
    m.rope_theta = theta;
    m.extraction_mode = flux3_mode ? QWEN3_EXTRACT_FLUX3 : 0;
    m.rope_cos = cos_o;
    m.rope_sin = sin_o;
    qwen3_set_rope_positions(&m, mask, seq);
}

void ref_qwen3_head_rms_norm(float *out, const float *x, const float *w, int seq, int heads,
                             int hd, float eps) {
    qwen3_head_rms_norm(out, x, w, seq, heads, hd, eps);
}

void ref_qwen3_apply_rope(float *q, float *k, const float *c, const float *s, int seq,
                          int heads, int kv_heads, int hd) {
    apply_rope(q, k, c, s, seq, heads, kv_heads, hd);
}

/* One layer's attention up to (not including) the output projection:
 * x [seq, hidden] -> projections -> per-head norm -> RoPE -> causal/padded
 * GQA softmax attention. Returns q/k after norm+RoPE and the attention
 * output [seq, heads*hd]. */
void ref_qwen3_attention(float *attn_out, float *q_out, float *k_out, float *v_out,
                         const float *x, float *wq, float *wk, float *wv,
                         float *norm_q, float *norm_k, const int *mask, int seq, int hidden,
                         int heads, int kv_heads, int hd, float theta) {
    qwen3_model_t m;
    qwen3_layer_t l;
    memset(&m, 0, sizeof(m));
    memset(&l, 0, sizeof(l));
    int q_dim = heads * hd, kv_dim = kv_heads * hd;
    m.hidden_size = hidden; m.num_heads = heads; m.num_kv_heads = kv_heads; m.head_dim = hd;
    m.rope_theta = theta;
    m.rope_cos = malloc((size_t)seq * hd / 2 * sizeof(float));
    m.rope_sin = malloc((size_t)seq * hd / 2 * sizeof(float));
    m.norm_buf = (float *)x;
    m.q_buf = q_out; m.k_buf = k_out; m.v_buf = v_out;
    m.attn_scores = malloc((size_t)heads * seq * seq * sizeof(float));
    m.attn_out = attn_out;
    m.hidden_state = malloc((size_t)seq * hidden * sizeof(float));
    l.attn.q_proj_weight = wq; l.attn.k_proj_weight = wk; l.attn.v_proj_weight = wv;
    l.attn.o_proj_weight = calloc((size_t)hidden * q_dim, sizeof(float));
    l.attn.q_norm_weight = norm_q; l.attn.k_norm_weight = norm_k;
    (void)kv_dim;
    qwen3_set_rope_positions(&m, mask, seq);
    qwen3_attention_forward(&m, &l, seq, mask);
    free(m.rope_cos); free(m.rope_sin); free(m.attn_scores); free(m.hidden_state);
    free(l.attn.o_proj_weight);
}
