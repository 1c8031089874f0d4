/*
 * Parity check of the device library from plain C, the language of its callers.
 *
 * It does what a transformer block of the reference does for one sequence
 * (iris_transformer_flux.c:3834-3839): per-head RMSNorm + RoPE on Q, on K,
 * then joint attention, on the fused q|k|v row buffer, through the entry
 * points of include/iris_dev.h only, and compares every output element with
 * the CPU oracle run on the same inputs; the library's one-call form of the
 * Q normalisation + attention is held to the two calls bit for bit. The device side takes its rotary
 * tables from the library's own generators (include/iris_rope.h), the oracle
 * side from the oracle's, so the table builders are part of what is checked.
 * A second pass covers the causal
 * grouped-KV + padding-mask form of the text encoder (iris_qwen3.c:1590-1596),
 * a third the single 512-wide head of the VAE (iris_vae.c:1112-1124).
 *
 * Test program: links libiris_dev.so (product) and libiris_oracle.so (checker).
 * Exit status 0 = all checks passed.
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "iris_dev.h"
#include "iris_rope.h"
#include "iris_oracle.h"

static int failures = 0;

/* Absolute bar (max_tol, mean_tol) and, so that small outputs are held as tightly as large ones,
 * the same errors against the size of the expected values: max-abs <= 4e-2 max|want|,
 * mean-abs <= 1e-2 mean|want|. An all-zero reference is refused. */
static void compare(const char *what, const uint16_t *got, const float *want, size_t n,
                    double max_tol, double mean_tol) {
    double mx = 0.0, sum = 0.0, ref_mx = 0.0, ref_sum = 0.0;
    for (size_t i = 0; i < n; i++) {
        double d = fabs((double)orc_bf2f(got[i]) - (double)want[i]);
        if (!(d <= mx)) mx = d;                    /* also catches NaN */
        sum += d;
        double w = fabs((double)want[i]);
        if (w > ref_mx) ref_mx = w;
        ref_sum += w;
    }
    const double mean = sum / (double)n, ref_mean = ref_sum / (double)n;
    int ok = mx <= max_tol && mean <= mean_tol && ref_mean > 0.0 && mx <= 4e-2 * ref_mx && mean <= 1e-2 * ref_mean;
    printf("%-34s max-abs %.3e (max|want| %.3e)  mean-abs %.3e (mean|want| %.3e)  %s\n", what, mx, ref_mx, mean,
           ref_mean, ok ? "ok" : "FAIL");
    if (!ok) failures++;
}

static uint16_t *randn_bf16(orc_rng_t *g, size_t n, float sigma) {
    float *f = malloc(n * sizeof(float));
    uint16_t *b = malloc(n * sizeof(uint16_t));
    orc_randn(g, f, n);
    for (size_t i = 0; i < n; i++) f[i] *= sigma;
    orc_f2bf_n(b, f, n);
    free(f);
    return b;
}

static void *to_device(const void *src, size_t bytes) {
    void *d = iris_dev_alloc(bytes);
    if (!d) { fprintf(stderr, "alloc of %zu bytes failed\n", bytes); exit(2); }
    iris_dev_upload(d, src, bytes);
    return d;
}

/* norm+rope on Q and K, then attention; rows = [q | k | v], strides in elements.
 * d_cos / d_sin: device tables from the library; cos_t / sin_t: the oracle's tables for the same rows. */
static void block_case(const char *name, int seq, int heads, int kv_heads, int split_half, int causal,
                       const int *mask, float *d_cos, float *d_sin, const float *cos_t, const float *sin_t,
                       float eps, uint64_t seed) {
    const int hd = 128, qd = heads * hd, kd = kv_heads * hd, ldi = qd + 2 * kd, ldo = qd;
    orc_rng_t g;
    orc_rng_seed(&g, seed);
    uint16_t *rows = randn_bf16(&g, (size_t)seq * ldi, 1.0f);
    float wq[128], wk[128];
    orc_randn(&g, wq, 128);
    orc_randn(&g, wk, 128);
    for (int i = 0; i < 128; i++) { wq[i] = 1.0f + 0.02f * wq[i]; wk[i] = 1.0f + 0.02f * wk[i]; }
    const float scale = 1.0f / sqrtf((float)hd);

    /* device */
    uint16_t *d_rows = to_device(rows, (size_t)seq * ldi * 2);
    float *d_wq = to_device(wq, sizeof wq), *d_wk = to_device(wk, sizeof wk);
    int *d_mask = mask ? to_device(mask, (size_t)seq * sizeof(int)) : NULL;
    uint16_t *d_out = iris_dev_alloc((size_t)seq * ldo * 2);
    uint16_t *d_out_fused = iris_dev_alloc((size_t)seq * ldo * 2);
    iris_dev_head_norm_rope(d_rows + qd, ldi, d_wk, d_cos, d_sin, seq, kv_heads, hd, eps, split_half);
    /* the library's one-call form of "normalise Q, then attend", on the still raw Q ... */
    iris_dev_attention_qnorm(d_out_fused, ldo, d_rows, d_rows + qd, d_rows + qd + kd, ldi, seq, seq, heads, kv_heads, hd,
                             scale, causal, d_mask, d_wq, d_cos, d_sin, eps, split_half);
    /* ... and the reference's two calls */
    iris_dev_head_norm_rope(d_rows, ldi, d_wq, d_cos, d_sin, seq, heads, hd, eps, split_half);
    iris_dev_attention(d_out, ldo, d_rows, d_rows + qd, d_rows + qd + kd, ldi, seq, seq, heads, kv_heads, hd,
                       scale, causal, d_mask);
    uint16_t *rows_back = malloc((size_t)seq * ldi * 2), *out = malloc((size_t)seq * ldo * 2);
    uint16_t *out_fused = malloc((size_t)seq * ldo * 2);
    iris_dev_download(rows_back, d_rows, (size_t)seq * ldi * 2);
    iris_dev_download(out, d_out, (size_t)seq * ldo * 2);
    iris_dev_download(out_fused, d_out_fused, (size_t)seq * ldo * 2);
    if (iris_dev_last_error() != 0) { printf("%s: device error\n", name); failures++; }
    {
        const int same = memcmp(out, out_fused, (size_t)seq * ldo * 2) == 0;
        printf("%-34s %s\n", "  attention_qnorm == the two calls", same ? "bit for bit" : "FAIL");
        if (!same) failures++;
    }

    /* oracle: same bf16 rows, same order of operations */
    orc_head_norm_rope_bf16(rows, ldi, wq, cos_t, sin_t, seq, heads, hd, eps, split_half);
    orc_head_norm_rope_bf16(rows + qd, ldi, wk, cos_t, sin_t, seq, kv_heads, hd, eps, split_half);
    float *rows_f = malloc((size_t)seq * ldi * sizeof(float));
    orc_bf2f_n(rows_f, rows, (size_t)seq * ldi);
    char label[96];
    snprintf(label, sizeof label, "%s norm+rope rows", name);
    compare(label, rows_back, rows_f, (size_t)seq * ldi, 0.04, 1e-3);      /* <= 1 bf16 ulp of values up to ~4 */
    /* attention is checked on the device's own normalised rows, so the two stages are judged separately */
    float *want = malloc((size_t)seq * ldo * sizeof(float));
    orc_attention_bf16(want, ldo, rows_back, rows_back + qd, rows_back + qd + kd, ldi, seq, seq, heads, kv_heads,
                       hd, scale, causal, mask);
    snprintf(label, sizeof label, "%s attention", name);
    compare(label, out, want, (size_t)seq * ldo, 2e-2, 2e-3);

    iris_dev_free(d_rows); iris_dev_free(d_wq); iris_dev_free(d_wk); iris_dev_free(d_cos); iris_dev_free(d_sin);
    if (d_mask) iris_dev_free(d_mask);
    iris_dev_free(d_out); iris_dev_free(d_out_fused);
    free(rows); free(rows_back); free(out); free(out_fused); free(rows_f); free(want);
}

static void vae_case(int seq, uint64_t seed) {
    const int hd = 512, ldi = 3 * hd;
    orc_rng_t g;
    orc_rng_seed(&g, seed);
    uint16_t *rows = randn_bf16(&g, (size_t)seq * ldi, 1.0f);
    const float scale = 1.0f / sqrtf((float)hd);
    uint16_t *d_rows = to_device(rows, (size_t)seq * ldi * 2);
    uint16_t *d_out = iris_dev_alloc((size_t)seq * hd * 2);
    iris_dev_attention(d_out, hd, d_rows, d_rows + hd, d_rows + 2 * hd, ldi, seq, seq, 1, 1, hd, scale, 0, NULL);
    uint16_t *out = malloc((size_t)seq * hd * 2);
    iris_dev_download(out, d_out, (size_t)seq * hd * 2);
    float *want = malloc((size_t)seq * hd * sizeof(float));
    orc_attention_bf16(want, hd, rows, rows + hd, rows + 2 * hd, ldi, seq, seq, 1, 1, hd, scale, 0, NULL);
    compare("vae 1 head x 512 attention", out, want, (size_t)seq * hd, 2e-2, 2e-3);
    printf("  kernel: %s\n", iris_dev_last_kernel());
    iris_dev_free(d_rows); iris_dev_free(d_out);
    free(rows); free(out); free(want);
}

int main(void) {
    if (!iris_dev_init()) {
        fprintf(stderr, "c_abi_parity: no usable gfx950 device\n");
        return 3;
    }
    printf("device: %s\n", iris_dev_name());

    /* joint text + image block: 24 heads, 40 text + 12 x 12 image tokens, FLUX.2-style tables */
    {
        const int txt = 40, gh = 12, gw = 12, seq = txt + gh * gw;
        float *c = malloc((size_t)seq * 64 * 4), *s = malloc((size_t)seq * 64 * 4);
        orc_flux2_joint_tables(c, s, txt, gh, gw, NULL, NULL, 0, 32, 2000.0f);
        float *hc = malloc((size_t)seq * 64 * 4), *hs = malloc((size_t)seq * 64 * 4);
        if (iris_rope_joint_rows(txt, gh, gw, NULL, NULL, 0) != seq ||
            iris_rope_flux2_tables(hc, hs, txt, gh, gw, NULL, NULL, NULL, 0, 32, 2000.0f) != 0 ||
            memcmp(hc, c, (size_t)seq * 64 * 4) || memcmp(hs, s, (size_t)seq * 64 * 4)) {
            printf("host flux2 tables differ from the oracle's\n");
            failures++;
        }
        float *d_cos = iris_dev_alloc((size_t)seq * 64 * 4), *d_sin = iris_dev_alloc((size_t)seq * 64 * 4);
        iris_dev_rope_flux2_tables(d_cos, d_sin, txt, gh, gw, NULL, NULL, NULL, 0, 32, 2000.0f);
        block_case("joint 24h", seq, 24, 24, 0, 0, NULL, d_cos, d_sin, c, s, 1e-6f, 20250101);
        free(c); free(s); free(hc); free(hs);
    }
    /* text encoder layer: causal, 32 query heads on 8 kv heads, split-half rotation, right padding */
    {
        const int seq = 200, len = 137;
        float *c = malloc((size_t)seq * 64 * 4), *s = malloc((size_t)seq * 64 * 4);
        int *mask = malloc(seq * sizeof(int));
        for (int i = 0; i < seq; i++) mask[i] = i < len;
        orc_qwen3_rope_table(c, s, mask, seq, 128, 1e6f, 0);
        float *d_cos = iris_dev_alloc((size_t)seq * 64 * 4), *d_sin = iris_dev_alloc((size_t)seq * 64 * 4);
        iris_dev_rope_qwen3_tables(d_cos, d_sin, mask, seq, 128, 1e6f, 0);
        block_case("causal gqa 32/8", seq, 32, 8, 1, 1, mask, d_cos, d_sin, c, s, 1e-6f, 20250104);
        free(c); free(s); free(mask);
    }
    vae_case(300, 20250107);

    iris_dev_cleanup();
    printf(failures ? "FAILED (%d)\n" : "all checks passed\n", failures);
    return failures ? 1 : 0;
}
