/*
 * CPU oracle for the attention hot path -- TEST INFRASTRUCTURE ONLY.
 * See iris_oracle.h for scope, the list of pins, and who may call this.
 * Citations are file:line in the reference tree.
 */
#include "iris_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ======================================================================
 * Seeded inputs
 * ====================================================================== */

static inline uint64_t rol64(uint64_t v, int r) { return (v << r) | (v >> (64 - r)); }

/* SplitMix64 expansion of the seed into the 4-word state (iris_kernels.c:72-81). */
void orc_rng_seed(orc_rng_t *g, uint64_t seed) {
    for (int w = 0; w < 4; w++) {
        seed += 0x9e3779b97f4a7c15ULL;
        uint64_t z = seed;
        z ^= z >> 30; z *= 0xbf58476d1ce4e5b9ULL;
        z ^= z >> 27; z *= 0x94d049bb133111ebULL;
        g->s[w] = z ^ (z >> 31);
    }
}

/* xoshiro256** step (iris_kernels.c:59-70). */
uint64_t orc_rng_next(orc_rng_t *g) {
    uint64_t *s = g->s;
    uint64_t out = rol64(s[1] * 5, 7) * 9;
    uint64_t t = s[1] << 17;
    s[2] ^= s[0];
    s[3] ^= s[1];
    s[1] ^= s[2];
    s[0] ^= s[3];
    s[2] ^= t;
    s[3] = rol64(s[3], 45);
    return out;
}

/* 53 random bits scaled in double, then narrowed (iris_kernels.c:83-85). */
float orc_rng_uniform(orc_rng_t *g) {
    return (orc_rng_next(g) >> 11) * (1.0 / 9007199254740992.0);
}

/* Box-Muller, cosine branch only; u1 redrawn while zero (iris_kernels.c:87-94). */
float orc_rng_normal(orc_rng_t *g) {
    float u1 = orc_rng_uniform(g);
    float u2 = orc_rng_uniform(g);
    while (u1 == 0.0f) u1 = orc_rng_uniform(g);
    return sqrtf(-2.0f * logf(u1)) * cosf(2.0f * 3.14159265358979323846f * u2);
}

void orc_randn(orc_rng_t *g, float *out, size_t n) {
    for (size_t i = 0; i < n; i++) out[i] = orc_rng_normal(g);
}

/* ======================================================================
 * bf16
 * ====================================================================== */

/* Round to nearest even by integer add on the bit pattern, no NaN special
 * case (iris_cuda.cu:241-245). */
uint16_t orc_f2bf(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

float orc_bf2f(uint16_t v) {   /* iris_cuda.cu:236-238 */
    uint32_t u = (uint32_t)v << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

void orc_f2bf_n(uint16_t *dst, const float *src, size_t n) {
    for (size_t i = 0; i < n; i++) dst[i] = orc_f2bf(src[i]);
}

void orc_bf2f_n(float *dst, const uint16_t *src, size_t n) {
    for (size_t i = 0; i < n; i++) dst[i] = orc_bf2f(src[i]);
}

/* ======================================================================
 * exp / softmax
 * ====================================================================== */

/* Range reduction by ln2 and a degree-5 Taylor polynomial, exponent added
 * to the bit pattern; hard 0 below -87.3 (iris_kernels.h:21-32). */
float orc_fast_expf(float x) {
    if (x < -87.3f) return 0.0f;
    if (x > 88.7f) return 1e38f;
    float n = floorf(x * 1.4426950408889634f + 0.5f);
    float r = x - n * 0.6931471805599453f;
    float p = 0.00833333f;
    p = 0.04166667f + r * p;
    p = 0.16666667f + r * p;
    p = 0.5f + r * p;
    p = 1.0f + r * p;
    p = 1.0f + r * p;
    int32_t bits;
    memcpy(&bits, &p, 4);
    bits += (int32_t)n << 23;
    memcpy(&p, &bits, 4);
    return p;
}

/* Max-subtracted softmax of each row (iris_kernels.c:611-634). */
void orc_softmax_rows(float *x, int rows, int cols) {
    for (int r = 0; r < rows; r++) {
        float *v = x + (size_t)r * cols;
        float mx = v[0];
        for (int c = 1; c < cols; c++) mx = v[c] > mx ? v[c] : mx;
        float total = 0.0f;
        for (int c = 0; c < cols; c++) {
            v[c] = orc_fast_expf(v[c] - mx);
            total += v[c];
        }
        float inv = 1.0f / total;
        for (int c = 0; c < cols; c++) v[c] *= inv;
    }
}

/* ======================================================================
 * Norms
 * ====================================================================== */

/* x * (1/sqrt(mean(x^2)+eps)) * w per row (iris_kernels.c:479-508). */
void orc_rms_norm_rows(float *out, const float *x, const float *w,
                       int rows, int hidden, float eps) {
    for (int r = 0; r < rows; r++) {
        const float *xr = x + (size_t)r * hidden;
        float *yr = out + (size_t)r * hidden;
        float ss = 0.0f;
        for (int i = 0; i < hidden; i++) ss += xr[i] * xr[i];
        float inv = 1.0f / sqrtf(ss / hidden + eps);
        for (int i = 0; i < hidden; i++) yr[i] = xr[i] * inv * w[i];
    }
}

/* Per-head RMSNorm in place on [seq, heads*hd]; one weight vector shared by
 * every head (iris_transformer_flux.c:1316-1341, iris_transformer_zimage.c:680-691,
 * iris_transformer_flux3.c:172-181, iris_qwen3.c:228-249). */
void orc_head_rms_norm(float *x, const float *w, int seq, int heads,
                       int head_dim, float eps) {
    orc_rms_norm_rows(x, x, w, seq * heads, head_dim, eps);
}

/* ======================================================================
 * Rotary embedding application
 * ====================================================================== */

void orc_rope_pairs(float *x, const float *cos_t, const float *sin_t,
                    int seq, int heads, int head_dim) {
    int half = head_dim / 2;
    for (int s = 0; s < seq; s++) {
        const float *c = cos_t + (size_t)s * half, *sn = sin_t + (size_t)s * half;
        for (int h = 0; h < heads; h++) {
            float *v = x + ((size_t)s * heads + h) * head_dim;
            for (int i = 0; i < half; i++) {
                float a = v[2 * i], b = v[2 * i + 1];
                v[2 * i] = a * c[i] - b * sn[i];
                v[2 * i + 1] = b * c[i] + a * sn[i];
            }
        }
    }
}

void orc_rope_pairs_dup(float *x, const float *cos_t, const float *sin_t,
                        int seq, int heads, int head_dim) {
    for (int s = 0; s < seq; s++) {
        const float *c = cos_t + (size_t)s * head_dim, *sn = sin_t + (size_t)s * head_dim;
        for (int h = 0; h < heads; h++) {
            float *v = x + ((size_t)s * heads + h) * head_dim;
            for (int d = 0; d < head_dim; d += 2) {
                float a = v[d], b = v[d + 1];
                v[d] = a * c[d] - b * sn[d];
                v[d + 1] = b * c[d] + a * sn[d];
            }
        }
    }
}

void orc_rope_split(float *x, const float *cos_t, const float *sin_t,
                    int seq, int heads, int head_dim) {
    int half = head_dim / 2;
    for (int s = 0; s < seq; s++) {
        const float *c = cos_t + (size_t)s * half, *sn = sin_t + (size_t)s * half;
        for (int h = 0; h < heads; h++) {
            float *v = x + ((size_t)s * heads + h) * head_dim;
            for (int i = 0; i < half; i++) {
                float a = v[i], b = v[i + half];
                v[i] = a * c[i] - b * sn[i];
                v[i + half] = a * sn[i] + b * c[i];
            }
        }
    }
}

void orc_rope_split_interleaved(float *x, const float *freqs, int batch,
                                int seq, int heads, int head_dim) {
    int half = head_dim / 2;
    for (int b = 0; b < batch; b++)
        for (int s = 0; s < seq; s++) {
            const float *f = freqs + (size_t)s * half * 2;
            for (int h = 0; h < heads; h++) {
                float *v = x + (((size_t)b * seq + s) * heads + h) * head_dim;
                for (int i = 0; i < half; i++) {
                    float c = f[2 * i], sn = f[2 * i + 1];
                    float a = v[i], bb = v[i + half];
                    v[i] = a * c - bb * sn;
                    v[i + half] = a * sn + bb * c;
                }
            }
        }
}

void orc_rope_freqs_interleaved(float *freqs, const int *pos, int seq,
                                int dim, float theta) {
    int half = dim / 2;
    for (int s = 0; s < seq; s++) {
        float p = (float)pos[s];
        for (int i = 0; i < half; i++) {
            float freq = 1.0f / powf(theta, (float)(2 * i) / (float)dim);
            float ang = p * freq;
            freqs[((size_t)s * half + i) * 2] = cosf(ang);
            freqs[((size_t)s * half + i) * 2 + 1] = sinf(ang);
        }
    }
}

/* ======================================================================
 * The device op, restated on the CPU (iris_cuda.cu:402-420)
 * ====================================================================== */

static void norm_rope_one(float *v, const float *w, const float *c, const float *sn,
                          int head_dim, float eps, int split_half) {
    int half = head_dim / 2;
    float ss = 0.0f;
    for (int d = 0; d < head_dim; d++) ss += v[d] * v[d];
    float inv = 1.0f / sqrtf(ss / head_dim + eps);
    for (int i = 0; i < half; i++) {
        int i0 = split_half ? i : 2 * i;
        int i1 = split_half ? i + half : 2 * i + 1;
        float a = v[i0] * (inv * w[i0]);
        float b = v[i1] * (inv * w[i1]);
        v[i0] = a * c[i] - b * sn[i];
        v[i1] = b * c[i] + a * sn[i];
    }
}

void orc_head_norm_rope_f32(float *x, int ld, const float *w,
                            const float *cos_t, const float *sin_t,
                            int seq, int heads, int head_dim, float eps,
                            int split_half) {
    int half = head_dim / 2;
    for (int s = 0; s < seq; s++)
        for (int h = 0; h < heads; h++)
            norm_rope_one(x + (size_t)s * ld + (size_t)h * head_dim, w,
                          cos_t + (size_t)s * half, sin_t + (size_t)s * half,
                          head_dim, eps, split_half);
}

void orc_head_norm_rope_bf16(uint16_t *x, int ld, const float *w,
                             const float *cos_t, const float *sin_t,
                             int seq, int heads, int head_dim, float eps,
                             int split_half) {
    int half = head_dim / 2;
    float *tmp = (float *)malloc((size_t)head_dim * sizeof(float));
    for (int s = 0; s < seq; s++)
        for (int h = 0; h < heads; h++) {
            uint16_t *v = x + (size_t)s * ld + (size_t)h * head_dim;
            for (int d = 0; d < head_dim; d++) tmp[d] = orc_bf2f(v[d]);
            norm_rope_one(tmp, w, cos_t + (size_t)s * half, sin_t + (size_t)s * half,
                          head_dim, eps, split_half);
            for (int d = 0; d < head_dim; d++) v[d] = orc_f2bf(tmp[d]);
        }
    free(tmp);
}

/* ======================================================================
 * RoPE tables -- FLUX.2 (4 axes T,H,W,L of axis_dim each, f32 libm)
 * ====================================================================== */

static void flux2_base(float *base, int axis_dim, float theta) {
    for (int d = 0; d < axis_dim / 2; d++)
        base[d] = 1.0f / powf(theta, (float)(2 * d) / (float)axis_dim);
}

/* One axis block of the duplicated table: entry pair (2d, 2d+1) <- angle pos*base[d]. */
static void flux2_axis(float *c, float *s, int pos_is_zero, int pos, const float *base,
                       int axis_dim) {
    if (pos_is_zero) {   /* identity axes are written as exact 1/0 */
        for (int d = 0; d < axis_dim; d++) { c[d] = 1.0f; s[d] = 0.0f; }
        return;
    }
    for (int d = 0; d < axis_dim / 2; d++) {
        float ang = (float)pos * base[d];
        float cv = cosf(ang), sv = sinf(ang);
        c[2 * d] = cv; c[2 * d + 1] = cv;
        s[2 * d] = sv; s[2 * d + 1] = sv;
    }
}

/* Text rows: only the last axis (L = token index) rotates
 * (iris_transformer_flux.c:981-1013). Row 0 still goes through cosf/sinf on
 * that axis, as in the reference. */
void orc_flux2_rope_text(float *cos_o, float *sin_o, int txt_seq, int axis_dim, float theta) {
    float base[64];
    int hd = 4 * axis_dim;
    flux2_base(base, axis_dim, theta);
    for (int t = 0; t < txt_seq; t++) {
        float *c = cos_o + (size_t)t * hd, *s = sin_o + (size_t)t * hd;
        for (int ax = 0; ax < 3; ax++) flux2_axis(c + ax * axis_dim, s + ax * axis_dim, 1, 0, base, axis_dim);
        flux2_axis(c + 3 * axis_dim, s + 3 * axis_dim, 0, t, base, axis_dim);
    }
}

/* Image rows on a ph x pw grid: H = y, W = x; L identity; T identity for
 * the target image (t_offset < 0 selects that form, iris_transformer_flux.c:823-881)
 * or rotated by t_offset for reference images (:887-944). */
void orc_flux2_rope_image(float *cos_o, float *sin_o, int ph, int pw, int axis_dim,
                          float theta, int t_offset) {
    float base[64];
    int hd = 4 * axis_dim;
    flux2_base(base, axis_dim, theta);
    for (int y = 0; y < ph; y++)
        for (int xx = 0; xx < pw; xx++) {
            size_t row = (size_t)y * pw + xx;
            float *c = cos_o + row * hd, *s = sin_o + row * hd;
            if (t_offset < 0) flux2_axis(c, s, 1, 0, base, axis_dim);
            else flux2_axis(c, s, 0, t_offset, base, axis_dim);
            flux2_axis(c + axis_dim, s + axis_dim, 0, y, base, axis_dim);
            flux2_axis(c + 2 * axis_dim, s + 2 * axis_dim, 0, xx, base, axis_dim);
            flux2_axis(c + 3 * axis_dim, s + 3 * axis_dim, 1, 0, base, axis_dim);
        }
}

void orc_flux2_compact(float *t, size_t seq, int head_dim) {
    size_t n = seq * (size_t)(head_dim / 2);
    for (size_t i = 0; i < n; i++) t[i] = t[2 * i];
}

void orc_flux2_joint_tables(float *cos_o, float *sin_o, int txt_seq, int img_h, int img_w,
                            const int *ref_h, const int *ref_w, int num_refs,
                            int axis_dim, float theta) {
    int hd = 4 * axis_dim;
    size_t seq = (size_t)txt_seq + (size_t)img_h * img_w;
    for (int r = 0; r < num_refs; r++) seq += (size_t)ref_h[r] * ref_w[r];
    float *c = (float *)malloc(seq * hd * sizeof(float));
    float *s = (float *)malloc(seq * hd * sizeof(float));
    orc_flux2_rope_text(c, s, txt_seq, axis_dim, theta);
    size_t off = txt_seq;
    orc_flux2_rope_image(c + off * hd, s + off * hd, img_h, img_w, axis_dim, theta, -1);
    off += (size_t)img_h * img_w;
    for (int r = 0; r < num_refs; r++) {
        orc_flux2_rope_image(c + off * hd, s + off * hd, ref_h[r], ref_w[r], axis_dim, theta,
                             10 * (r + 1));
        off += (size_t)ref_h[r] * ref_w[r];
    }
    orc_flux2_compact(c, seq, hd);
    orc_flux2_compact(s, seq, hd);
    memcpy(cos_o, c, seq * (hd / 2) * sizeof(float));
    memcpy(sin_o, s, seq * (hd / 2) * sizeof(float));
    free(c); free(s);
}

/* ======================================================================
 * RoPE tables -- Z-Image (axes 32/48/48, theta 256, integer positions)
 * ====================================================================== */

/* Per-axis table [max_pos, axis_dim/2] (iris_transformer_zimage.c:604-622). */
void orc_zimage_axis_table(float *cos_o, float *sin_o, int axis_dim, int max_pos, float theta) {
    int half = axis_dim / 2;
    for (int p = 0; p < max_pos; p++)
        for (int i = 0; i < half; i++) {
            float freq = 1.0f / powf(theta, (float)(2 * i) / (float)axis_dim);
            float ang = (float)p * freq;
            cos_o[(size_t)p * half + i] = cosf(ang);
            sin_o[(size_t)p * half + i] = sinf(ang);
        }
}

/* pos[seq][3] and mask[seq] for the [IMAGE(pad to x32) | CAPTION(pad to x32)]
 * sequence (iris_transformer_zimage.c:1965-1994). */
void orc_zimage_positions(int *pos, int *mask, int img_seq, int wt, int cap_seq,
                          int *ip_out, int *cp_out) {
    int ip = (img_seq + 31) / 32 * 32, cp = (cap_seq + 31) / 32 * 32;
    memset(pos, 0, (size_t)(ip + cp) * 3 * sizeof(int));
    for (int s = 0; s < ip; s++) {
        mask[s] = s < img_seq;
        if (s < img_seq) {
            pos[3 * s] = cp + 1;
            pos[3 * s + 1] = s / wt;
            pos[3 * s + 2] = s % wt;
        }
    }
    for (int s = 0; s < cp; s++) {
        mask[ip + s] = s < cap_seq;
        pos[3 * (ip + s)] = 1 + s;
    }
    if (ip_out) *ip_out = ip;
    if (cp_out) *cp_out = cp;
}

/* Gather per-axis rows into [seq, 64]; a position outside [0, len) leaves
 * that axis unrotated (iris_transformer_zimage.c:1924-1938). */
void orc_zimage_gather(float *cos_o, float *sin_o, const int *pos, int seq,
                       const int axes_dims[3], const int axes_lens[3], float theta) {
    float *tc[3], *ts[3];
    int half = 0;
    for (int ax = 0; ax < 3; ax++) {
        size_t n = (size_t)axes_lens[ax] * (axes_dims[ax] / 2);
        tc[ax] = (float *)malloc(n * sizeof(float));
        ts[ax] = (float *)malloc(n * sizeof(float));
        orc_zimage_axis_table(tc[ax], ts[ax], axes_dims[ax], axes_lens[ax], theta);
        half += axes_dims[ax] / 2;
    }
    for (int s = 0; s < seq; s++) {
        int off = 0;
        for (int ax = 0; ax < 3; ax++) {
            int n = axes_dims[ax] / 2, p = pos[3 * s + ax];
            int ok = p >= 0 && p < axes_lens[ax];
            for (int i = 0; i < n; i++) {
                cos_o[(size_t)s * half + off + i] = ok ? tc[ax][(size_t)p * n + i] : 1.0f;
                sin_o[(size_t)s * half + off + i] = ok ? ts[ax][(size_t)p * n + i] : 0.0f;
            }
            off += n;
        }
    }
    for (int ax = 0; ax < 3; ax++) { free(tc[ax]); free(ts[ax]); }
}

/* ======================================================================
 * RoPE tables -- FLUX.3 (4 axes, double math, half-integer positions)
 * ====================================================================== */

void orc_flux3_rope_rows(float *cos_o, float *sin_o, const float *pos4, int seq,
                         const int axes_dim[4], float theta) {
    int half = 0;
    for (int ax = 0; ax < 4; ax++) half += axes_dim[ax] / 2;
    for (int s = 0; s < seq; s++) {
        int p = 0;
        for (int ax = 0; ax < 4; ax++) {
            int d = axes_dim[ax];
            for (int j = 0; j < d / 2; j++, p++) {
                double freq = 1.0 / pow(theta, (double)(2 * j) / d);
                double ang = pos4[(size_t)s * 4 + ax] * freq;
                cos_o[(size_t)s * half + p] = (float)cos(ang);
                sin_o[(size_t)s * half + p] = (float)sin(ang);
            }
        }
    }
}

static void flux3_grid(float *pos4, int h, int w, float l) {
    for (int r = 0; r < h; r++)
        for (int c = 0; c < w; c++) {
            float *p = pos4 + ((size_t)r * w + c) * 4;
            p[0] = 0.0f; p[1] = 0.5f * r; p[2] = 0.5f * c; p[3] = l;
        }
}

/* [TXT | IMG | REFS]: text l = s, image l = 0, ref i l = -(i+1)
 * (iris_transformer_flux3.c:296-333). */
void orc_flux3_joint_positions(float *pos4, int txt_seq, int img_h, int img_w,
                               const int *ref_h, const int *ref_w, int num_refs) {
    size_t total = (size_t)txt_seq + (size_t)img_h * img_w;
    for (int i = 0; i < num_refs; i++) total += (size_t)ref_h[i] * ref_w[i];
    memset(pos4, 0, total * 4 * sizeof(float));
    for (int s = 0; s < txt_seq; s++) pos4[(size_t)s * 4 + 3] = (float)s;
    size_t off = txt_seq;
    flux3_grid(pos4 + off * 4, img_h, img_w, 0.0f);
    off += (size_t)img_h * img_w;
    for (int i = 0; i < num_refs; i++) {
        flux3_grid(pos4 + off * 4, ref_h[i], ref_w[i], -(float)(i + 1));
        off += (size_t)ref_h[i] * ref_w[i];
    }
}

/* ======================================================================
 * RoPE table -- Qwen3 (1 axis over the whole head, split-half pairing)
 * ====================================================================== */

void orc_qwen3_rope_table(float *cos_o, float *sin_o, const int *attention_mask,
                          int seq, int head_dim, float theta, int pad_at_one) {
    int half = head_dim / 2;
    int relocate = pad_at_one && attention_mask;
    for (int s = 0; s < seq; s++) {
        int pos = (relocate && !attention_mask[s]) ? 1 : s;
        for (int i = 0; i < half; i++) {
            float freq = 1.0f / powf(theta, (float)(2 * i) / head_dim);
            float ang = pos * freq;
            cos_o[(size_t)s * half + i] = cosf(ang);
            sin_o[(size_t)s * half + i] = sinf(ang);
        }
    }
}

/* ======================================================================
 * Attention
 * ====================================================================== */

void orc_attention_naive(float *out, const float *Q, const float *K, const float *V,
                         int batch, int heads, int seq_q, int seq_k, int head_dim, float scale) {
    float *sc = (float *)malloc((size_t)seq_q * seq_k * sizeof(float));
    for (int bh = 0; bh < batch * heads; bh++) {
        const float *q = Q + (size_t)bh * seq_q * head_dim;
        const float *k = K + (size_t)bh * seq_k * head_dim;
        const float *v = V + (size_t)bh * seq_k * head_dim;
        float *o = out + (size_t)bh * seq_q * head_dim;
        for (int i = 0; i < seq_q; i++)
            for (int j = 0; j < seq_k; j++) {
                float dot = 0.0f;
                for (int d = 0; d < head_dim; d++) dot += q[(size_t)i * head_dim + d] * k[(size_t)j * head_dim + d];
                sc[(size_t)i * seq_k + j] = dot * scale;
            }
        orc_softmax_rows(sc, seq_q, seq_k);
        for (int i = 0; i < seq_q; i++)
            for (int d = 0; d < head_dim; d++) {
                float acc = 0.0f;
                for (int j = 0; j < seq_k; j++) acc += sc[(size_t)i * seq_k + j] * v[(size_t)j * head_dim + d];
                o[(size_t)i * head_dim + d] = acc;
            }
    }
    free(sc);
}

/* Key-at-a-time online softmax (iris_kernels.c:722-776): running max starts
 * at -1e30; a new maximum rescales the accumulators, otherwise the key is
 * added with weight exp(score - max). */
static void flash_small(float *out, const float *Q, const float *K, const float *V,
                        int ld, int seq_q, int seq_k, int hd, float scale) {
    for (int i = 0; i < seq_q; i++) {
        const float *q = Q + (size_t)i * ld;
        float *o = out + (size_t)i * ld;
        float mx = -1e30f, den = 0.0f;
        for (int d = 0; d < hd; d++) o[d] = 0.0f;
        for (int j = 0; j < seq_k; j++) {
            const float *k = K + (size_t)j * ld, *v = V + (size_t)j * ld;
            float sc = 0.0f;
            for (int d = 0; d < hd; d++) sc += q[d] * k[d];
            sc *= scale;
            if (sc > mx) {
                float corr = orc_fast_expf(mx - sc);
                den = den * corr + 1.0f;
                for (int d = 0; d < hd; d++) o[d] = o[d] * corr + v[d];
                mx = sc;
            } else {
                float wgt = orc_fast_expf(sc - mx);
                den += wgt;
                for (int d = 0; d < hd; d++) o[d] += wgt * v[d];
            }
        }
        float inv = 1.0f / den;
        for (int d = 0; d < hd; d++) o[d] *= inv;
    }
}

/* Tiled online softmax, 32 queries x 64 keys (iris_kernels.c:787-886): per
 * tile take the tile max, rescale prior sums when there are any
 * (old max > -1e29), then add every key of the tile. */
static void flash_tiled(float *out, const float *Q, const float *K, const float *V,
                        int ld, int seq_q, int seq_k, int hd, float scale) {
    enum { QT = 32, KT = 64 };
    float *mxs = (float *)malloc((size_t)seq_q * sizeof(float));
    float *dens = (float *)malloc((size_t)seq_q * sizeof(float));
    float tile[QT * KT];
    for (int i = 0; i < seq_q; i++) {
        mxs[i] = -1e30f; dens[i] = 0.0f;
        for (int d = 0; d < hd; d++) out[(size_t)i * ld + d] = 0.0f;
    }
    for (int k0 = 0; k0 < seq_k; k0 += KT) {
        int kn = seq_k - k0 < KT ? seq_k - k0 : KT;
        for (int q0 = 0; q0 < seq_q; q0 += QT) {
            int qn = seq_q - q0 < QT ? seq_q - q0 : QT;
            for (int a = 0; a < qn; a++)
                for (int b = 0; b < kn; b++) {
                    const float *q = Q + (size_t)(q0 + a) * ld, *k = K + (size_t)(k0 + b) * ld;
                    float dot = 0.0f;
                    for (int d = 0; d < hd; d++) dot += q[d] * k[d];
                    tile[a * KT + b] = dot * scale;
                }
            for (int a = 0; a < qn; a++) {
                int i = q0 + a;
                const float *row = tile + a * KT;
                float *o = out + (size_t)i * ld;
                float tmx = row[0];
                for (int b = 1; b < kn; b++) tmx = row[b] > tmx ? row[b] : tmx;
                float old = mxs[i], nmx = tmx > old ? tmx : old;
                if (old > -1e29f) {
                    float corr = orc_fast_expf(old - nmx);
                    dens[i] *= corr;
                    for (int d = 0; d < hd; d++) o[d] *= corr;
                }
                for (int b = 0; b < kn; b++) {
                    float wgt = orc_fast_expf(row[b] - nmx);
                    dens[i] += wgt;
                    const float *v = V + (size_t)(k0 + b) * ld;
                    for (int d = 0; d < hd; d++) o[d] += wgt * v[d];
                }
                mxs[i] = nmx;
            }
        }
    }
    for (int i = 0; i < seq_q; i++) {
        float inv = 1.0f / dens[i];
        for (int d = 0; d < hd; d++) out[(size_t)i * ld + d] *= inv;
    }
    free(mxs); free(dens);
}

/* Per head: small problems (seq_q <= 64 and seq_k <= 128) go key by key,
 * everything else through the tiled form (iris_kernels.c:899-991). The
 * reference copies each head to contiguous buffers first; reading the
 * strided rows directly performs the same arithmetic. */
void orc_attention_flash(float *out, const float *Q, const float *K, const float *V,
                         int seq_q, int seq_k, int heads, int head_dim, float scale) {
    int ld = heads * head_dim;
    for (int h = 0; h < heads; h++) {
        size_t off = (size_t)h * head_dim;
        if (seq_q <= 64 && seq_k <= 128)
            flash_small(out + off, Q + off, K + off, V + off, ld, seq_q, seq_k, head_dim, scale);
        else
            flash_tiled(out + off, Q + off, K + off, V + off, ld, seq_q, seq_k, head_dim, scale);
    }
}

/* One (head, query) row with the masked-score convention of the CPU
 * models: score = dot*scale, then -1e9 where the key is in the future
 * (causal) or has mask 0, then the fast_expf softmax, then P.V
 * (iris_transformer_zimage.c:729-768, iris_qwen3.c:452-478). */
static void strided_row(float *o, const float *q, const float *kbase, const float *vbase,
                        int ldkv, int i, int seq_k, int hd, float scale, int causal,
                        const int *key_mask, float *sc) {
    for (int j = 0; j < seq_k; j++) {
        const float *k = kbase + (size_t)j * ldkv;
        float dot = 0.0f;
        for (int d = 0; d < hd; d++) dot += q[d] * k[d];
        dot *= scale;
        if (causal && j > i) dot = -1e9f;
        if (key_mask && key_mask[j] == 0) dot = -1e9f;
        sc[j] = dot;
    }
    orc_softmax_rows(sc, 1, seq_k);
    for (int d = 0; d < hd; d++) o[d] = 0.0f;
    for (int j = 0; j < seq_k; j++) {
        float p = sc[j];
        if (p == 0.0f) continue;
        const float *v = vbase + (size_t)j * ldkv;
        for (int d = 0; d < hd; d++) o[d] += p * v[d];
    }
}

void orc_attention_strided(float *out, int ldo, const float *q, const float *k, const float *v,
                           int ldq, int ldkv, int seq_q, int seq_k, int heads, int kv_heads,
                           int head_dim, float scale, int causal, const int *key_mask) {
    int per_kv = heads / kv_heads;
#pragma omp parallel
    {
        float *sc = (float *)malloc((size_t)(seq_k > 0 ? seq_k : 1) * sizeof(float));
#pragma omp for collapse(2) schedule(dynamic, 8)
        for (int h = 0; h < heads; h++)
            for (int i = 0; i < seq_q; i++) {
                int g = h / per_kv;
                strided_row(out + (size_t)i * ldo + (size_t)h * head_dim,
                            q + (size_t)i * ldq + (size_t)h * head_dim,
                            k + (size_t)g * head_dim, v + (size_t)g * head_dim, ldkv, i, seq_k,
                            head_dim, scale, causal, key_mask, sc);
            }
        free(sc);
    }
}

/* bf16 storage: every head's q/k/v is widened exactly to f32 first, then
 * the f32 algorithm above runs; the result stays f32. */
void orc_attention_bf16(float *out, int ldo, const uint16_t *q, const uint16_t *k,
                        const uint16_t *v, int ldi, int seq_q, int seq_k, int heads,
                        int kv_heads, int head_dim, float scale, int causal,
                        const int *key_mask) {
    size_t qn = (size_t)seq_q * heads * head_dim, kn = (size_t)seq_k * kv_heads * head_dim;
    float *qf = (float *)malloc(qn * sizeof(float));
    float *kf = (float *)malloc(kn * sizeof(float));
    float *vf = (float *)malloc(kn * sizeof(float));
    int qd = heads * head_dim, kd = kv_heads * head_dim;
    for (int i = 0; i < seq_q; i++)
        orc_bf2f_n(qf + (size_t)i * qd, q + (size_t)i * ldi, qd);
    for (int j = 0; j < seq_k; j++) {
        orc_bf2f_n(kf + (size_t)j * kd, k + (size_t)j * ldi, kd);
        orc_bf2f_n(vf + (size_t)j * kd, v + (size_t)j * ldi, kd);
    }
    orc_attention_strided(out, ldo, qf, kf, vf, qd, kd, seq_q, seq_k, heads, kv_heads,
                          head_dim, scale, causal, key_mask);
    free(qf); free(kf); free(vf);
}

/* Selected query rows only (absolute indices in rows[]); out is
 * [nrows, heads*hd] contiguous f32. Used to check full-size problems on a
 * sample of queries against all keys. */
void orc_attention_bf16_rows(float *out, const uint16_t *q, const uint16_t *k,
                             const uint16_t *v, int ldi, const int *rows, int nrows, int seq_k,
                             int heads, int kv_heads, int head_dim, float scale, int causal,
                             const int *key_mask) {
    int qd = heads * head_dim, kd = kv_heads * head_dim, per_kv = heads / kv_heads;
    float *qf = (float *)malloc((size_t)nrows * qd * sizeof(float));
    float *kf = (float *)malloc((size_t)seq_k * kd * sizeof(float));
    float *vf = (float *)malloc((size_t)seq_k * kd * sizeof(float));
    for (int r = 0; r < nrows; r++) orc_bf2f_n(qf + (size_t)r * qd, q + (size_t)rows[r] * ldi, qd);
    for (int j = 0; j < seq_k; j++) {
        orc_bf2f_n(kf + (size_t)j * kd, k + (size_t)j * ldi, kd);
        orc_bf2f_n(vf + (size_t)j * kd, v + (size_t)j * ldi, kd);
    }
#pragma omp parallel
    {
        float *sc = (float *)malloc((size_t)(seq_k > 0 ? seq_k : 1) * sizeof(float));
#pragma omp for collapse(2) schedule(dynamic, 4)
        for (int h = 0; h < heads; h++)
            for (int r = 0; r < nrows; r++) {
                int g = h / per_kv;
                strided_row(out + (size_t)r * qd + (size_t)h * head_dim,
                            qf + (size_t)r * qd + (size_t)h * head_dim,
                            kf + (size_t)g * head_dim, vf + (size_t)g * head_dim, kd, rows[r],
                            seq_k, head_dim, scale, causal, key_mask, sc);
            }
        free(sc);
    }
    free(qf); free(kf); free(vf);
}
