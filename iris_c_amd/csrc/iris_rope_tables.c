/*
 * Host builders of the rotary-position tables (include/iris_rope.h).
 *
 * Every model of the reference has its own table routine, but all of them
 * compute the same thing: row s, axis a, column j of that axis holds
 * cos / sin of  position(s, a) * theta^(-2j / axis_dim[a]). They differ in
 * how positions are laid out and in the arithmetic type:
 *
 *   float  : FLUX.2 (iris_transformer_flux.c:823-1013), Z-Image
 *            (iris_transformer_zimage.c:604-622, 1924-1938), Qwen3 (iris_qwen3.c:277-291):
 *            freq = 1.0f / powf(theta, (float)(2j) / (float)dim), angle = (float)p * freq, cosf / sinf;
 *   double : FLUX.3 (iris_transformer_flux3.c:282-294):
 *            freq = 1.0 / pow(theta, (double)(2j) / dim), angle = p * freq, cos / sin, rounded to float.
 *
 * So this file has one position builder per model and one expansion engine
 * with the two arithmetic modes. The engine evaluates each distinct
 * (axis, position) once and copies it to the rows that share it: an image of
 * h x w cells has h + w distinct positions per axis, not h * w, which takes
 * the libm work of a 4608-row table from 590 k calls to a few thousand.
 * Reuse cannot change a value: libm's functions are deterministic, and the
 * arguments are formed exactly as written above. An axis the reference writes
 * as the constants (1, 0) is a position-0 axis here: cosf(0) = 1 and
 * sinf(0) = 0 exactly.
 *
 * No device code and no dependency on the HIP runtime in this file.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "iris_rope.h"
#include "iris_rope_internal.h"

#define MAX_AXES 8
#define MEMO_SLOTS 1024            /* per axis, direct mapped */

typedef struct {
    int cols;                      /* axis_dim / 2 */
    float *freq32;                 /* [cols] */
    double *freq64;                /* [cols] */
    uint32_t *key;                 /* [MEMO_SLOTS] position bits held by each slot */
    unsigned char *used;           /* [MEMO_SLOTS] */
    float *cs;                     /* [MEMO_SLOTS][2][cols]: cos row then sin row */
} axis_memo;

/* the one place the column frequencies are written down */
static float iris_rope_freq32_(float theta, int j, int dim) { return 1.0f / powf(theta, (float)(2 * j) / (float)dim); }
static double iris_rope_freq64_(float theta, int j, int dim) { return 1.0 / pow(theta, (double)(2 * j) / dim); }

static void memo_free(axis_memo *m, int naxes) {
    for (int a = 0; a < naxes; a++) {
        free(m[a].freq32); free(m[a].freq64); free(m[a].key); free(m[a].used); free(m[a].cs);
    }
}

static int memo_init(axis_memo *m, int naxes, const int *axis_dims, float theta, int use_double) {
    memset(m, 0, sizeof(axis_memo) * (size_t)naxes);
    for (int a = 0; a < naxes; a++) {
        const int dim = axis_dims[a], cols = dim / 2;
        m[a].cols = cols;
        m[a].freq32 = malloc(sizeof(float) * (size_t)(cols ? cols : 1));
        m[a].freq64 = malloc(sizeof(double) * (size_t)(cols ? cols : 1));
        m[a].key = malloc(sizeof(uint32_t) * MEMO_SLOTS);
        m[a].used = calloc(MEMO_SLOTS, 1);
        m[a].cs = malloc(sizeof(float) * 2 * (size_t)(cols ? cols : 1) * MEMO_SLOTS);
        if (!m[a].freq32 || !m[a].freq64 || !m[a].key || !m[a].used || !m[a].cs) {
            memo_free(m, naxes);
            return 0;
        }
        for (int j = 0; j < cols; j++) {
            if (use_double) m[a].freq64[j] = iris_rope_freq64_(theta, j, dim);
            else m[a].freq32[j] = iris_rope_freq32_(theta, j, dim);
        }
    }
    return 1;
}

/* The one place a table entry is evaluated: cos row then sin row of one (axis, position). */
static void eval_row(float *row, int cols, const float *freq32, const double *freq64, float value, int use_double) {
    for (int j = 0; j < cols; j++) {
        if (use_double) {
            const double angle = value * freq64[j];
            row[j] = (float)cos(angle);
            row[cols + j] = (float)sin(angle);
        } else {
            const float angle = value * freq32[j];
            row[j] = cosf(angle);
            row[cols + j] = sinf(angle);
        }
    }
}

/* cos / sin rows of one (axis, position); bits identify the position, value is what is multiplied */
static const float *memo_row(axis_memo *m, uint32_t bits, float value, int use_double) {
    const uint32_t slot = (bits * 2654435761u) >> 22;          /* top 10 bits of a Fibonacci hash */
    float *row = m->cs + (size_t)slot * 2 * m->cols;
    if (m->used[slot] && m->key[slot] == bits) return row;
    eval_row(row, m->cols, m->freq32, m->freq64, value, use_double);
    m->used[slot] = 1;
    m->key[slot] = bits;
    return row;
}

static int axes_ok(int seq, int naxes, const int *axis_dims) {
    if (seq < 0 || naxes < 1 || naxes > MAX_AXES || !axis_dims) return 0;
    for (int a = 0; a < naxes; a++)
        if (axis_dims[a] < 0 || (axis_dims[a] & 1)) return 0;
    return 1;
}

int iris_rope_expand_i32(float *cos_t, float *sin_t, const int *pos, int seq, int naxes,
                         const int *axis_dims, const int *axis_lens, float theta) {
    axis_memo memo[MAX_AXES];
    if (!axes_ok(seq, naxes, axis_dims) || (seq && (!cos_t || !sin_t || !pos))) return -1;
    if (!memo_init(memo, naxes, axis_dims, theta, 0)) return -1;
    size_t half = 0;
    for (int a = 0; a < naxes; a++) half += (size_t)memo[a].cols;
    for (int s = 0; s < seq; s++) {
        float *c = cos_t + (size_t)s * half, *sn = sin_t + (size_t)s * half;
        for (int a = 0; a < naxes; a++) {
            int p = pos[(size_t)s * naxes + a];
            if (axis_lens && (p < 0 || p >= axis_lens[a])) p = 0;     /* out of range: unrotated */
            const float *row = memo_row(&memo[a], (uint32_t)p, (float)p, 0);
            memcpy(c, row, sizeof(float) * (size_t)memo[a].cols);
            memcpy(sn, row + memo[a].cols, sizeof(float) * (size_t)memo[a].cols);
            c += memo[a].cols;
            sn += memo[a].cols;
        }
    }
    memo_free(memo, naxes);
    return 0;
}

int iris_rope_expand_f64(float *cos_t, float *sin_t, const float *pos, int seq, int naxes,
                         const int *axis_dims, float theta) {
    axis_memo memo[MAX_AXES];
    if (!axes_ok(seq, naxes, axis_dims) || (seq && (!cos_t || !sin_t || !pos))) return -1;
    if (!memo_init(memo, naxes, axis_dims, theta, 1)) return -1;
    size_t half = 0;
    for (int a = 0; a < naxes; a++) half += (size_t)memo[a].cols;
    for (int s = 0; s < seq; s++) {
        float *c = cos_t + (size_t)s * half, *sn = sin_t + (size_t)s * half;
        for (int a = 0; a < naxes; a++) {
            const float p = pos[(size_t)s * naxes + a];
            uint32_t bits;
            memcpy(&bits, &p, sizeof bits);
            const float *row = memo_row(&memo[a], bits, p, 1);
            memcpy(c, row, sizeof(float) * (size_t)memo[a].cols);
            memcpy(sn, row + memo[a].cols, sizeof(float) * (size_t)memo[a].cols);
            c += memo[a].cols;
            sn += memo[a].cols;
        }
    }
    memo_free(memo, naxes);
    return 0;
}

/* ---- dictionary form, for the device entries ------------------------------------------------ */

/* The same table as a dictionary: `values` holds, for every distinct (axis, position) of the
 * sequence, the cos row and the sin row of that axis (2 * axis_dim / 2 floats, evaluated by
 * eval_row like the tables above), and index[s * naxes + a] is the offset in floats of the pair of
 * rows that row s uses on axis a. Expanding it is pure copying, so a table gathered from the
 * dictionary has the bits of the table built here directly. pos is int32 [seq][naxes]
 * (use_double 0, axis_lens as in iris_rope_expand_i32) or float (use_double 1). Returns 0 and
 * malloc'd arrays, or -1. */
int iris_rope_dictionary_(const void *pos, int use_double, int seq, int naxes, const int *axis_dims,
                          const int *axis_lens, float theta, float **values, size_t *n_values, uint32_t **index) {
    axis_memo memo[MAX_AXES];
    *values = NULL; *index = NULL; *n_values = 0;
    if (!axes_ok(seq, naxes, axis_dims) || (seq && !pos)) return -1;
    if (!memo_init(memo, naxes, axis_dims, theta, use_double)) return -1;
    /* open-addressing map position bits -> offset, one per axis, at most half full */
    size_t cap = 16;
    while (cap < 2 * (size_t)seq) cap <<= 1;
    uint32_t *keys = malloc(sizeof(uint32_t) * cap), *offs = malloc(sizeof(uint32_t) * cap);
    unsigned char *used = malloc(cap);
    uint32_t *idx = malloc(sizeof(uint32_t) * (size_t)(seq ? seq : 1) * (size_t)naxes);
    size_t room = 1024, n = 0;
    float *vals = malloc(sizeof(float) * room);
    int ok = keys && offs && used && idx && vals;
    for (int a = 0; ok && a < naxes; a++) {
        const int cols = memo[a].cols;
        memset(used, 0, cap);
        for (int s = 0; ok && s < seq; s++) {
            uint32_t bits;
            float value;
            if (use_double) {
                value = ((const float *)pos)[(size_t)s * naxes + a];
                memcpy(&bits, &value, sizeof bits);
            } else {
                int p = ((const int *)pos)[(size_t)s * naxes + a];
                if (axis_lens && (p < 0 || p >= axis_lens[a])) p = 0;     /* out of range: unrotated */
                bits = (uint32_t)p;
                value = (float)p;
            }
            size_t slot = (size_t)((bits * 2654435761u) >> 4) & (cap - 1);
            while (used[slot] && keys[slot] != bits) slot = (slot + 1) & (cap - 1);
            if (!used[slot]) {
                if (n + 2 * (size_t)cols > room) {
                    while (n + 2 * (size_t)cols > room) room *= 2;
                    float *grown = realloc(vals, sizeof(float) * room);
                    if (!grown) { ok = 0; break; }
                    vals = grown;
                }
                if (n + 2 * (size_t)cols >= 0x80000000u) { ok = 0; break; }    /* offsets are 32 bits */
                eval_row(vals + n, cols, memo[a].freq32, memo[a].freq64, value, use_double);
                used[slot] = 1;
                keys[slot] = bits;
                offs[slot] = (uint32_t)n;
                n += 2 * (size_t)cols;
            }
            idx[(size_t)s * naxes + a] = offs[slot];
        }
    }
    memo_free(memo, naxes);
    free(keys); free(offs); free(used);
    if (!ok) { free(idx); free(vals); return -1; }
    *values = vals; *n_values = n; *index = idx;
    return 0;
}

/* ---- joint [text | image | refs] layouts -------------------------------------------------- */

int iris_rope_joint_rows(int txt_seq, int img_h, int img_w, const int *ref_h, const int *ref_w, int num_refs) {
    long rows = (long)txt_seq + (long)img_h * img_w;
    for (int i = 0; i < num_refs; i++) rows += (long)ref_h[i] * ref_w[i];
    return rows > 0x7fffffffL || rows < 0 ? -1 : (int)rows;
}

void iris_rope_flux2_positions(int *pos4, int txt_seq, int img_h, int img_w,
                               const int *ref_h, const int *ref_w, const int *ref_t, int num_refs) {
    int *p = pos4;
    for (int t = 0; t < txt_seq; t++, p += 4) { p[0] = 0; p[1] = 0; p[2] = 0; p[3] = t; }
    for (int g = -1; g < num_refs; g++) {
        const int h = g < 0 ? img_h : ref_h[g], w = g < 0 ? img_w : ref_w[g];
        const int t = g < 0 ? 0 : (ref_t ? ref_t[g] : 10 * (g + 1));
        for (int y = 0; y < h; y++)
            for (int x = 0; x < w; x++, p += 4) { p[0] = t; p[1] = y; p[2] = x; p[3] = 0; }
    }
}

int iris_rope_flux2_tables(float *cos_t, float *sin_t, int txt_seq, int img_h, int img_w,
                           const int *ref_h, const int *ref_w, const int *ref_t, int num_refs,
                           int axis_dim, float theta) {
    const int rows = iris_rope_joint_rows(txt_seq, img_h, img_w, ref_h, ref_w, num_refs);
    if (rows < 0) return -1;
    int *pos = malloc(sizeof(int) * 4 * (size_t)(rows ? rows : 1));
    if (!pos) return -1;
    iris_rope_flux2_positions(pos, txt_seq, img_h, img_w, ref_h, ref_w, ref_t, num_refs);
    const int dims[4] = { axis_dim, axis_dim, axis_dim, axis_dim };
    const int rc = iris_rope_expand_i32(cos_t, sin_t, pos, rows, 4, dims, NULL, theta);
    free(pos);
    return rc;
}

void iris_rope_flux3_positions(float *pos4, int txt_seq, int img_h, int img_w,
                               const int *ref_h, const int *ref_w, int num_refs) {
    float *p = pos4;
    for (int s = 0; s < txt_seq; s++, p += 4) { p[0] = 0.0f; p[1] = 0.0f; p[2] = 0.0f; p[3] = (float)s; }
    for (int g = -1; g < num_refs; g++) {
        const int h = g < 0 ? img_h : ref_h[g], w = g < 0 ? img_w : ref_w[g];
        const float l = g < 0 ? 0.0f : -(float)(g + 1);
        for (int r = 0; r < h; r++)
            for (int c = 0; c < w; c++, p += 4) { p[0] = 0.0f; p[1] = 0.5f * r; p[2] = 0.5f * c; p[3] = l; }
    }
}

int iris_rope_flux3_tables(float *cos_t, float *sin_t, int txt_seq, int img_h, int img_w,
                           const int *ref_h, const int *ref_w, int num_refs,
                           const int axes_dim[4], float theta) {
    const int rows = iris_rope_joint_rows(txt_seq, img_h, img_w, ref_h, ref_w, num_refs);
    if (rows < 0) return -1;
    float *pos = malloc(sizeof(float) * 4 * (size_t)(rows ? rows : 1));
    if (!pos) return -1;
    iris_rope_flux3_positions(pos, txt_seq, img_h, img_w, ref_h, ref_w, num_refs);
    const int rc = iris_rope_expand_f64(cos_t, sin_t, pos, rows, 4, axes_dim, theta);
    free(pos);
    return rc;
}

/* ---- Z-Image ------------------------------------------------------------------------------- */

void iris_rope_zimage_positions(int *pos3, int *mask, int img_seq, int wt, int cap_seq,
                                int *img_pad, int *cap_pad) {
    const int ip = (img_seq + 31) & ~31, cp = (cap_seq + 31) & ~31;
    for (int s = 0; s < ip; s++) {
        const int live = s < img_seq;
        pos3[3 * s + 0] = live ? cp + 1 : 0;
        pos3[3 * s + 1] = live ? s / wt : 0;
        pos3[3 * s + 2] = live ? s % wt : 0;
        mask[s] = live;
    }
    for (int s = 0; s < cp; s++) {
        int *p = pos3 + 3 * (size_t)(ip + s);
        p[0] = 1 + s; p[1] = 0; p[2] = 0;
        mask[ip + s] = s < cap_seq;
    }
    if (img_pad) *img_pad = ip;
    if (cap_pad) *cap_pad = cp;
}

int iris_rope_zimage_tables(float *cos_t, float *sin_t, const int *pos3, int seq,
                            const int axes_dims[3], const int axes_lens[3], float theta) {
    return iris_rope_expand_i32(cos_t, sin_t, pos3, seq, 3, axes_dims, axes_lens, theta);
}

/* ---- Qwen3 --------------------------------------------------------------------------------- */

/* positions of the text encoder's rows; returns a malloc'd array (NULL on failure) */
static int *qwen3_positions(const int *attention_mask, int seq, int pad_at_one) {
    int *pos = malloc(sizeof(int) * (size_t)(seq > 0 ? seq : 1));
    if (!pos) return NULL;
    for (int s = 0; s < seq; s++)
        pos[s] = (pad_at_one && attention_mask && !attention_mask[s]) ? 1 : s;
    return pos;
}

int iris_rope_qwen3_tables(float *cos_t, float *sin_t, const int *attention_mask, int seq,
                           int head_dim, float theta, int pad_at_one) {
    if (seq < 0) return -1;
    int *pos = qwen3_positions(attention_mask, seq, pad_at_one);
    if (!pos) return -1;
    const int rc = iris_rope_expand_i32(cos_t, sin_t, pos, seq, 1, &head_dim, NULL, theta);
    free(pos);
    return rc;
}

int *iris_rope_qwen3_positions_(const int *attention_mask, int seq, int pad_at_one) {
    return qwen3_positions(attention_mask, seq, pad_at_one);
}

int iris_rope_axes_ok_(int seq, int naxes, const int *axis_dims) { return axes_ok(seq, naxes, axis_dims); }
