/*
 * CPU timing baseline -- TEST / BENCH INFRASTRUCTURE ONLY (never shipped,
 * never called by the product library).
 *
 * Restates the structure of the reference's BLAS-build CPU attention:
 * heads are distributed over pthreads, and each head runs
 *     sgemm(scale * Q K^T) -> max-subtracted softmax with the polynomial exp
 *     -> sgemm(P V)
 * on rows strided by the hidden size (iris_transformer_flux.c:1499-1519,
 * 1530-1565; thread count rule :1569-1579). With q_chunk > 0 the queries of
 * a head are processed in chunks so the score buffer stays bounded, as the
 * FLUX.3 CPU path does (iris_transformer_flux3.c:204-247). The causal /
 * padding-mask / grouped-kv variant sets masked scores to -1e9 after the
 * scaled product (iris_qwen3.c:415-491, iris_transformer_zimage.c:729-768).
 *
 * sgemm provider: resolved at run time with dlopen -- a system OpenBLAS, a
 * bundled OpenBLAS whose path the caller passes in, or the plain blocked
 * loop below (reported as provider "own").
 */
#define _GNU_SOURCE
#include <dlfcn.h>
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>

enum { ROW_MAJOR = 101, NO_TRANS = 111, TRANS = 112 };
typedef void (*sgemm_fn)(int order, int ta, int tb, int m, int n, int k, float alpha,
                         const float *a, int lda, const float *b, int ldb, float beta,
                         float *c, int ldc);
typedef void (*set_threads_fn)(int);

static sgemm_fn g_sgemm = NULL;
static char g_provider[512] = "own";

/* Fallback sgemm (row major, C = alpha * A * op(B) + 0): correct, not fast. */
static void own_sgemm(int order, int ta, int tb, int m, int n, int k, float alpha,
                      const float *a, int lda, const float *b, int ldb, float beta,
                      float *c, int ldc) {
    (void)order; (void)ta; (void)beta;
    for (int i = 0; i < m; i++) {
        float *ci = c + (size_t)i * ldc;
        if (tb == TRANS) {
            for (int j = 0; j < n; j++) {
                const float *ai = a + (size_t)i * lda, *bj = b + (size_t)j * ldb;
                float acc = 0.0f;
                for (int p = 0; p < k; p++) acc += ai[p] * bj[p];
                ci[j] = alpha * acc;
            }
        } else {
            for (int j = 0; j < n; j++) ci[j] = 0.0f;
            for (int p = 0; p < k; p++) {
                float av = alpha * a[(size_t)i * lda + p];
                const float *bp = b + (size_t)p * ldb;
                for (int j = 0; j < n; j++) ci[j] += av * bp[j];
            }
        }
    }
}

/* Try to bind cblas_sgemm from `path` (NULL: well-known system names).
 * `prefix` is prepended to the symbol names ("" or "scipy_"). Returns 1 on
 * success. BLAS-internal threading is switched off: heads are the unit of
 * parallelism, as in the reference. */
int cpu_baseline_bind_blas(const char *path, const char *prefix) {
    const char *sys[] = {"libopenblas.so.0", "libopenblas.so", NULL};
    void *h = NULL;
    if (path) h = dlopen(path, RTLD_NOW | RTLD_LOCAL);
    else for (int i = 0; sys[i] && !h; i++) { h = dlopen(sys[i], RTLD_NOW | RTLD_LOCAL); path = sys[i]; }
    if (!h) return 0;
    char name[128];
    snprintf(name, sizeof(name), "%scblas_sgemm", prefix ? prefix : "");
    sgemm_fn f = (sgemm_fn)dlsym(h, name);
    if (!f) return 0;
    snprintf(name, sizeof(name), "%sopenblas_set_num_threads", prefix ? prefix : "");
    set_threads_fn st = (set_threads_fn)dlsym(h, name);
    if (st) st(1);
    g_sgemm = f;
    snprintf(g_provider, sizeof(g_provider), "%s", path);
    return 1;
}

const char *cpu_baseline_provider(void) { return g_provider; }

int cpu_baseline_online_cpus(void) { return (int)sysconf(_SC_NPROCESSORS_ONLN); }

/* Largest divisor of `heads` that is <= the CPU limit
 * (iris_transformer_flux.c:1569-1579). limit <= 0 means the online CPUs. */
int cpu_baseline_threads(int heads, int limit) {
    int n = limit > 0 ? limit : cpu_baseline_online_cpus();
    if (n < 2) return 1;
    if (n > heads) n = heads;
    while (heads % n) n--;
    return n;
}

static inline float poly_expf(float x) {   /* iris_kernels.h:21-32 */
    if (x < -87.3f) return 0.0f;
    if (x > 88.7f) return 1e38f;
    float n = floorf(x * 1.4426950408889634f + 0.5f);
    float r = x - n * 0.6931471805599453f;
    float p = 1.0f + r * (1.0f + r * (0.5f + r * (0.16666667f + r * (0.04166667f + r * 0.00833333f))));
    int32_t b;
    memcpy(&b, &p, 4);
    b += (int32_t)n << 23;
    memcpy(&p, &b, 4);
    return p;
}

static void softmax_rows(float *x, int rows, int cols) {   /* iris_kernels.c:611-634 */
    for (int r = 0; r < rows; r++) {
        float *v = x + (size_t)r * cols, mx = v[0], sum = 0.0f;
        for (int c = 1; c < cols; c++) if (v[c] > mx) mx = v[c];
        for (int c = 0; c < cols; c++) { v[c] = poly_expf(v[c] - mx); sum += v[c]; }
        float inv = 1.0f / sum;
        for (int c = 0; c < cols; c++) v[c] *= inv;
    }
}

typedef struct {
    float *out; const float *q, *k, *v;
    int ldo, ldq, ldkv, seq_q, seq_k, hd, per_kv, q_chunk, causal;
    const int *key_mask;
    float scale;
    int h0, h1;
    int failed;
} job_t;

static void *worker(void *arg) {
    job_t *w = (job_t *)arg;
    sgemm_fn mm = g_sgemm ? g_sgemm : own_sgemm;
    int chunk = w->q_chunk > 0 && w->q_chunk < w->seq_q ? w->q_chunk : w->seq_q;
    float *sc = (float *)malloc((size_t)chunk * w->seq_k * sizeof(float));
    if (!sc) { w->failed = 1; return NULL; }
    for (int h = w->h0; h < w->h1; h++) {
        int g = h / w->per_kv;
        const float *qh = w->q + (size_t)h * w->hd;
        const float *kh = w->k + (size_t)g * w->hd, *vh = w->v + (size_t)g * w->hd;
        float *oh = w->out + (size_t)h * w->hd;
        for (int q0 = 0; q0 < w->seq_q; q0 += chunk) {
            int nq = w->seq_q - q0 < chunk ? w->seq_q - q0 : chunk;
            mm(ROW_MAJOR, NO_TRANS, TRANS, nq, w->seq_k, w->hd, w->scale,
               qh + (size_t)q0 * w->ldq, w->ldq, kh, w->ldkv, 0.0f, sc, w->seq_k);
            if (w->causal || w->key_mask)
                for (int i = 0; i < nq; i++) {
                    float *row = sc + (size_t)i * w->seq_k;
                    for (int j = 0; j < w->seq_k; j++) {
                        if (w->causal && j > q0 + i) row[j] = -1e9f;
                        if (w->key_mask && !w->key_mask[j]) row[j] = -1e9f;
                    }
                }
            softmax_rows(sc, nq, w->seq_k);
            mm(ROW_MAJOR, NO_TRANS, NO_TRANS, nq, w->hd, w->seq_k, 1.0f, sc, w->seq_k,
               vh, w->ldkv, 0.0f, oh + (size_t)q0 * w->ldo, w->ldo);
        }
    }
    free(sc);
    return NULL;
}

/* f32 attention over strided [seq, heads*hd] rows with heads split over
 * `threads` pthreads (0: the reference's rule). Returns the thread count
 * used, or -1 when a score buffer could not be allocated. */
int cpu_baseline_attention(float *out, int ldo, const float *q, const float *k, const float *v,
                           int ldq, int ldkv, int seq_q, int seq_k, int heads, int kv_heads,
                           int hd, float scale, int causal, const int *key_mask,
                           int q_chunk, int threads) {
    int nt = cpu_baseline_threads(heads, threads);
    pthread_t tid[256];
    job_t jobs[256];
    int started[256];
    if (nt > 256) nt = 256;
    while (heads % nt) nt--;
    int per = heads / nt;
    for (int t = 0; t < nt; t++) {
        jobs[t] = (job_t){out, q, k, v, ldo, ldq, ldkv, seq_q, seq_k, hd, heads / kv_heads,
                          q_chunk, causal, key_mask, scale, t * per, (t + 1) * per, 0};
        started[t] = nt > 1 && pthread_create(&tid[t], NULL, worker, &jobs[t]) == 0;
        if (!started[t]) worker(&jobs[t]);
    }
    int bad = 0;
    for (int t = 0; t < nt; t++) {
        if (started[t]) pthread_join(tid[t], NULL);
        bad |= jobs[t].failed;
    }
    return bad ? -1 : nt;
}

/* Per-head RMSNorm then pair rotation on f32 [seq, heads*hd], the scalar
 * loops of the CPU models (iris_transformer_flux.c:1316-1341, 952-974;
 * split-half form iris_qwen3.c:317-360). Single thread, as in the reference. */
void cpu_baseline_norm_rope(float *x, const float *w, const float *cos_t, const float *sin_t,
                            int seq, int heads, int hd, float eps, int split_half) {
    int half = hd / 2;
    for (int s = 0; s < seq; s++)
        for (int h = 0; h < heads; h++) {
            float *v = x + ((size_t)s * heads + h) * hd, ss = 0.0f;
            for (int d = 0; d < hd; d++) ss += v[d] * v[d];
            float inv = 1.0f / sqrtf(ss / hd + eps);
            for (int d = 0; d < hd; d++) v[d] = v[d] * inv * w[d];
        }
    for (int s = 0; s < seq; s++) {
        const float *c = cos_t + (size_t)s * half, *sn = sin_t + (size_t)s * half;
        for (int h = 0; h < heads; h++) {
            float *v = x + ((size_t)s * heads + h) * hd;
            for (int i = 0; i < half; i++) {
                int i0 = split_half ? i : 2 * i, i1 = split_half ? i + half : 2 * i + 1;
                float a = v[i0], b = v[i1];
                v[i0] = a * c[i] - b * sn[i];
                v[i1] = b * c[i] + a * sn[i];
            }
        }
    }
}
