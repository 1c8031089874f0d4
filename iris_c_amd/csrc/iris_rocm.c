/*
 * Host side of the MI355X backend: plain C over the HIP runtime C API.
 * Owns the device state (one stream, device 0), the memory entries, and the
 * argument checks that choose a kernel for the two hot-path operators. The
 * kernels themselves live in the .hip files and are reached through the
 * launchers of iris_kernels_hip.h.
 *
 * Behaviour follows the reference backend (iris_cuda.cu:108-230, 445-453,
 * 878-937): compute entries never abort and never return a status; a failure
 * is one line on stderr prefixed "iris_dev:". There is no CPU fallback: if
 * the device is missing or the library was not initialised, the entries
 * report the error and leave the output untouched.
 */
#include <hip/hip_runtime_api.h>

#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "iris_dev.h"
#include "iris_kernels_hip.h"
#include "iris_rope.h"
#include "iris_rope_internal.h"

static int g_ready = 0;
static char g_name[640] = "none";
static hipStream_t g_stream = NULL;
static int g_last_error = 0;
static const char *g_last_kernel = "none";
/* private scratch, allocated on first use and kept until cleanup (as the reference backend
 * does, iris_cuda.cu:149-173): convolution patches and group-norm partial sums */
#ifndef IRIS_DEV_PATH_ONLY
#define CONV_SCRATCH_BYTES ((size_t)256 << 20)
static uint16_t *g_conv_scratch = NULL;
static float *g_gn_scratch = NULL;
static size_t g_gn_scratch_floats = 0;
#endif
/* normalised copy of Q for the iris_dev_attention_qnorm calls that the matrix-core kernel does not take */
static uint16_t *g_q_scratch = NULL;
static size_t g_q_scratch_bytes = 0;
/* padded, aligned copy of q | k | v (and the padded output) for attention calls on other head sizes or alignments */
static uint16_t *g_pack = NULL;
static size_t g_pack_bytes = 0;
/* partial results of the key ranges of a head_dim-512 attention call (f32 rows, maxima and sums) */
static void *g_split = NULL;
static size_t g_split_bytes = 0;
#ifndef IRIS_DEV_PATH_ONLY
/* staging buffer of the rotary tables being expanded: column map, row offsets, dictionary */
static void *g_rope_stage = NULL;
static size_t g_rope_stage_bytes = 0;
#endif

static void fail(int code, const char *what, const char *detail) {
    g_last_error = code ? code : -1;
    fprintf(stderr, "iris_dev: %s failed: %s\n", what, detail);
}

static int check(hipError_t err, const char *what) {
    if (err == hipSuccess) return 1;
    fail((int)err, what, hipGetErrorString(err));
    return 0;
}

static int need_ready(const char *what) {
    if (g_ready) return 1;
    fail(-1, what, "device not initialised (iris_dev_init() did not succeed)");
    return 0;
}

#ifndef IRIS_DEV_PATH_ONLY
int iris_dev_init(void) {
    if (g_ready) return 1;
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count == 0) return 0;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, 0) != hipSuccess) return 0;
    /* The kernels are compiled for gfx950 only. */
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        fprintf(stderr, "iris_dev: device 0 is %s, this backend needs gfx950\n", prop.gcnArchName);
        return 0;
    }
    if (hipSetDevice(0) != hipSuccess) return 0;
    /* some hosts report an empty marketing name */
    snprintf(g_name, sizeof(g_name), "%s (%s, %d CUs, %d MHz)", prop.name[0] ? prop.name : "AMD Instinct",
             prop.gcnArchName, prop.multiProcessorCount, prop.clockRate / 1000);
    if (hipStreamCreate(&g_stream) != hipSuccess) return 0;
    /* address of the in-library scratch of iris_dev_group_norm_noalloc on this device; if the lookup
     * fails here the entry point tries again at its first call and reports it there */
    (void)iris_hip_group_norm_static_setup();
    g_ready = 1;
    g_last_error = 0;
    return 1;
}

#endif

#ifndef IRIS_DEV_PATH_ONLY
int iris_dev_available(void) { return g_ready; }
const char *iris_dev_name(void) { return g_name; }
void *iris_dev_stream(void) { return (void *)g_stream; }
#endif
const char *iris_dev_last_kernel(void) { return g_last_kernel; }

int iris_dev_last_error(void) {
    int e = g_last_error;
    g_last_error = 0;
    return e;
}

#ifndef IRIS_DEV_PATH_ONLY
void iris_dev_cleanup(void) {
    if (!g_ready) return;
    check(hipStreamSynchronize(g_stream), "sync");
    if (g_conv_scratch) check(hipFree(g_conv_scratch), "free");
    if (g_gn_scratch) check(hipFree(g_gn_scratch), "free");
    if (g_rope_stage) check(hipFree(g_rope_stage), "free");
    if (g_q_scratch) check(hipFree(g_q_scratch), "free");
    if (g_pack) check(hipFree(g_pack), "free");
    if (g_split) check(hipFree(g_split), "free");
    g_pack = NULL;
    g_pack_bytes = 0;
    g_split = NULL;
    g_split_bytes = 0;
    g_q_scratch = NULL;
    g_q_scratch_bytes = 0;
    iris_lt_release();
    g_conv_scratch = NULL;
    g_gn_scratch = NULL;
    g_gn_scratch_floats = 0;
    g_rope_stage = NULL;
    g_rope_stage_bytes = 0;
    check(hipStreamDestroy(g_stream), "stream destroy");
    g_stream = NULL;
    g_ready = 0;
}

void *iris_dev_alloc(size_t bytes) {
    void *p = NULL;
    if (!need_ready("alloc")) return NULL;
    if (hipMalloc(&p, bytes ? bytes : 1) != hipSuccess) {
        (void)hipGetLastError();
        return NULL;
    }
    return p;
}

void iris_dev_free(void *p) {
    if (!p || !need_ready("free")) return;
    check(hipStreamSynchronize(g_stream), "sync");   /* pending work may still use the buffer */
    check(hipFree(p), "free");
}

void iris_dev_upload_2d(void *dst, size_t dst_stride, const void *src, size_t src_stride,
                        size_t row_bytes, size_t rows) {
    if (!need_ready("upload") || !row_bytes || !rows) return;
    check(hipMemcpy2DAsync(dst, dst_stride, src, src_stride, row_bytes, rows,
                           hipMemcpyHostToDevice, g_stream), "upload");
    check(hipStreamSynchronize(g_stream), "sync");
}

void iris_dev_upload(void *dst, const void *src, size_t bytes) {
    if (!need_ready("upload") || !bytes) return;
    check(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, g_stream), "upload");
    check(hipStreamSynchronize(g_stream), "sync");
}

void iris_dev_download(void *dst, const void *src, size_t bytes) {
    if (!need_ready("download")) return;
    if (bytes) check(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, g_stream), "download");
    check(hipStreamSynchronize(g_stream), "sync");
}

void iris_dev_sync(void) {
    if (!need_ready("sync")) return;
    check(hipStreamSynchronize(g_stream), "sync");
}

#else
/* Path-only build (libiris_dev_path.a): the two hot-path operators for a host backend that keeps its own setup,
 * memory entries and stream. The host attaches the stream its other work runs on; the operators enqueue there. */
void iris_dev_path_attach(void *hip_stream) {
    (void)g_name;
    g_stream = (hipStream_t)hip_stream;
    g_ready = 1;
    g_last_error = 0;
}

void iris_dev_path_detach(void) {
    if (!g_ready) return;
    check(hipStreamSynchronize(g_stream), "sync");
    if (g_q_scratch) check(hipFree(g_q_scratch), "free");
    if (g_pack) check(hipFree(g_pack), "free");
    if (g_split) check(hipFree(g_split), "free");
    g_q_scratch = NULL;
    g_q_scratch_bytes = 0;
    g_pack = NULL;
    g_pack_bytes = 0;
    g_split = NULL;
    g_split_bytes = 0;
    g_stream = NULL;
    g_ready = 0;
}
#endif

static int aligned(const void *p, size_t a) { return ((uintptr_t)p & (a - 1)) == 0; }

/* Private scratch that only grows: makes *p hold at least `need` bytes (the old block is released once the
 * work that may still read it has drained). Returns 0 after reporting a failed allocation. */
static int scratch_fit(void **p, size_t *have, size_t need, const char *what) {
    if (need <= *have) return 1;
    /* Growing means synchronise + free + allocate, none of which may happen while the stream is being captured into
     * a graph (it would invalidate the capture): the call is refused with a message instead. A caller that captures a
     * layout served through private scratch issues the call once outside the capture first; the scratch then fits. */
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(g_stream, &capturing) == hipSuccess && capturing != hipStreamCaptureStatusNone) {
        fail(-1, what, "this layout needs private scratch that has to grow, which cannot happen during stream capture: "
                       "issue the same call once before the capture");
        return 0;
    }
    if (*p) {
        check(hipStreamSynchronize(g_stream), "sync");
        check(hipFree(*p), "free");
    }
    *p = NULL;
    *have = 0;
    if (hipMalloc(p, need) != hipSuccess) {
        (void)hipGetLastError();
        *p = NULL;
        fail(-1, what, "scratch allocation failed");
        return 0;
    }
    *have = need;
    return 1;
}

/* Shared by the one- and two-tensor entries; xk may be NULL with k_heads 0. */
static void norm_rope_streams(uint16_t *xq, uint16_t *xk, int ld, const float *wq, const float *wk,
                              const float *wq_b, const float *wk_b, int rows_a,
                              const float *rope_cos, const float *rope_sin, int seq, int q_heads,
                              int k_heads, int head_dim, float eps, int split_half) {
    if (!need_ready("head_norm_rope")) return;
    if (seq <= 0 || q_heads + k_heads <= 0) return;
    if (head_dim <= 0 || (head_dim & 1)) {                   /* the reference takes powers of two up to 2048 (iris_cuda.cu:445-453) */
        fail(-1, "head_norm_rope", "head_dim must be even");
        return;
    }
    int fast = head_dim == 128 && ld % 8 == 0 && aligned(xq, 16) && aligned(wq, 16) &&
               aligned(rope_cos, 16) && aligned(rope_sin, 16) &&
               (long long)seq * (q_heads + k_heads) < (1 << 24) && q_heads + k_heads < 256;
    if (k_heads > 0) fast = fast && aligned(xk, 16) && aligned(wk, 16);
    if (wq_b) fast = fast && aligned(wq_b, 16) && (k_heads == 0 || aligned(wk_b, 16));
    int err;
    if (fast) {
        g_last_kernel = "norm_rope_hd128";
        err = iris_hip_norm_rope_hd128_streams(g_stream, xq, xk, ld, wq, wk, wq_b, wk_b, rows_a, rope_cos, rope_sin, seq,
                                               q_heads, k_heads, eps, split_half != 0);
    } else {
        /* row range by row range (one when there is no second weight pair), tensor by tensor */
        g_last_kernel = "norm_rope_generic";
        err = 0;
        for (int part = 0; part < (wq_b ? 2 : 1) && !err; part++) {
            const int first = part ? rows_a : 0, n = wq_b ? (part ? seq - rows_a : rows_a) : seq;
            const float *c = rope_cos + (size_t)first * (head_dim / 2), *sn = rope_sin + (size_t)first * (head_dim / 2);
            if (n <= 0) continue;
            err = iris_hip_norm_rope_generic(g_stream, xq + (size_t)first * ld, ld, part ? wq_b : wq, c, sn, n, q_heads,
                                             head_dim, eps, split_half != 0);
            if (!err && k_heads > 0)
                err = iris_hip_norm_rope_generic(g_stream, xk + (size_t)first * ld, ld, part ? wk_b : wk, c, sn, n,
                                                 k_heads, head_dim, eps, split_half != 0);
        }
    }
    if (err) check((hipError_t)err, "head_norm_rope launch");
}

static void norm_rope(uint16_t *xq, uint16_t *xk, int ld, const float *wq, const float *wk,
                      const float *rope_cos, const float *rope_sin, int seq, int q_heads,
                      int k_heads, int head_dim, float eps, int split_half) {
    norm_rope_streams(xq, xk, ld, wq, wk, NULL, NULL, 0, rope_cos, rope_sin, seq, q_heads, k_heads, head_dim, eps, split_half);
}

void iris_dev_head_norm_rope(uint16_t *x, int ld, const float *w,
                             const float *rope_cos, const float *rope_sin,
                             int seq, int heads, int head_dim, float eps, int split_half) {
    norm_rope(x, NULL, ld, w, NULL, rope_cos, rope_sin, seq, heads, 0, head_dim, eps, split_half);
}

void iris_dev_head_norm_rope_qk(uint16_t *xq, uint16_t *xk, int ld,
                                const float *wq, const float *wk,
                                const float *rope_cos, const float *rope_sin,
                                int seq, int q_heads, int k_heads, int head_dim,
                                float eps, int split_half) {
    norm_rope(xq, xk, ld, wq, wk, rope_cos, rope_sin, seq, q_heads, k_heads, head_dim, eps,
              split_half);
}

void iris_dev_head_norm_rope_qk_streams(uint16_t *xq, uint16_t *xk, int ld,
                                        const float *wq_a, const float *wk_a, const float *wq_b, const float *wk_b,
                                        int rows_a, const float *rope_cos, const float *rope_sin,
                                        int seq, int q_heads, int k_heads, int head_dim, float eps, int split_half) {
    if (rows_a < 0 || rows_a > seq || !wq_a || !wq_b || (k_heads > 0 && (!wk_a || !wk_b || !xk))) {
        if (need_ready("head_norm_rope_qk_streams"))
            fail(-1, "head_norm_rope_qk_streams", "need 0 <= rows_a <= seq and both weight pairs");
        return;
    }
    norm_rope_streams(xq, xk, ld, wq_a, wk_a, wq_b, wk_b, rows_a, rope_cos, rope_sin, seq, q_heads, k_heads, head_dim, eps,
                      split_half);
}

/* head_dim 256 / 512 on the matrix cores (rows 16-byte aligned; the VAE's call at head_dim 512, key mask and causal
 * limit included): the kernel in which a wave owns 32 whole queries. Its key ranges, if it cuts any, leave their
 * partial results in private scratch, and so does its packed key mask. `kind`: 0 direct, 1 through the padded copy,
 * 2 that with Q normalised. Returns 0 or a HIP error; -1 when the scratch could not be had (already reported). */
static int attention_wide(const char *what, int kind, uint16_t *out, int ldo,
                          const uint16_t *q, const uint16_t *k, const uint16_t *v, int ldi, int seq_q, int seq_k,
                          int heads, int kv_heads, int head_dim, float scale, int causal, const int *key_mask) {
    static const char *const names[2][3] = {{"fa_hd512", "fa_hd512_packed", "fa_hd512_packed_qnorm"},
                                            {"fa_hd256", "fa_hd256_packed", "fa_hd256_packed_qnorm"}};
    int splits = 1;
    const size_t need = head_dim == 512 ? iris_hip_fa_hd512_plan(seq_q, seq_k, heads, causal != 0, key_mask != NULL, &splits)
                                        : iris_hip_fa_hd256_plan(seq_q, seq_k, heads, causal != 0, key_mask != NULL, &splits);
    if (need && !scratch_fit(&g_split, &g_split_bytes, need, what)) return -1;
    g_last_kernel = names[head_dim == 512 ? 0 : 1][kind];
    return head_dim == 512
               ? iris_hip_fa_hd512(g_stream, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, causal != 0, key_mask, splits, g_split)
               : iris_hip_fa_hd256(g_stream, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, scale, causal != 0, key_mask, splits, g_split);
}

/* wq == NULL: plain attention. Otherwise Q is normalised and rotated on the way in. */
static void attention(const char *what, uint16_t *out, int ldo,
                      const uint16_t *q, const uint16_t *k, const uint16_t *v,
                      int ldi, int seq_q, int seq_k, int heads, int kv_heads,
                      int head_dim, float scale, int causal, const int *key_mask,
                      const float *wq, const float *rope_cos, const float *rope_sin,
                      float eps, int split_half) {
    if (!need_ready(what)) return;
    if (seq_q <= 0 || heads <= 0) return;
    if (kv_heads <= 0 || heads % kv_heads != 0 || head_dim <= 0 || seq_k < 0) {
        fail(-1, what, "need heads % kv_heads == 0, head_dim > 0, seq_k >= 0");
        return;
    }
    if (wq && (!rope_cos || !rope_sin || (head_dim & 1))) {
        fail(-1, what, "need the rotary tables and an even head_dim");
        return;
    }
    int mfma_ok = seq_k > 0 && scale > 0.0f && ldi % 8 == 0 && ldo % 4 == 0 &&
                  aligned(q, 16) && aligned(k, 16) && aligned(v, 16) && aligned(out, 8);
    int err;
    if (mfma_ok && head_dim == 128 && (!key_mask || seq_k <= IRIS_FA_MAX_MASKED_KEYS) &&
        (!wq || (aligned(wq, 16) && aligned(rope_cos, 16) && aligned(rope_sin, 16)))) {
        if (wq) {
            g_last_kernel = "fa_hd128_qnorm";
            err = iris_hip_fa_hd128_qnorm(g_stream, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads,
                                          scale, causal != 0, key_mask, wq, rope_cos, rope_sin, eps, split_half != 0);
        } else {
            g_last_kernel = "fa_hd128";
            err = iris_hip_fa_hd128(g_stream, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads,
                                    scale, causal != 0, key_mask);
        }
        if (err) check((hipError_t)err, "attention launch");
        return;
    }
    /* Every other shape. Q normalised on the way in: a normalised copy of Q (rows of heads * head_dim) in
     * private scratch takes the place of q from here on. */
    const uint16_t *qq = q;
    int ldq = ldi;
    if (wq) {
        ldq = heads * head_dim;
        if (!scratch_fit((void **)&g_q_scratch, &g_q_scratch_bytes, (size_t)seq_q * ldq * sizeof(uint16_t), what)) return;
        if (!check(hipMemcpy2DAsync(g_q_scratch, (size_t)ldq * 2, q, (size_t)ldi * 2, (size_t)ldq * 2, (size_t)seq_q,
                                    hipMemcpyDeviceToDevice, g_stream), "copy of q"))
            return;
        norm_rope(g_q_scratch, NULL, ldq, wq, NULL, rope_cos, rope_sin, seq_q, heads, 0, head_dim, eps, split_half);
        qq = g_q_scratch;
    }
    const int mfma_args = seq_k > 0 && scale > 0.0f && head_dim <= 512 && (!key_mask || seq_k <= IRIS_FA_MAX_MASKED_KEYS);
    if (mfma_ok && !wq && (head_dim == 256 || head_dim == 512)) {
        err = attention_wide(what, 0, out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, head_dim, scale, causal, key_mask);
        if (err < 0) return;
    } else if (mfma_args) {
        /* Any head_dim <= 512, any stride and alignment: q | k | v copied into one fused row buffer with
         * every head padded with zeros to the next of 128 / 256 / 512 dims, the matrix-core kernel of that
         * width on the copy, and the first head_dim of every head's output columns copied back. */
        const int hdp = head_dim <= 128 ? 128 : head_dim <= 256 ? 256 : 512;
        const int rows = seq_q > seq_k ? seq_q : seq_k;
        const int ldp = (heads + 2 * kv_heads) * hdp, ldop = heads * hdp;
        const size_t in_bytes = ((size_t)rows * ldp * 2 + 255) & ~(size_t)255;
        const int direct_out = head_dim == hdp && ldo % 4 == 0 && aligned(out, 8);
        if (!scratch_fit((void **)&g_pack, &g_pack_bytes, in_bytes + (direct_out ? 0 : (size_t)seq_q * ldop * 2), what)) return;
        uint16_t *packed = g_pack, *outp = direct_out ? out : g_pack + in_bytes / 2;
        err = iris_hip_pack_heads(g_stream, packed, qq, ldq, seq_q, k, v, ldi, seq_k, heads, kv_heads, head_dim, hdp);
        if (!err) {
            const uint16_t *pk = packed + (size_t)heads * hdp, *pv = pk + (size_t)kv_heads * hdp;
            const int ldout = direct_out ? ldo : ldop;
            if (hdp == 128) {
                g_last_kernel = wq ? "fa_hd128_packed_qnorm" : "fa_hd128_packed";
                err = iris_hip_fa_hd128(g_stream, outp, ldout, packed, pk, pv, ldp, seq_q, seq_k, heads, kv_heads,
                                        scale, causal != 0, key_mask);
            } else {
                err = attention_wide(what, wq ? 2 : 1, outp, ldout, packed, pk, pv, ldp, seq_q, seq_k, heads, kv_heads, hdp,
                                     scale, causal, key_mask);
                if (err < 0) return;
            }
        }
        if (!err && !direct_out)
            err = iris_hip_unpack_heads(g_stream, out, ldo, outp, ldop, seq_q, heads, head_dim, hdp);
    } else {
        g_last_kernel = wq ? "attention_generic_qnorm" : "attention_generic";
        err = iris_hip_attention_generic(g_stream, out, ldo, qq, ldq, k, v, ldi, seq_q, seq_k, heads,
                                         kv_heads, head_dim, scale, causal != 0, key_mask);
    }
    if (err) check((hipError_t)err, "attention launch");
}

void iris_dev_attention(uint16_t *out, int ldo,
                        const uint16_t *q, const uint16_t *k, const uint16_t *v,
                        int ldi, int seq_q, int seq_k, int heads, int kv_heads,
                        int head_dim, float scale, int causal, const int *key_mask) {
    attention("attention", out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, head_dim, scale, causal, key_mask,
              NULL, NULL, NULL, 0.0f, 0);
}

void iris_dev_attention_qnorm(uint16_t *out, int ldo,
                              const uint16_t *q, const uint16_t *k, const uint16_t *v,
                              int ldi, int seq_q, int seq_k, int heads, int kv_heads,
                              int head_dim, float scale, int causal, const int *key_mask,
                              const float *wq, const float *rope_cos, const float *rope_sin,
                              float eps, int split_half) {
    if (!wq) { fail(-1, "attention_qnorm", "the norm weights are missing"); return; }
    attention("attention_qnorm", out, ldo, q, k, v, ldi, seq_q, seq_k, heads, kv_heads, head_dim, scale, causal,
              key_mask, wq, rope_cos, rope_sin, eps, split_half);
}

/* ---- the other operators: thin checked wrappers over the launchers ---- */

#ifndef IRIS_DEV_PATH_ONLY
#define LAUNCH(what, call)                                        \
    do {                                                          \
        if (!need_ready(what)) return;                            \
        int err_ = (call);                                        \
        if (err_) check((hipError_t)err_, what " launch");        \
    } while (0)

void iris_dev_f32_to_bf16(uint16_t *dst, const float *src, size_t n) {
    LAUNCH("f32_to_bf16", iris_hip_f32_to_bf16(g_stream, dst, src, n));
}

/* Plain GEMMs run on this library's own MFMA kernels. iris_dev_linear_backend(2) sends them to the vendor
 * library instead, where it can be opened and takes the problem (aligned operands, in % 8 == 0): the yardstick
 * the benchmark compares the own kernels with. 0 and 1 select the own kernels. */
static int g_linear_backend = 0;

void iris_dev_linear_backend(int which) { g_linear_backend = which == 2 ? 2 : 0; }

static int linear_by_library(void *y, int out_bf16, const uint16_t *x, const uint16_t *W, int rows, int in, int out) {
    if (g_linear_backend != 2 || in % 8 != 0 || !aligned(y, 16) || !aligned(x, 16) || !aligned(W, 16)) return 0;
    if (iris_lt_linear(g_stream, y, out_bf16, x, W, rows, in, out) != 0) return 0;
    g_last_kernel = "linear_hipblaslt";
    return 1;
}

void iris_dev_linear_f32(float *y, const uint16_t *x, const uint16_t *W, int rows, int in, int out) {
    if (rows <= 0 || out <= 0) return;
    if (in <= 0) { fail(-1, "linear", "in must be positive"); return; }
    if (!need_ready("linear")) return;
    if (linear_by_library(y, 0, x, W, rows, in, out)) return;
    g_last_kernel = "linear_mfma";
    LAUNCH("linear", iris_hip_linear_f32(g_stream, y, x, W, rows, in, out));
}

void iris_dev_linear_bf16(uint16_t *y, const uint16_t *x, const uint16_t *W, int rows, int in, int out) {
    if (rows <= 0 || out <= 0) return;
    if (in <= 0) { fail(-1, "linear", "in must be positive"); return; }
    if (!need_ready("linear")) return;
    if (linear_by_library(y, 1, x, W, rows, in, out)) return;
    g_last_kernel = "linear_mfma";
    LAUNCH("linear", iris_hip_linear_bf16(g_stream, y, x, W, rows, in, out));
}

void iris_dev_linear_bf16_qknorm(uint16_t *y, const uint16_t *x, const uint16_t *W, int rows, int in, int out,
                                 int q_heads, int k_heads, int head_dim, const float *wq, const float *wk,
                                 const float *rope_cos, const float *rope_sin, float eps, int split_half) {
    if (rows <= 0 || out <= 0) return;
    if (in <= 0) { fail(-1, "linear_qknorm", "in must be positive"); return; }
    if (q_heads < 0 || k_heads < 0 || head_dim <= 0 || (long long)(q_heads + k_heads) * head_dim > out) {
        fail(-1, "linear_qknorm", "need (q_heads + k_heads) * head_dim <= out");
        return;
    }
    if (!need_ready("linear_qknorm")) return;
    /* With the vendor GEMM selected and present, the entry is its linear layer followed by the norm kernel. */
    int one_launch = head_dim == 128 && q_heads + k_heads > 0 &&
                     (g_linear_backend != 2 || !iris_lt_available() || in % 8 != 0);
    if (one_launch) {
        int err = iris_hip_linear_bf16_qknorm(g_stream, y, x, W, rows, in, out, q_heads * 128, k_heads * 128, wq, wk,
                                              rope_cos, rope_sin, eps, split_half != 0);
        if (err == 0) { g_last_kernel = "linear_mfma_qknorm"; return; }
        if (err != -2) { check((hipError_t)err, "linear_qknorm launch"); return; }
    }
    /* the two steps one after the other */
    iris_dev_linear_bf16(y, x, W, rows, in, out);
    if (q_heads > 0)
        norm_rope(y, k_heads ? y + (size_t)q_heads * head_dim : NULL, out, wq, wk, rope_cos, rope_sin, rows, q_heads, k_heads,
                  head_dim, eps, split_half);
    else if (k_heads > 0)
        norm_rope(y, NULL, out, wk, NULL, rope_cos, rope_sin, rows, k_heads, 0, head_dim, eps, split_half);
}

void iris_dev_layer_norm_mod(uint16_t *out, const float *x, const float *shift, const float *scale,
                             int rows, int dim, float eps) {
    LAUNCH("layer_norm_mod", iris_hip_layer_norm_mod(g_stream, out, x, shift, scale, rows, dim, eps));
}

void iris_dev_rms_norm(uint16_t *out, const float *x, const float *w, int rows, int dim, float eps) {
    LAUNCH("rms_norm", iris_hip_rms_norm_mod(g_stream, out, x, w, NULL, rows, dim, eps));
}

void iris_dev_rms_norm_mod(uint16_t *out, const float *x, const float *w, const float *scale,
                           int rows, int dim, float eps) {
    LAUNCH("rms_norm_mod", iris_hip_rms_norm_mod(g_stream, out, x, w, scale, rows, dim, eps));
}

void iris_dev_rms_norm_residual(float *x, const float *a, const float *w, const float *gate,
                                int rows, int dim, float eps) {
    LAUNCH("rms_norm_residual", iris_hip_rms_norm_residual(g_stream, x, a, w, gate, rows, dim, eps));
}

void iris_dev_swiglu(uint16_t *out, int ldo, const uint16_t *gate, const uint16_t *up, int ldi,
                     int rows, int cols) {
    if (rows <= 0 || cols <= 0) return;
    LAUNCH("swiglu", iris_hip_swiglu(g_stream, out, ldo, gate, up, ldi, rows, cols));
}

void iris_dev_residual(float *x, const float *a, const float *gate, int rows, int dim) {
    if (rows <= 0 || dim <= 0) return;
    LAUNCH("residual", iris_hip_residual(g_stream, x, a, gate, rows, dim));
}

void iris_dev_silu(float *x, size_t n) { LAUNCH("silu", iris_hip_silu(g_stream, x, n)); }
void iris_dev_add(float *x, const float *a, size_t n) { LAUNCH("add", iris_hip_add(g_stream, x, a, n)); }

void iris_dev_add_bias(float *y, const float *bias, int rows, int cols) {
    if (rows <= 0 || cols <= 0) return;
    LAUNCH("add_bias", iris_hip_add_bias(g_stream, y, bias, rows, cols));
}

void iris_dev_fill_rows(float *out, const float *row, int rows, int dim) {
    if (rows <= 0 || dim <= 0) return;
    LAUNCH("fill_rows", iris_hip_fill_rows(g_stream, out, row, rows, dim));
}

void iris_dev_conv2d(float *out, const float *in, const uint16_t *w, const float *bias,
                     int h, int width, int cin, int cout, int k, int stride,
                     int pad_before, int pad_after) {
    if (!need_ready("conv2d")) return;
    if (h <= 0 || width <= 0 || cin <= 0 || cout <= 0 || k <= 0 || stride <= 0 || pad_before < 0 || pad_after < 0 ||
        (size_t)k * k * cin * sizeof(uint16_t) > CONV_SCRATCH_BYTES - IRIS_CONV_ZERO_BYTES) {
        fail(-1, "conv2d", "bad shape");
        return;
    }
    if (!g_conv_scratch) {
        if (hipMalloc((void **)&g_conv_scratch, CONV_SCRATCH_BYTES) != hipSuccess) {
            (void)hipGetLastError();
            g_conv_scratch = NULL;
            fail(-1, "conv2d", "scratch allocation failed");
            return;
        }
        int e = iris_hip_conv2d_prepare_scratch(g_stream, g_conv_scratch);
        if (e) { check((hipError_t)e, "conv2d scratch"); return; }
    }
    int err = iris_hip_conv2d(g_stream, g_conv_scratch, CONV_SCRATCH_BYTES, out, in, w, bias, h, width, cin, cout,
                              k, stride, pad_before, pad_after);
    if (err) check((hipError_t)err, "conv2d launch");
}

void iris_dev_group_norm(float *out, const float *in, const float *gamma, const float *beta,
                         int hw, int c, int groups, float eps, int silu) {
    if (!need_ready("group_norm")) return;
    if (hw <= 0 || c <= 0) return;
    if (groups <= 0 || c % groups != 0) { fail(-1, "group_norm", "need c % groups == 0"); return; }
    size_t need = iris_hip_group_norm_scratch_floats(groups);
    if (need > g_gn_scratch_floats) {
        if (g_gn_scratch) {
            check(hipStreamSynchronize(g_stream), "sync");
            check(hipFree(g_gn_scratch), "free");
        }
        g_gn_scratch = NULL;
        g_gn_scratch_floats = 0;
        if (hipMalloc((void **)&g_gn_scratch, need * sizeof(float)) != hipSuccess) {
            (void)hipGetLastError();
            g_gn_scratch = NULL;
            fail(-1, "group_norm", "scratch allocation failed");
            return;
        }
        g_gn_scratch_floats = need;
    }
    int err = iris_hip_group_norm(g_stream, g_gn_scratch, out, in, gamma, beta, hw, c, groups, eps, silu != 0);
    if (err) check((hipError_t)err, "group_norm launch");
}

/* The same operator for callers that cannot allocate: scratch is an array inside the library. */
void iris_dev_group_norm_noalloc(float *out, const float *in, const float *gamma, const float *beta,
                                 int hw, int c, int groups, float eps, int silu) {
    if (!need_ready("group_norm_noalloc")) return;
    if (hw <= 0 || c <= 0) return;
    if (groups <= 0 || c % groups != 0) { fail(-1, "group_norm_noalloc", "need c % groups == 0"); return; }
    if (groups > iris_hip_group_norm_static_max_groups()) {
        fail(-1, "group_norm_noalloc", "more than 64 groups: beyond the built-in scratch, use iris_dev_group_norm");
        return;
    }
    int err = iris_hip_group_norm_static(g_stream, out, in, gamma, beta, hw, c, groups, eps, silu != 0);
    if (err) check((hipError_t)err, "group_norm_noalloc launch");
}

void iris_dev_upsample2x(float *out, const float *in, int h, int width, int c) {
    if (h <= 0 || width <= 0 || c <= 0) return;
    LAUNCH("upsample2x", iris_hip_upsample2x(g_stream, out, in, h, width, c));
}

/* ---- rotary tables generated on the device (include/iris_rope.h) ---- */

/* The host evaluates every distinct (axis, position) of the sequence once, with the arithmetic
 * of the host builders (iris_rope_tables.c), and stages [columns: half x 16 B | index: seq x
 * naxes x 4 B | dictionary] in one upload; the kernel expands it into the two tables. pos is
 * int32 (use_double 0) or float (use_double 1). */
static void rope_tables(const char *what, float *d_cos, float *d_sin, const void *pos, int seq, int naxes,
                        const int *axis_dims, const int *axis_lens, float theta, int use_double) {
    if (!need_ready(what)) return;
    if (!iris_rope_axes_ok_(seq, naxes, axis_dims) || (seq && (!d_cos || !d_sin || !pos))) {
        fail(-1, what, "bad arguments");
        return;
    }
    size_t half = 0;
    for (int a = 0; a < naxes; a++) half += (size_t)(axis_dims[a] / 2);
    if (!seq || !half) return;
    float *values = NULL;
    uint32_t *index = NULL;
    size_t n_values = 0;
    if (iris_rope_dictionary_(pos, use_double, seq, naxes, axis_dims, axis_lens, theta, &values, &n_values, &index) != 0) {
        fail(-1, what, "out of host memory");
        return;
    }
    const size_t col_bytes = half * 16, idx_bytes = (size_t)seq * naxes * 4, val_bytes = n_values * 4;
    const size_t total = col_bytes + idx_bytes + val_bytes;
    if (total > g_rope_stage_bytes) {
        if (g_rope_stage) {
            check(hipStreamSynchronize(g_stream), "sync");
            check(hipFree(g_rope_stage), "free");
        }
        g_rope_stage = NULL;
        g_rope_stage_bytes = 0;
        if (hipMalloc(&g_rope_stage, total) != hipSuccess) {
            (void)hipGetLastError();
            g_rope_stage = NULL;
            free(values); free(index);
            fail(-1, what, "out of device memory for the staging buffer");
            return;
        }
        g_rope_stage_bytes = total;
    }
    unsigned char *blob = malloc(total);
    if (!blob) { free(values); free(index); fail(-1, what, "out of host memory"); return; }
    int *col = (int *)blob;
    for (int a = 0; a < naxes; a++)
        for (int j = 0; j < axis_dims[a] / 2; j++, col += 4) {
            col[0] = a; col[1] = j; col[2] = axis_dims[a] / 2; col[3] = 0;
        }
    memcpy(blob + col_bytes, index, idx_bytes);
    memcpy(blob + col_bytes + idx_bytes, values, val_bytes);
    free(values); free(index);
    /* stream order keeps an earlier table kernel's reads ahead of this overwrite of the staging buffer */
    int ok = check(hipMemcpyAsync(g_rope_stage, blob, total, hipMemcpyHostToDevice, g_stream), "upload") &&
             check(hipStreamSynchronize(g_stream), "sync");
    free(blob);
    if (!ok) return;
    const unsigned char *d = g_rope_stage;
    int err = iris_hip_rope_gather(g_stream, d_cos, d_sin, (const float *)(d + col_bytes + idx_bytes),
                                   (const uint32_t *)(d + col_bytes), d, seq, (int)half, naxes);
    if (err) check((hipError_t)err, "rope tables launch");
}

void iris_dev_rope_expand_i32(float *d_cos, float *d_sin, const int *pos, int seq, int naxes,
                              const int *axis_dims, const int *axis_lens, float theta) {
    rope_tables("rope_expand_i32", d_cos, d_sin, pos, seq, naxes, axis_dims, axis_lens, theta, 0);
}

void iris_dev_rope_expand_f64(float *d_cos, float *d_sin, const float *pos, int seq, int naxes,
                              const int *axis_dims, float theta) {
    rope_tables("rope_expand_f64", d_cos, d_sin, pos, seq, naxes, axis_dims, NULL, theta, 1);
}

void iris_dev_rope_flux2_tables(float *d_cos, float *d_sin, int txt_seq, int img_h, int img_w,
                                const int *ref_h, const int *ref_w, const int *ref_t, int num_refs,
                                int axis_dim, float theta) {
    const int rows = iris_rope_joint_rows(txt_seq, img_h, img_w, ref_h, ref_w, num_refs);
    int *pos = rows < 0 ? NULL : malloc(sizeof(int) * 4 * (size_t)(rows ? rows : 1));
    if (!pos) { fail(-1, "rope_flux2_tables", "bad sizes or out of host memory"); return; }
    iris_rope_flux2_positions(pos, txt_seq, img_h, img_w, ref_h, ref_w, ref_t, num_refs);
    const int dims[4] = { axis_dim, axis_dim, axis_dim, axis_dim };
    rope_tables("rope_flux2_tables", d_cos, d_sin, pos, rows, 4, dims, NULL, theta, 0);
    free(pos);
}

void iris_dev_rope_flux3_tables(float *d_cos, float *d_sin, int txt_seq, int img_h, int img_w,
                                const int *ref_h, const int *ref_w, int num_refs,
                                const int axes_dim[4], float theta) {
    const int rows = iris_rope_joint_rows(txt_seq, img_h, img_w, ref_h, ref_w, num_refs);
    float *pos = rows < 0 ? NULL : malloc(sizeof(float) * 4 * (size_t)(rows ? rows : 1));
    if (!pos) { fail(-1, "rope_flux3_tables", "bad sizes or out of host memory"); return; }
    iris_rope_flux3_positions(pos, txt_seq, img_h, img_w, ref_h, ref_w, num_refs);
    rope_tables("rope_flux3_tables", d_cos, d_sin, pos, rows, 4, axes_dim, NULL, theta, 1);
    free(pos);
}

void iris_dev_rope_zimage_tables(float *d_cos, float *d_sin, const int *pos3, int seq,
                                 const int axes_dims[3], const int axes_lens[3], float theta) {
    rope_tables("rope_zimage_tables", d_cos, d_sin, pos3, seq, 3, axes_dims, axes_lens, theta, 0);
}

void iris_dev_rope_qwen3_tables(float *d_cos, float *d_sin, const int *attention_mask, int seq,
                                int head_dim, float theta, int pad_at_one) {
    int *pos = seq < 0 ? NULL : iris_rope_qwen3_positions_(attention_mask, seq, pad_at_one);
    if (!pos) { fail(-1, "rope_qwen3_tables", "bad sizes or out of host memory"); return; }
    rope_tables("rope_qwen3_tables", d_cos, d_sin, pos, seq, 1, &head_dim, NULL, theta, 0);
    free(pos);
}
#endif /* !IRIS_DEV_PATH_ONLY */
