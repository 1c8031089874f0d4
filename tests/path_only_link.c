/* Link check of the path-only archive (libiris_dev_path.a): a host program that brings its own device backend
 * -- its own iris_dev_init, memory entries and stream, standing in for the reference's backend object
 * (iris_cuda.cu:117-230) -- and takes iris_dev_head_norm_rope and iris_dev_attention from the archive. Linking
 * proves that the archive defines no symbol the host defines; run on a GPU it also calls the path once. */
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "iris_dev_path.h"

/* ---- the host's own backend: the names of the reference's ---- */
static hipStream_t host_stream;
int iris_dev_init(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n == 0) return 0;
    if (hipSetDevice(0) != hipSuccess || hipStreamCreate(&host_stream) != hipSuccess) return 0;
    iris_dev_path_attach((void *)host_stream);
    return 1;
}
int iris_dev_available(void) { return host_stream != NULL; }
const char *iris_dev_name(void) { return "host backend"; }
void iris_dev_cleanup(void) { iris_dev_path_detach(); (void)hipStreamDestroy(host_stream); host_stream = NULL; }
void *iris_dev_alloc(size_t bytes) { void *p = NULL; return hipMalloc(&p, bytes ? bytes : 1) == hipSuccess ? p : NULL; }
void iris_dev_free(void *p) { (void)hipStreamSynchronize(host_stream); (void)hipFree(p); }
void iris_dev_upload(void *dst, const void *src, size_t bytes) { (void)hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, host_stream); (void)hipStreamSynchronize(host_stream); }
void iris_dev_download(void *dst, const void *src, size_t bytes) { (void)hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, host_stream); (void)hipStreamSynchronize(host_stream); }
void iris_dev_sync(void) { (void)hipStreamSynchronize(host_stream); }
void iris_dev_linear_bf16(uint16_t *y, const uint16_t *x, const uint16_t *W, int rows, int in, int out) {
    (void)y; (void)x; (void)W; (void)rows; (void)in; (void)out;      /* the host's own operator */
}

int main(void) {
    if (!iris_dev_init()) { printf("no GPU: linked only\n"); return 0; }
    /* constant V: every output row must equal that constant, whatever the scores */
    const int seq = 300, heads = 2, hd = 128, ld = 3 * heads * hd;
    uint16_t *host = malloc((size_t)seq * ld * 2), *res = malloc((size_t)seq * heads * hd * 2);
    for (int s = 0; s < seq; s++)
        for (int c = 0; c < ld; c++) host[(size_t)s * ld + c] = c < 2 * heads * hd ? (uint16_t)(0x3c00 + ((s * 31 + c * 7) & 0xff)) : 0x4040; /* v = 3.0 */
    float w[128], tab[300 * 64];
    for (int i = 0; i < 128; i++) w[i] = 1.0f;
    uint16_t *rows = iris_dev_alloc((size_t)seq * ld * 2), *out = iris_dev_alloc((size_t)seq * heads * hd * 2);
    float *dw = iris_dev_alloc(sizeof w), *dcos = iris_dev_alloc(sizeof tab), *dsin = iris_dev_alloc(sizeof tab);
    iris_dev_upload(rows, host, (size_t)seq * ld * 2);
    iris_dev_upload(dw, w, sizeof w);
    for (int i = 0; i < 300 * 64; i++) tab[i] = 1.0f;
    iris_dev_upload(dcos, tab, sizeof tab);
    memset(tab, 0, sizeof tab);
    iris_dev_upload(dsin, tab, sizeof tab);
    iris_dev_head_norm_rope(rows, ld, dw, dcos, dsin, seq, heads, hd, 1e-6f, 0);
    iris_dev_head_norm_rope(rows + heads * hd, ld, dw, dcos, dsin, seq, heads, hd, 1e-6f, 0);
    iris_dev_attention(out, heads * hd, rows, rows + heads * hd, rows + 2 * heads * hd, ld, seq, seq, heads, heads, hd, 0.0884f, 0, NULL);
    iris_dev_download(res, out, (size_t)seq * heads * hd * 2);
    int bad = iris_dev_last_error() != 0;
    for (int i = 0; i < seq * heads * hd; i++) bad |= res[i] != 0x4040;
    printf("%s (%s)\n", bad ? "FAILED" : "ok", iris_dev_last_kernel());
    iris_dev_cleanup();
    return bad;
}
