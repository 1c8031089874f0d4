/*
 * CPU oracle for the remaining device operators (TEST INFRASTRUCTURE, not product):
 * linear layers, normalisations, gated activations, residuals, and the VAE's
 * convolution / group norm / upsampling on channels-last images.
 *
 * Each function states the operator exactly as the reference device header
 * defines it (iris_dev.h:45-127) and follows the reference kernel named
 * beside it (iris_cuda.cu) for the points the header leaves open: where
 * values are rounded to bf16, and what is accumulated in which precision.
 * Sums are accumulated in double so that the checker itself adds no
 * order-of-summation noise; device results are compared within a tolerance.
 *
 * Pin status (tests/test_oracle_ops.py):
 *   orc_dev_linear            compiled reference iris_linear_nobias_bf16, numpy matmul
 *   orc_dev_layer_norm_mod    numpy closed form; shift/scale = 0 reduces to torch layer_norm
 *   orc_dev_rms_norm_mod      compiled reference iris_rms_norm (scale NULL), numpy
 *   orc_dev_rms_norm_residual numpy closed form built on the pinned rms norm
 *   orc_dev_swiglu / silu     compiled reference iris_silu, iris_silu_mul; torch silu
 *   orc_dev_residual/add/add_bias/fill_rows   numpy one-liners
 *   orc_dev_conv2d            compiled reference iris_conv2d through a layout transpose
 *                             (NCHW <-> channels-last) on bf16-representable data; torch conv2d
 *   orc_dev_group_norm        compiled reference iris_group_norm through the same transpose;
 *                             torch group_norm
 *   orc_dev_upsample2x        compiled reference iris_upsample_nearest through the transpose
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>

#include "iris_oracle.h"

/* y[rows, out] = x[rows, in] @ W[out, in]^T, bf16 inputs (iris_dev.h:48-53; iris_cuda.cu:456-505) */
void orc_dev_linear(float *y, const uint16_t *x, const uint16_t *W, int rows, int in, int out) {
#pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; r++)
        for (int o = 0; o < out; o++) {
            const uint16_t *xr = x + (size_t)r * in, *wr = W + (size_t)o * in;
            double acc = 0.0;
            for (int i = 0; i < in; i++) acc += (double)orc_bf2f(xr[i]) * (double)orc_bf2f(wr[i]);
            y[(size_t)r * out + o] = (float)acc;
        }
}

/* out = LayerNorm(x) * (1 + scale) + shift, bf16 out (iris_dev.h:55-59; iris_cuda.cu:349-370) */
void orc_dev_layer_norm_mod(uint16_t *out, const float *x, const float *shift, const float *scale,
                            int rows, int dim, float eps) {
    for (int r = 0; r < rows; r++) {
        const float *xr = x + (size_t)r * dim;
        double s = 0.0, v = 0.0;
        for (int i = 0; i < dim; i++) s += xr[i];
        const double mean = s / dim;
        for (int i = 0; i < dim; i++) v += (xr[i] - mean) * (xr[i] - mean);
        const double inv = 1.0 / sqrt(v / dim + (double)eps);
        for (int i = 0; i < dim; i++) {
            double n = (xr[i] - mean) * inv;
            if (scale) n *= 1.0 + (double)scale[i];
            if (shift) n += (double)shift[i];
            out[(size_t)r * dim + i] = orc_f2bf((float)n);
        }
    }
}

/* out = RMSNorm(x) * w * (1 + scale), scale optional, bf16 out
 * (iris_dev.h:61-68; iris_cuda.cu:372-386) */
void orc_dev_rms_norm_mod(uint16_t *out, const float *x, const float *w, const float *scale,
                          int rows, int dim, float eps) {
    for (int r = 0; r < rows; r++) {
        const float *xr = x + (size_t)r * dim;
        double s = 0.0;
        for (int i = 0; i < dim; i++) s += (double)xr[i] * xr[i];
        const double inv = 1.0 / sqrt(s / dim + (double)eps);
        for (int i = 0; i < dim; i++) {
            double v = xr[i] * inv * (double)w[i];
            if (scale) v *= 1.0 + (double)scale[i];
            out[(size_t)r * dim + i] = orc_f2bf((float)v);
        }
    }
}

/* x += tanh(gate) * RMSNorm(a) * w in f32, gate optional (iris_dev.h:70-73; iris_cuda.cu:388-400) */
void orc_dev_rms_norm_residual(float *x, const float *a, const float *w, const float *gate,
                               int rows, int dim, float eps) {
    for (int r = 0; r < rows; r++) {
        const float *ar = a + (size_t)r * dim;
        double s = 0.0;
        for (int i = 0; i < dim; i++) s += (double)ar[i] * ar[i];
        const double inv = 1.0 / sqrt(s / dim + (double)eps);
        for (int i = 0; i < dim; i++) {
            const double v = ar[i] * inv * (double)w[i];
            x[(size_t)r * dim + i] = (float)(x[(size_t)r * dim + i] + (gate ? tanh((double)gate[i]) : 1.0) * v);
        }
    }
}

static double silu_d(double g) { return g / (1.0 + exp(-g)); }

/* out[r, c] = silu(gate[r, c]) * up[r, c], bf16 in/out with row strides (iris_dev.h:94-97; iris_cuda.cu:300-307) */
void orc_dev_swiglu(uint16_t *out, int ldo, const uint16_t *gate, const uint16_t *up, int ldi,
                    int rows, int cols) {
    for (int r = 0; r < rows; r++)
        for (int c = 0; c < cols; c++) {
            const double g = orc_bf2f(gate[(size_t)r * ldi + c]);
            out[(size_t)r * ldo + c] = orc_f2bf((float)(silu_d(g) * (double)orc_bf2f(up[(size_t)r * ldi + c])));
        }
}

/* x[r, c] += gate[c] * a[r, c] (gate optional) (iris_dev.h:99-101; iris_cuda.cu:309-314) */
void orc_dev_residual(float *x, const float *a, const float *gate, int rows, int dim) {
    for (size_t i = 0; i < (size_t)rows * dim; i++) x[i] += (gate ? gate[i % dim] : 1.0f) * a[i];
}

/* elementwise helpers (iris_dev.h:103-107; iris_cuda.cu:285-298, 943-946) */
void orc_dev_silu(float *x, size_t n) {
    for (size_t i = 0; i < n; i++) x[i] = (float)silu_d(x[i]);
}
void orc_dev_add(float *x, const float *a, size_t n) {
    for (size_t i = 0; i < n; i++) x[i] += a[i];
}
void orc_dev_add_bias(float *y, const float *bias, int rows, int cols) {
    for (size_t i = 0; i < (size_t)rows * cols; i++) y[i] += bias[i % cols];
}
void orc_dev_fill_rows(float *out, const float *row, int rows, int dim) {
    for (size_t i = 0; i < (size_t)rows * dim; i++) out[i] = row[i % dim];
}

/* k x k convolution on a channels-last f32 image, bf16 weights [cout, k*k*cin] in (ky, kx, c)
 * order, zero padding (iris_dev.h:111-121). The reference gathers the input patches as bf16
 * before its GEMM (iris_cuda.cu:959-985), so the input is rounded to bf16 here as well. */
void orc_dev_conv2d(float *out, const float *in, const uint16_t *w, const float *bias, int h, int width,
                    int cin, int cout, int k, int stride, int pad_before, int pad_after) {
    const int oh = (h + pad_before + pad_after - k) / stride + 1;
    const int ow = (width + pad_before + pad_after - k) / stride + 1;
#pragma omp parallel for schedule(static)
    for (int p = 0; p < oh * ow; p++) {
        const int oy = p / ow, ox = p % ow;
        for (int o = 0; o < cout; o++) {
            double acc = 0.0;
            for (int ky = 0; ky < k; ky++)
                for (int kx = 0; kx < k; kx++) {
                    const int y = oy * stride + ky - pad_before, x = ox * stride + kx - pad_before;
                    if (y < 0 || y >= h || x < 0 || x >= width) continue;
                    const float *src = in + ((size_t)y * width + x) * cin;
                    const uint16_t *wr = w + (size_t)o * k * k * cin + (size_t)(ky * k + kx) * cin;
                    for (int c = 0; c < cin; c++)
                        acc += (double)orc_bf2f(orc_f2bf(src[c])) * (double)orc_bf2f(wr[c]);
                }
            out[(size_t)p * cout + o] = (float)(acc + (bias ? (double)bias[o] : 0.0));
        }
    }
}

/* GroupNorm over [hw, c] with affine gamma/beta, optional SiLU (iris_dev.h:123-126;
 * iris_cuda.cu:1018-1055: mean first, then the variance about it, population variance) */
void orc_dev_group_norm(float *out, const float *in, const float *gamma, const float *beta, int hw, int c,
                        int groups, float eps, int silu) {
    const int cg = c / groups;
    for (int g = 0; g < groups; g++) {
        double s = 0.0, v = 0.0;
        for (int p = 0; p < hw; p++)
            for (int j = 0; j < cg; j++) s += in[(size_t)p * c + g * cg + j];
        const double mean = s / ((double)hw * cg);
        for (int p = 0; p < hw; p++)
            for (int j = 0; j < cg; j++) {
                const double d = in[(size_t)p * c + g * cg + j] - mean;
                v += d * d;
            }
        const double rstd = 1.0 / sqrt(v / ((double)hw * cg) + (double)eps);
        for (int p = 0; p < hw; p++)
            for (int j = 0; j < cg; j++) {
                const int ch = g * cg + j;
                const double y = (in[(size_t)p * c + ch] - mean) * rstd * (double)gamma[ch] + (double)beta[ch];
                out[(size_t)p * c + ch] = (float)(silu ? silu_d(y) : y);
            }
    }
}

/* nearest-neighbour 2x upsampling of [h*w, c] into [2h*2w, c] (iris_dev.h:128-129; iris_cuda.cu:1080-1087) */
void orc_dev_upsample2x(float *out, const float *in, int h, int width, int c) {
    for (int y = 0; y < 2 * h; y++)
        for (int x = 0; x < 2 * width; x++)
            for (int ch = 0; ch < c; ch++)
                out[((size_t)y * 2 * width + x) * c + ch] = in[((size_t)(y / 2) * width + x / 2) * c + ch];
}
