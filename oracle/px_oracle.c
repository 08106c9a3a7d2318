/*
 * px_oracle.c -- CPU restatement of PixieNN's non-convolution CPU layer math.
 *
 * TEST INFRASTRUCTURE ONLY: the checker for the HIP kernels and the CPU
 * baseline that bench.py times.  The product never calls into this file.
 *
 * The code below is a fresh statement of the reference's arithmetic, written
 * to reproduce its floating-point behaviour operation by operation:
 *   - fp32 everywhere the reference stores to float between passes;
 *   - double where C++ overload resolution makes the reference promote
 *     (unqualified sqrt/pow inside namespace px bind to the C double
 *     versions; literals such as 1. and 2. are double);
 *   - no fused multiply-add (build with -ffp-contract=off).
 *
 * Pinning status of each group (what a test checks it against):
 *   activations      reference known-answer tests + the reference's own
 *                    Activation.h compiled as oracle/_ref
 *   BN primitives    reference known-answer tests (tests/src/blas.cpp),
 *                    fp64 closed forms, finite differences
 *   max-pool         reference known-answer test (tests/src/maxpool.cpp),
 *                    torch max_pool2d on tiny inputs, brute force
 *   upsample         parity unpinned by reference tests; closed form
 *                    (index copy), torch nearest interpolate, brute force
 *   shortcut         parity unpinned by reference tests; closed form a+b
 *   route            parity unpinned by reference tests; closed form (copy,
 *                    x + y per element)
 *   boxes / IoU      reference known-answer tests (tests/src/darkbox.cpp)
 *   YOLO head        reference known-answer tests (tests/src/yolo_cpu.cpp,
 *                    tests/src/yolo_cuda.cpp kernel-level vectors)
 *   Adam             parity unpinned by reference tests (the reference has
 *                    no CPU Adam and no numeric Adam test); pinned by the
 *                    t=1 closed form and an fp64 Adam-with-L2 recurrence
 *   SGD, rescale +   parity unpinned by reference tests; closed forms,
 *   clip, detections invariants and hand-computed cases (see px_oracle.h)
 *   nms              reference known-answer tests (tests/src/box.cpp),
 *                    hand-worked scenarios, an independent restatement
 */
#include "px_oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ */
/* activations -- include/Activation.h                                 */
/* ------------------------------------------------------------------ */

/* Activation.h:126-148, threshold 20 */
static float softplus_apply(float x)
{
    const float t = 20.0f;
    if (x > t) return x;
    if (x < -t) return expf(x);
    return logf(expf(x) + 1.0f);
}

static float softplus_gradient(float x)
{
    const float t = 20.0f;
    if (x > t) return 1.0f;
    if (x < -t) return expf(x);
    return 1.0f / (1.0f + expf(-x));
}

float pxo_act_apply(int type, float x)
{
    switch (type) {
    case PXO_LEAKY:    /* Activation.h:49-52, alpha = 0.1f */
        return x > 0.0f ? x : 0.1f * x;
    case PXO_LINEAR:   /* 67-70 */
        return x;
    case PXO_LOGGY:    /* 84-87 */
        return 2.0f / (1.0f + expf(-x)) - 1.0f;
    case PXO_LOGISTIC: /* 101-104 */
        return 1.0f / (1.0f + expf(-x));
    case PXO_MISH: {   /* 152-158 */
        float sp = softplus_apply(x);
        float th = tanhf(sp);
        return x * th;
    }
    case PXO_RELU:     /* 179-182 */
        return x > 0.0f ? x : 0.0f;
    case PXO_SOFTPLUS:
        return softplus_apply(x);
    case PXO_SWISH:    /* 198-201, beta = 1 */
        return x / (1.0f + expf(-1.0f * x));
    case PXO_TANH:     /* 218-221 */
        return tanhf(x);
    default:
        return x;
    }
}

float pxo_act_gradient(int type, float x)
{
    switch (type) {
    case PXO_LEAKY:
        return x > 0.0f ? 1.0f : 0.1f;
    case PXO_LINEAR:
        return 1.0f;
    case PXO_LOGGY: {  /* 89-93: differentiates through the OUTPUT convention */
        float y = (x + 1.0f) / 2.0f;
        return 2.0f * (1.0f - y) * y;
    }
    case PXO_LOGISTIC: { /* 106-110 */
        float y = 1.0f / (1.0f + expf(-x));
        return y * (1.0f - y);
    }
    case PXO_MISH: {   /* 160-168 */
        float sp = softplus_apply(x);
        float gsp = softplus_gradient(x);
        float tsp = tanhf(sp);
        float gtsp = (1.0f - tsp * tsp) * gsp;
        return x * gtsp + tsp;
    }
    case PXO_RELU:
        return x > 0.0f ? 1.0f : 0.0f;
    case PXO_SOFTPLUS:
        return softplus_gradient(x);
    case PXO_SWISH: {  /* 203-207 */
        const float beta = 1.0f;
        float val = 1.0f / (1.0f + expf(-beta * x));
        return x * val + beta * val * (1.0f - x * val);
    }
    case PXO_TANH: {
        float y = tanhf(x);
        return 1.0f - y * y;
    }
    default:
        return 1.0f;
    }
}

/* Activation.h:292-304 */
void pxo_activate(int type, float* x, size_t n)
{
    for (size_t i = 0; i < n; ++i) x[i] = pxo_act_apply(type, x[i]);
}

/* Activation.h:312-324: delta *= f'(x) */
void pxo_gradient(int type, const float* x, size_t n, float* delta)
{
    for (size_t i = 0; i < n; ++i) delta[i] = delta[i] * pxo_act_gradient(type, x[i]);
}

/* ------------------------------------------------------------------ */
/* per-channel primitives -- src/CpuUtil.cpp                           */
/* ------------------------------------------------------------------ */

/* CpuUtil.cpp:178-187 */
void pxo_add_bias(float* out, const float* bias, int batch, int n, int size)
{
    for (int b = 0; b < batch; ++b)
        for (int c = 0; c < n; ++c) {
            float* plane = out + ((size_t) b * n + c) * size;
            const float add = bias[c];
            for (int k = 0; k < size; ++k) plane[k] += add;
        }
}

/* CpuUtil.cpp:208-215: left-to-right fp32 sum */
float pxo_sum_array(const float* a, int n)
{
    float s = 0.0f;
    for (int i = 0; i < n; ++i) s += a[i];
    return s;
}

/* CpuUtil.cpp:217-220 hands this to cblas_snrm2, whose internal summation is
 * implementation defined; carried in double here and rounded once. */
float pxo_mag_array(const float* a, size_t n)
{
    double ss = 0.0;
    for (size_t i = 0; i < n; ++i) ss += (double) a[i] * (double) a[i];
    return (float) sqrt(ss);
}

/* CpuUtil.cpp:189-196: one fp32 plane sum per (image, filter), added to the update */
void pxo_backward_bias(float* bias_updates, const float* delta, int batch, int n, int size)
{
    for (int b = 0; b < batch; ++b)
        for (int c = 0; c < n; ++c)
            bias_updates[c] += pxo_sum_array(delta + (size_t) size * (c + (size_t) b * n), size);
}

/* cblas_sdot stand-in for CpuUtil.cpp:203; OpenBLAS's order of summation is
 * implementation defined, a left-to-right fp32 sum is used. */
static float dot_f32(const float* a, const float* b, int n)
{
    float s = 0.0f;
    for (int i = 0; i < n; ++i) s += a[i] * b[i];
    return s;
}

/* CpuUtil.cpp:198-206: filter-major, one dot per plane */
void pxo_backward_scale(const float* xnorm, const float* delta, int batch, int n, int size,
                        float* scale_updates)
{
    for (int c = 0; c < n; ++c)
        for (int b = 0; b < batch; ++b) {
            size_t off = (size_t) size * (c + (size_t) b * n);
            scale_updates[c] += dot_f32(delta + off, xnorm + off, size);
        }
}

/* CpuUtil.cpp:248-262 */
static void mean_impl(const float* x, int batch, int filters, int spatial, float* mean, int wide)
{
    const float scale = 1.0f / (batch * spatial);
    for (int c = 0; c < filters; ++c) {
        if (wide) {
            double acc = 0.0;
            for (int b = 0; b < batch; ++b) {
                const float* p = x + ((size_t) b * filters + c) * spatial;
                for (int k = 0; k < spatial; ++k) acc += p[k];
            }
            mean[c] = (float) acc * scale;
        } else {
            float acc = 0.0f;
            for (int b = 0; b < batch; ++b) {
                const float* p = x + ((size_t) b * filters + c) * spatial;
                for (int k = 0; k < spatial; ++k) acc += p[k];
            }
            mean[c] = acc * scale;
        }
    }
}

void pxo_mean(const float* x, int batch, int filters, int spatial, float* mean)
{
    mean_impl(x, batch, filters, spatial, mean, 0);
}

/* CpuUtil.cpp:264-280.  Population variance.  Each term is pow(double(x-mean), 2)
 * (exact in double for a float argument) and the float accumulator is updated
 * as float(double(acc) + term). */
static void variance_impl(const float* x, const float* mean, int batch, int filters, int spatial,
                          float* var, int wide)
{
    const float scale = 1.0f / (batch * spatial);
    for (int c = 0; c < filters; ++c) {
        const float mu = mean[c];
        if (wide) {
            double acc = 0.0;
            for (int b = 0; b < batch; ++b) {
                const float* p = x + ((size_t) b * filters + c) * spatial;
                for (int k = 0; k < spatial; ++k) {
                    double d = (double) (p[k] - mu);
                    acc += d * d;
                }
            }
            var[c] = (float) acc * scale;
        } else {
            float acc = 0.0f;
            for (int b = 0; b < batch; ++b) {
                const float* p = x + ((size_t) b * filters + c) * spatial;
                for (int k = 0; k < spatial; ++k) {
                    double d = (double) (p[k] - mu);
                    acc = (float) ((double) acc + d * d);
                }
            }
            var[c] = acc * scale;
        }
    }
}

void pxo_variance(const float* x, const float* mean, int batch, int filters, int spatial, float* var)
{
    variance_impl(x, mean, batch, filters, spatial, var, 0);
}

/* CpuUtil.cpp:282-292.  fp32 subtract; denominator sqrt(double(var)) + 1e-5f in
 * double; quotient rounded to float once. */
void pxo_normalize(float* x, const float* mean, const float* var, int batch, int filters, int spatial)
{
    for (int b = 0; b < batch; ++b)
        for (int c = 0; c < filters; ++c) {
            float* p = x + ((size_t) b * filters + c) * spatial;
            const float mu = mean[c];
            const double denom = sqrt((double) var[c]) + (double) .00001f;
            for (int k = 0; k < spatial; ++k) p[k] = (float) ((double) (p[k] - mu) / denom);
        }
}

/* CpuUtil.cpp:294-301 (cblas_sscal per plane) */
void pxo_scale_bias(float* out, const float* scales, int batch, int n, int size)
{
    for (int b = 0; b < batch; ++b)
        for (int c = 0; c < n; ++c) {
            float* p = out + ((size_t) b * n + c) * size;
            const float s = scales[c];
            for (int k = 0; k < size; ++k) p[k] = s * p[k];
        }
}

/* CpuUtil.cpp:303-312: plane sums in fp32, then *= (-1. / sqrtf(var + 1e-5f)) in double */
static void mean_delta_impl(const float* delta, const float* var, int batch, int filters,
                            int spatial, float* mean_delta, int wide)
{
    for (int c = 0; c < filters; ++c) {
        float acc = 0.0f;
        double wacc = 0.0;
        for (int b = 0; b < batch; ++b) {
            const float* p = delta + ((size_t) b * filters + c) * spatial;
            if (wide) {
                for (int k = 0; k < spatial; ++k) wacc += p[k];
            } else {
                acc += pxo_sum_array(p, spatial);
            }
        }
        if (wide) acc = (float) wacc;
        mean_delta[c] = (float) ((double) acc * (-1. / (double) sqrtf(var[c] + .00001f)));
    }
}

void pxo_mean_delta(const float* delta, const float* var, int batch, int filters, int spatial,
                    float* mean_delta)
{
    mean_delta_impl(delta, var, batch, filters, spatial, mean_delta, 0);
}

/* CpuUtil.cpp:314-327: all fp32; factor -.5f * powf(var + 1e-5f, -1.5f) */
static void variance_delta_impl(const float* x, const float* delta, const float* mean,
                                const float* var, int batch, int filters, int spatial,
                                float* var_delta, int wide)
{
    for (int c = 0; c < filters; ++c) {
        const float mu = mean[c];
        float acc = 0.0f;
        double wacc = 0.0;
        for (int b = 0; b < batch; ++b) {
            size_t off = ((size_t) b * filters + c) * spatial;
            for (int k = 0; k < spatial; ++k) {
                float term = delta[off + k] * (x[off + k] - mu);
                if (wide) wacc += term; else acc += term;
            }
        }
        if (wide) acc = (float) wacc;
        var_delta[c] = acc * (-.5f * powf(var[c] + .00001f, -3.0f / 2.0f));
    }
}

void pxo_variance_delta(const float* x, const float* delta, const float* mean, const float* var,
                        int batch, int filters, int spatial, float* var_delta)
{
    variance_delta_impl(x, delta, mean, var, batch, filters, spatial, var_delta, 0);
}

/* CpuUtil.cpp:329-342.  The expression is evaluated in double apart from
 * float(var + 1e-5f), float(x - mean) and float(mean_delta / float(count)). */
void pxo_normalize_delta(const float* x, const float* mean, const float* var, const float* mean_delta,
                         const float* var_delta, int batch, int filters, int spatial, float* delta)
{
    const int count = spatial * batch;
    for (int b = 0; b < batch; ++b)
        for (int c = 0; c < filters; ++c) {
            size_t off = ((size_t) b * filters + c) * spatial;
            const float mu = mean[c];
            const double root = sqrt((double) (var[c] + .00001f));
            const double vd = (double) var_delta[c];
            const float md_term = mean_delta[c] / (float) count;
            for (int k = 0; k < spatial; ++k) {
                double v = (double) delta[off + k] * 1. / root
                           + vd * 2. * (double) (x[off + k] - mu) / (double) count
                           + (double) md_term;
                delta[off + k] = (float) v;
            }
        }
}

/* CpuUtil.cpp:357-362 */
void pxo_constrain(int n, float alpha, float* x)
{
    for (int i = 0; i < n; ++i) x[i] = fminf(alpha, fmaxf(-alpha, x[i]));
}

/* ------------------------------------------------------------------ */
/* batch norm -- src/BatchNorm.cpp                                     */
/* ------------------------------------------------------------------ */

/* BatchNorm.cpp:24-67 */
void pxo_batchnorm_forward(int training, int batch, int channels, int height, int width,
                           const float* input, float* output, float* mean, float* var,
                           float* rolling_mean, float* rolling_var, const float* scales,
                           const float* biases, float* x, float* xnorm, int wide)
{
    const int spatial = height * width;
    const size_t total = (size_t) batch * channels * spatial;

    if (input != output) memcpy(output, input, total * sizeof(float));

    if (training) {
        memcpy(x, output, total * sizeof(float));
        mean_impl(output, batch, channels, spatial, mean, wide);
        variance_impl(output, mean, batch, channels, spatial, var, wide);
        /* sscal then saxpy: two roundings per statistic */
        for (int c = 0; c < channels; ++c) {
            float r = 0.99f * rolling_mean[c];
            rolling_mean[c] = r + .01f * mean[c];
        }
        for (int c = 0; c < channels; ++c) {
            float r = 0.99f * rolling_var[c];
            rolling_var[c] = r + .01f * var[c];
        }
        pxo_normalize(output, mean, var, batch, channels, spatial);
        memcpy(xnorm, output, total * sizeof(float));
    } else {
        pxo_normalize(output, rolling_mean, rolling_var, batch, channels, spatial);
    }
    pxo_scale_bias(output, scales, batch, channels, spatial);
    pxo_add_bias(output, biases, batch, channels, spatial);
}

/* BatchNorm.cpp:69-96 */
void pxo_batchnorm_backward(int batch, int channels, int height, int width, float* delta,
                            const float* mean, const float* var, float* mean_delta, float* var_delta,
                            const float* scales, float* scale_updates, float* bias_updates,
                            const float* x, const float* xnorm, int wide)
{
    const int spatial = height * width;
    if (wide) {
        for (int c = 0; c < channels; ++c) {
            double sb = 0.0, ss = 0.0;
            for (int b = 0; b < batch; ++b) {
                size_t off = ((size_t) b * channels + c) * spatial;
                for (int k = 0; k < spatial; ++k) {
                    sb += delta[off + k];
                    ss += (double) (delta[off + k] * xnorm[off + k]);
                }
            }
            bias_updates[c] += (float) sb;
            scale_updates[c] += (float) ss;
        }
    } else {
        pxo_backward_bias(bias_updates, delta, batch, channels, spatial);
        pxo_backward_scale(xnorm, delta, batch, channels, spatial, scale_updates);
    }
    pxo_scale_bias(delta, scales, batch, channels, spatial);
    mean_delta_impl(delta, var, batch, channels, spatial, mean_delta, wide);
    variance_delta_impl(x, delta, mean, var, batch, channels, spatial, var_delta, wide);
    pxo_normalize_delta(x, mean, var, mean_delta, var_delta, batch, channels, spatial, delta);
}

/* ------------------------------------------------------------------ */
/* conv-layer epilogue -- include/ConvLayer.h:227-252                  */
/* ------------------------------------------------------------------ */

void pxo_conv_epilogue_forward(int batch_normalize, int training, int act, int batch, int channels,
                               int height, int width, float* output, float* pre_activation,
                               float* mean, float* var, float* rolling_mean, float* rolling_var,
                               const float* scales, const float* biases, float* x, float* xnorm,
                               int wide)
{
    const size_t total = (size_t) batch * channels * height * width;
    if (batch_normalize) {
        pxo_batchnorm_forward(training, batch, channels, height, width, output, output, mean, var,
                              rolling_mean, rolling_var, scales, biases, x, xnorm, wide);
    } else {
        pxo_add_bias(output, biases, batch, channels, height * width);
    }
    if (pre_activation) memcpy(pre_activation, output, total * sizeof(float));
    pxo_activate(act, output, total);
}

void pxo_conv_epilogue_backward(int batch_normalize, int act, int batch, int channels, int height,
                                int width, float* delta, const float* pre_activation, const float* mean,
                                const float* var, float* mean_delta, float* var_delta,
                                const float* scales, float* scale_updates, float* bias_updates,
                                const float* x, const float* xnorm, int wide)
{
    const size_t total = (size_t) batch * channels * height * width;
    pxo_gradient(act, pre_activation, total, delta);
    if (batch_normalize) {
        pxo_batchnorm_backward(batch, channels, height, width, delta, mean, var, mean_delta, var_delta,
                               scales, scale_updates, bias_updates, x, xnorm, wide);
    } else {
        pxo_backward_bias(bias_updates, delta, batch, channels, height * width);
    }
}

/* ------------------------------------------------------------------ */
/* max-pool -- include/MaxPoolLayer.h                                  */
/* ------------------------------------------------------------------ */

/* MaxPoolLayer.h:62-63 */
int pxo_maxpool_out_dim(int in, int kernel, int stride, int padding)
{
    return (in + padding - kernel) / stride + 1;
}

/* MaxPoolLayer.h:88-135.  Window origin -padding/2 (C truncation); taps are
 * visited rows first then columns; an in-bounds tap replaces the running
 * maximum when none has been taken yet or when it compares strictly greater. */
void pxo_maxpool_forward(const float* in, float* out, int* indexes, int batch, int channels,
                         int ih, int iw, int oh, int ow, int kernel, int stride, int padding)
{
    const int origin = -padding / 2;
    for (int b = 0; b < batch; ++b)
        for (int c = 0; c < channels; ++c) {
            const int plane = c + channels * b;
            for (int oy = 0; oy < oh; ++oy)
                for (int ox = 0; ox < ow; ++ox) {
                    float best = -FLT_MAX;
                    int best_at = -1;
                    for (int ky = 0; ky < kernel; ++ky) {
                        int y = origin + oy * stride + ky;
                        if (y < 0 || y >= ih) continue;
                        for (int kx = 0; kx < kernel; ++kx) {
                            int xx = origin + ox * stride + kx;
                            if (xx < 0 || xx >= iw) continue;
                            int at = xx + iw * (y + ih * plane);
                            float v = in[at];
                            if (best_at < 0 || v > best) {
                                best_at = at;
                                best = v;
                            }
                        }
                    }
                    int o = ox + ow * (oy + oh * plane);
                    out[o] = best;
                    indexes[o] = best_at;
                }
        }
}

/* MaxPoolLayer.h:137-158: ascending output order */
void pxo_maxpool_backward(const float* delta, const int* indexes, float* grad, size_t size)
{
    for (size_t i = 0; i < size; ++i) {
        int at = indexes[i];
        if (at >= 0) grad[at] += delta[i];
    }
}

/* ------------------------------------------------------------------ */
/* upsample -- include/UpsampleLayer.h:97-121                          */
/* ------------------------------------------------------------------ */

void pxo_upsample(const float* in, int w, int h, int c, int batch, int stride, int forward,
                  float scale, float* acc, float* out)
{
    const int ow = w * stride, oh = h * stride;
    for (int b = 0; b < batch; ++b)
        for (int k = 0; k < c; ++k) {
            const size_t ibase = ((size_t) b * c + k) * w * h;
            const size_t obase = ((size_t) b * c + k) * ow * oh;
            for (int j = 0; j < oh; ++j)
                for (int i = 0; i < ow; ++i) {
                    size_t ii = ibase + (size_t) (j / stride) * w + i / stride;
                    size_t oi = obase + (size_t) j * ow + i;
                    if (forward) out[oi] = scale * in[ii];
                    else acc[ii] += scale * out[oi];
                }
        }
}

/* ------------------------------------------------------------------ */
/* shortcut -- include/ShortcutLayer.h                                 */
/* ------------------------------------------------------------------ */

/* ShortcutLayer.h:113-141; returns non-zero when the x/y stride or sample
 * factors disagree (the reference throws there). */
int pxo_shortcut(int batch, int w1, int h1, int c1, const float* add, int w2, int h2, int c2,
                 float out_scale, float add_scale, float* out)
{
    int stride = w1 / w2; if (stride < 1) stride = 1;
    int sample = w2 / w1; if (sample < 1) sample = 1;
    if (stride != h1 / h2) return 1;
    if (sample != h2 / h1) return 1;
    const int minw = w1 < w2 ? w1 : w2;
    const int minh = h1 < h2 ? h1 : h2;
    const int minc = c1 < c2 ? c1 : c2;
    for (int b = 0; b < batch; ++b)
        for (int k = 0; k < minc; ++k)
            for (int j = 0; j < minh; ++j)
                for (int i = 0; i < minw; ++i) {
                    size_t oi = (size_t) i * sample + (size_t) w2 * (j * sample + (size_t) h2 * (k + (size_t) c2 * b));
                    size_t ai = (size_t) i * stride + (size_t) w1 * (j * stride + (size_t) h1 * (k + (size_t) c1 * b));
                    out[oi] = out_scale * out[oi] + add_scale * add[ai];
                }
    return 0;
}

/* ShortcutLayer.h:84-96: copy input, blend with the source layer's output, keep
 * the pre-activation, activate.  The call site passes this layer's own
 * dimensions on both sides, so both index maps are the identity. */
void pxo_shortcut_forward(int act, int batch, int w, int h, int c, const float* input,
                          const float* from_output, float alpha, float beta, float* output,
                          float* pre_activation)
{
    const size_t total = (size_t) batch * c * h * w;
    memcpy(output, input, total * sizeof(float));
    pxo_shortcut(batch, w, h, c, from_output, w, h, c, alpha, beta, output);
    if (pre_activation) memcpy(pre_activation, output, total * sizeof(float));
    pxo_activate(act, output, total);
}

/* ShortcutLayer.h:98-111 */
void pxo_shortcut_backward(int act, int batch, int w, int h, int c, float* delta,
                           const float* pre_activation, float* from_delta, float* grad,
                           float alpha, float beta)
{
    const size_t total = (size_t) batch * c * h * w;
    pxo_gradient(act, pre_activation, total, delta);
    pxo_shortcut(batch, w, h, c, delta, w, h, c, 1.0f, beta, from_delta);
    if (grad) pxo_axpy(total, alpha, delta, grad);
}

/* cblas_saxpy as used at ShortcutLayer.h:109 and YoloLayer.h:748 */
void pxo_axpy(size_t n, float alpha, const float* x, float* y)
{
    for (size_t i = 0; i < n; ++i) y[i] = y[i] + alpha * x[i];
}

/* include/RouteLayer.h:91-113: cblas_scopy of each image of one source layer into its slice */
void pxo_route_forward(const float* layer_output, float* route_output, int batch, int layer_outputs,
                       int route_outputs, int offset)
{
    for (int b = 0; b < batch; ++b) {
        const float* in = layer_output + (size_t) b * layer_outputs;
        float* out = route_output + (size_t) b * route_outputs + offset;
        for (int i = 0; i < layer_outputs; ++i) out[i] = in[i];
    }
}

/* include/RouteLayer.h:115-137: cblas_saxpy(alpha = 1) of each slice into the source layer's delta */
void pxo_route_backward(const float* route_delta, float* layer_delta, int batch, int layer_outputs,
                        int route_outputs, int offset)
{
    for (int b = 0; b < batch; ++b)
        pxo_axpy((size_t) layer_outputs, 1.0f, route_delta + (size_t) b * route_outputs + offset,
                 layer_delta + (size_t) b * layer_outputs);
}

/* ------------------------------------------------------------------ */
/* boxes -- src/DarkBox.cpp:84-151                                     */
/* ------------------------------------------------------------------ */

typedef struct { float x, y, w, h; } rect_f;  /* top-left + size */

/* DarkBox.cpp:84-118: the half-extent is only subtracted for a positive extent */
static rect_f box_rect(const float b[4])
{
    rect_f r;
    r.x = b[2] > 0.0f ? b[0] - b[2] / 2.0f : b[0];
    r.y = b[3] > 0.0f ? b[1] - b[3] / 2.0f : b[1];
    r.w = b[2];
    r.h = b[3];
    return r;
}

/* cv::Rect_<float>::operator& of OpenCV >= 4.5.4 (the version floor in the
 * reference's CMakeLists.txt:86; modules/core/include/opencv2/core/types.hpp).
 * Either operand empty (w <= 0 or h <= 0) gives the empty rectangle; with
 * lo/hi the operands ordered by left (resp. top) edge, the overlap extent is
 * min(lo.size - (hi.origin - lo.origin), hi.size); a negative-origin early-out
 * returns empty when lo.origin + lo.size < hi.origin; a non-positive extent
 * gives the empty rectangle. */
static float rect_intersection_area(rect_f a, rect_f b)
{
    if (a.w <= 0.0f || a.h <= 0.0f || b.w <= 0.0f || b.h <= 0.0f) return 0.0f;
    const rect_f* xlo = (a.x < b.x) ? &a : &b;
    const rect_f* xhi = (a.x < b.x) ? &b : &a;
    const rect_f* ylo = (a.y < b.y) ? &a : &b;
    const rect_f* yhi = (a.y < b.y) ? &b : &a;
    if ((xlo->x < 0.0f && xlo->x + xlo->w < xhi->x) || (ylo->y < 0.0f && ylo->y + ylo->h < yhi->y))
        return 0.0f;
    float iw = fminf(xlo->w - (xhi->x - xlo->x), xhi->w);
    float ih = fminf(ylo->h - (yhi->y - ylo->y), yhi->h);
    if (iw <= 0.0f || ih <= 0.0f) return 0.0f;
    return iw * ih;
}

/* DarkBox.cpp:120-131 */
float pxo_box_intersection(const float a[4], const float b[4])
{
    return rect_intersection_area(box_rect(a), box_rect(b));
}

/* DarkBox.cpp:133-136 */
float pxo_box_union(const float a[4], const float b[4])
{
    float u = a[2] * a[3] + b[2] * b[3] - pxo_box_intersection(a, b);
    return u > 0.0f ? u : 0.0f;
}

/* DarkBox.cpp:138-147 */
float pxo_box_iou(const float a[4], const float b[4])
{
    float i = pxo_box_intersection(a, b);
    float u = pxo_box_union(a, b);
    if (u == 0.0f) return 0.0f;
    return i / u;
}

/* ------------------------------------------------------------------ */
/* YOLO head -- include/YoloLayer.h                                    */
/* ------------------------------------------------------------------ */

/* YoloLayer.h:730-739 */
static size_t yolo_entry(const pxo_yolo_cfg* g, int b, int location, int entry)
{
    int area = g->width * g->height;
    if (area < 1) area = 1;
    int n = location / area;
    int loc = location % area;
    size_t outputs = (size_t) g->width * g->height * g->num_masks * (g->classes + 5);
    return (size_t) b * outputs + (size_t) n * area * (g->classes + 5) + (size_t) entry * area + loc;
}

/* YoloLayer.h:164-196: copy, logistic on x, y and on objectness + classes */
void pxo_yolo_decode(const pxo_yolo_cfg* g, const float* input, float* output)
{
    int area = g->width * g->height;
    if (area < 1) area = 1;
    size_t outputs = (size_t) g->width * g->height * g->num_masks * (g->classes + 5);
    memcpy(output, input, (size_t) g->batch * outputs * sizeof(float));
    for (int b = 0; b < g->batch; ++b)
        for (int n = 0; n < g->num_masks; ++n) {
            float* p = output + yolo_entry(g, b, n * area, 0);
            pxo_activate(PXO_LOGISTIC, p, (size_t) 2 * area);
            p = output + yolo_entry(g, b, n * area, 4);
            pxo_activate(PXO_LOGISTIC, p, (size_t) (1 + g->classes) * area);
        }
}

/* YoloLayer.h:637-651; anchors are ints, network size ints */
static void yolo_box(const pxo_yolo_cfg* g, const float* p, int anchor, size_t index, int i, int j,
                     float box[4])
{
    size_t stride = (size_t) g->width * g->height;
    box[0] = ((float) i + p[index]) / (float) g->width;
    box[1] = ((float) j + p[index + stride]) / (float) g->height;
    box[2] = expf(p[index + 2 * stride]) * (float) g->anchors[2 * anchor] / (float) g->net_width;
    box[3] = expf(p[index + 3 * stride]) * (float) g->anchors[2 * anchor + 1] / (float) g->net_height;
}

/* YoloLayer.h:408-436; returns IoU(pred, truth) */
static float yolo_delta_box(const pxo_yolo_cfg* g, const float* out, float* delta, const float truth[4],
                            int anchor, size_t index, int i, int j)
{
    float pred[4];
    yolo_box(g, out, anchor, index, i, j, pred);
    float iou = pxo_box_iou(pred, truth);
    size_t stride = (size_t) g->width * g->height;

    float tx = truth[0] * (float) g->width - (float) i;
    float ty = truth[1] * (float) g->height - (float) j;
    float tw = logf(fmaxf(1e-9f, truth[2] * (float) g->net_width / (float) g->anchors[2 * anchor]));
    float th = logf(fmaxf(1e-9f, truth[3] * (float) g->net_height / (float) g->anchors[2 * anchor + 1]));
    float scale = g->coord_scale * (2.0f - truth[2] * truth[3]);

    delta[index] = scale * (tx - out[index]);
    delta[index + stride] = scale * (ty - out[index + stride]);
    delta[index + 2 * stride] = scale * (tw - out[index + 2 * stride]);
    delta[index + 3 * stride] = scale * (th - out[index + 3 * stride]);
    return iou;
}

/* YoloLayer.h:390-406 */
static void yolo_delta_class(const pxo_yolo_cfg* g, const float* out, float* delta, size_t index,
                             int class_id, float* avg_cat)
{
    size_t stride = (size_t) g->width * g->height;
    for (int k = 0; k < g->classes; ++k) {
        float t = (k == class_id) ? 1.0f : 0.0f;
        delta[index + k * stride] = g->class_scale * (t - out[index + k * stride]);
        if (t != 0.0f) *avg_cat += fminf(1.0f, out[index + k * stride]);
    }
}

static int yolo_mask_index(const pxo_yolo_cfg* g, int anchor)
{
    for (int k = 0; k < g->num_masks; ++k)
        if (g->mask[k] == anchor) return k;
    return -1;
}

/* best anchor over ALL anchors against the origin-shifted truth,
 * YoloLayer.h:467-478 == YoloTargetBuilder.cpp:34-46 */
static int yolo_best_anchor(const pxo_yolo_cfg* g, const float truth[4])
{
    float shifted[4] = { 0.0f, 0.0f, truth[2], truth[3] };
    float best = -FLT_MAX;
    int best_n = 0;
    for (int n = 0; n < g->num_anchors; ++n) {
        float cand[4] = { 0.0f, 0.0f,
                          (float) g->anchors[2 * n] / (float) g->net_width,
                          (float) g->anchors[2 * n + 1] / (float) g->net_height };
        float iou = pxo_box_iou(cand, shifted);
        if (iou > best) { best = iou; best_n = n; }
    }
    return best_n;
}

static int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

/* YoloLayer.h:164-239 (forwardCpu in a loss-computing mode), 450-547, 562-599 */
void pxo_yolo_forward(const pxo_yolo_cfg* g, const float* input, const float* truths,
                      const int* truth_counts, int max_truth, float* output, float* delta,
                      float* cost, float* stats)
{
    const int W = g->width, H = g->height;
    const int area = W * H;
    const size_t outputs = (size_t) area * g->num_masks * (g->classes + 5);
    const size_t total = (size_t) g->batch * outputs;

    pxo_yolo_decode(g, input, output);
    memset(delta, 0, total * sizeof(float));

    float avg_iou = 0, recall = 0, recall75 = 0, avg_cat = 0, avg_obj = 0, avg_anyobj = 0;
    int count = 0, class_count = 0;

    for (int b = 0; b < g->batch; ++b) {
        const float* tb = truths + (size_t) b * max_truth * 5;
        const int nt = truth_counts[b];

        /* processRegion for every cell, row-major (212-216, 511-547) */
        for (int j = 0; j < H; ++j)
            for (int i = 0; i < W; ++i)
                for (int n = 0; n < g->num_masks; ++n) {
                    int entry = n * area + j * W + i;
                    size_t box_index = yolo_entry(g, b, entry, 0);
                    float pred[4];
                    yolo_box(g, output, g->mask[n], box_index, i, j, pred);

                    /* bestGT 752-767: strict >, first wins */
                    float best = -FLT_MAX;
                    int best_t = -1;
                    for (int t = 0; t < nt; ++t) {
                        float iou = pxo_box_iou(pred, tb + 5 * t);
                        if (iou > best) { best = iou; best_t = t; }
                    }

                    size_t obj_index = yolo_entry(g, b, entry, 4);
                    avg_anyobj += output[obj_index];
                    if (best_t < 0 || best < g->ignore_thresh)
                        delta[obj_index] = g->noobject_scale * (0.0f - output[obj_index]);
                    if (best_t >= 0 && best > g->truth_thresh) {
                        delta[obj_index] = g->object_scale * (1.0f - output[obj_index]);
                        size_t cls_index = yolo_entry(g, b, entry, 5);
                        yolo_delta_class(g, output, delta, cls_index, (int) tb[5 * best_t + 4], &avg_cat);
                        yolo_delta_box(g, output, delta, tb + 5 * best_t, g->mask[n], box_index, i, j);
                    }
                }

        /* processObjects (217, 450-509): truths in order, later overwrites earlier */
        for (int t = 0; t < nt; ++t) {
            const float* gt = tb + 5 * t;
            int i = clampi((int) (gt[0] * (float) W), 0, W - 1);
            int j = clampi((int) (gt[1] * (float) H), 0, H - 1);
            int best_n = yolo_best_anchor(g, gt);
            int mask_n = yolo_mask_index(g, best_n);
            if (mask_n < 0) continue;
            int location = mask_n * area + j * W + i;
            size_t box_index = yolo_entry(g, b, location, 0);
            float iou = yolo_delta_box(g, output, delta, gt, best_n, box_index, i, j);
            size_t obj_index = yolo_entry(g, b, location, 4);
            avg_obj += output[obj_index];
            delta[obj_index] = g->object_scale * (1.0f - output[obj_index]);
            size_t cls_index = yolo_entry(g, b, location, 5);
            yolo_delta_class(g, output, delta, cls_index, (int) gt[4], &avg_cat);
            ++count;
            ++class_count;
            if (iou > .5) recall += 1.0f;
            if (iou > .75) recall75 += 1.0f;
            avg_iou += iou;
        }
    }

    /* 221: cost = pow(|delta|_2, 2) / max(1, batch), evaluated in double */
    float mag = pxo_mag_array(delta, total);
    *cost = (float) (pow((double) mag, 2) / (double) (g->batch > 1 ? g->batch : 1));

    /* updateLossComponents 562-599 */
    float box_cost = 0, obj_cost = 0, noobj_cost = 0, class_cost = 0;
    for (int b = 0; b < g->batch; ++b)
        for (int n = 0; n < g->num_masks; ++n)
            for (int cell = 0; cell < area; ++cell) {
                size_t base = yolo_entry(g, b, n * area + cell, 0);
                for (int k = 0; k < 4; ++k) {
                    float v = delta[base + (size_t) k * area];
                    box_cost += v * v;
                }
                float o = delta[base + (size_t) 4 * area];
                if (o >= 0.0f) obj_cost += o * o; else noobj_cost += o * o;
                for (int k = 0; k < g->classes; ++k) {
                    float v = delta[base + (size_t) (5 + k) * area];
                    class_cost += v * v;
                }
            }

    if (stats) {
        stats[0] = avg_iou; stats[1] = recall; stats[2] = recall75; stats[3] = avg_cat;
        stats[4] = avg_obj; stats[5] = avg_anyobj; stats[6] = (float) count;
        stats[7] = (float) class_count; stats[8] = box_cost; stats[9] = obj_cost;
        stats[10] = noobj_cost; stats[11] = class_cost;
    }
}

/* src/YoloTargetBuilder.cpp:21-62 for one image; tables are [num_masks * area] */
int pxo_yolo_build_targets(const pxo_yolo_cfg* g, const float* truths, int count,
                           int* classes, int* anchors, float* boxes)
{
    const int area = g->width * g->height;
    const int slots = g->num_masks * area;
    for (int s = 0; s < slots; ++s) {
        classes[s] = -1;
        anchors[s] = -1;
        boxes[4 * s] = boxes[4 * s + 1] = boxes[4 * s + 2] = boxes[4 * s + 3] = 0.0f;
    }
    int assigned = 0;
    for (int t = 0; t < count; ++t) {
        const float* gt = truths + 5 * t;
        int best = yolo_best_anchor(g, gt);
        int mask_slot = yolo_mask_index(g, best);
        if (mask_slot < 0) continue;
        int x = clampi((int) (gt[0] * (float) g->width), 0, g->width - 1);
        int y = clampi((int) (gt[1] * (float) g->height), 0, g->height - 1);
        int slot = mask_slot * area + y * g->width + x;
        classes[slot] = (int) gt[4];
        anchors[slot] = best;
        memcpy(boxes + 4 * slot, gt, 4 * sizeof(float));
        ++assigned;
    }
    return assigned;
}

/* ------------------------------------------------------------------ */
/* Adam -- include/cuda/Adam.h:49-90 + src/Adam.cu:26-37               */
/* ------------------------------------------------------------------ */

/* One fp32 rounding per BLAS call of the reference sequence, in its order:
 * scale the update by 1/batch; fold L2 decay into it (weights only); decay
 * both moments; add the update / its square; bias-corrected step ADDED to the
 * weights (updates are negative gradients); clear the update buffer.
 * apply_decay: 0 no decay; 1 the reference's L2 term, folded into the update before
 * the moments; 2 decoupled decay, w += step - (lr * decay) * w with the moments formed
 * from the plain update.  The reference has no such form (parity unpinned by the
 * reference): it is the textbook AdamW recurrence in the reference's sign convention,
 * held against that recurrence in fp64 and against its closed form at t = 1. */
void pxo_adam_update(size_t n, float* w, float* d, float* m, float* v, int batch, int t, float lr,
                     float beta1, float beta2, float eps, float decay, int apply_decay)
{
    const float inv_batch = 1.0f / (float) batch;
    const float neg_decay = -decay;
    const float neg_lr_decay = -(lr * decay);
    const float a1 = 1.0f - beta1;
    const float a2 = 1.0f - beta2;
    const float c1 = 1.0f - powf(beta1, (float) t);
    const float c2 = 1.0f - powf(beta2, (float) t);
    for (size_t i = 0; i < n; ++i) {
        float g = d[i] * inv_batch;
        if (apply_decay == 1) {
            float l2 = neg_decay * w[i];
            g = g + l2;
        }
        float mi = m[i] * beta1;
        float vi = v[i] * beta2;
        float am = a1 * g;
        mi = mi + am;
        float g2 = g * g;
        float av = a2 * g2;
        vi = vi + av;
        float mhat = mi / c1;
        float vhat = vi / c2;
        float step = lr * mhat / (sqrtf(vhat) + eps);
        float wi = w[i] + step;
        if (apply_decay == 2) {
            float shrink = neg_lr_decay * w[i];
            wi = wi + shrink;
        }
        w[i] = wi;
        m[i] = mi;
        v[i] = vi;
        d[i] = 0.0f;
    }
}

/* ------------------------------------------------------------------ */
/* SGD with momentum -- include/ConvLayer.h:309-311                    */
/* ------------------------------------------------------------------ */

/* three BLAS passes: saxpy(-decay*batch, w, d); saxpy(lr/batch, d, w); sscal(momentum, d) */
void pxo_sgd_update(size_t n, float* w, float* d, int batch, float lr, float momentum, float decay,
                    int apply_decay)
{
    const float a0 = -decay * (float) batch;
    const float a1 = lr / (float) batch;
    if (apply_decay) pxo_axpy(n, a0, w, d);
    pxo_axpy(n, a1, d, w);
    for (size_t i = 0; i < n; ++i) d[i] = momentum * d[i];
}

/* ------------------------------------------------------------------ */
/* gradient rescale + clip -- include/Layer.h:385-397, 479-499         */
/* ------------------------------------------------------------------ */

/* scaleTensor (when threshold > 0) then constrain (when clip > 0); returns the norm before */
float pxo_rescale_clip(float* x, size_t n, float threshold, float clip)
{
    const float norm = pxo_mag_array(x, n);
    if (threshold > 0.0f && norm > 0.0f && norm > threshold) {
        const float scale = threshold / norm;
        for (size_t i = 0; i < n; ++i) x[i] = scale * x[i];
    }
    if (clip > 0.0f) pxo_constrain((int) n, clip, x);
    return norm;
}

/* ------------------------------------------------------------------ */
/* detections -- include/YoloLayer.h:601-698                           */
/* ------------------------------------------------------------------ */

/* YoloLayer.h:601-634: box in pixels of a w x h image that was letterboxed into the network input.
 * The float expressions are converted to int by std::max<int> / std::min<int> (truncation). */
static void yolo_scaled_box(const pxo_yolo_cfg* g, const float* p, int anchor, size_t index, int i, int j,
                            int w, int h, float box[4])
{
    const size_t stride = (size_t) g->width * g->height;
    const int netW = g->net_width, netH = g->net_height;
    int newW, newH;
    if (((float) netW / w) < ((float) netH / h)) {
        newW = netW;
        newH = (h * netW) / w;
    } else {
        newH = netH;
        newW = (w * netH) / h;
    }
    float x = ((float) i + p[index]) / (float) g->width;
    x = (x - (float) (netW - newW) / 2.0f / (float) netW) / ((float) newW / (float) netW);
    float y = ((float) j + p[index + stride]) / (float) g->height;
    y = (y - (float) (netH - newH) / 2.0f / (float) netH) / ((float) newH / (float) netH);
    float width = expf(p[index + 2 * stride]) * (float) g->anchors[2 * anchor] / (float) netW;
    width *= (float) netW / (float) newW;
    float height = expf(p[index + 3 * stride]) * (float) g->anchors[2 * anchor + 1] / (float) netH;
    height *= (float) netH / (float) newH;
    int left = (int) ((x - width / 2) * (float) w);
    if (left < 0) left = 0;
    int right = (int) ((x + width / 2) * (float) w);
    if (right > w - 1) right = w - 1;
    int top = (int) ((y - height / 2) * (float) h);
    if (top < 0) top = 0;
    int bottom = (int) ((y + height / 2) * (float) h);
    if (bottom > h - 1) bottom = h - 1;
    box[0] = (float) left; box[1] = (float) top;
    box[2] = (float) (right - left); box[3] = (float) (bottom - top);
}

int pxo_yolo_detections(const pxo_yolo_cfg* g, const float* predictions, float threshold,
                        int image_width, int image_height, pxo_detection* out, int capacity)
{
    const int scaled = image_width > 0 && image_height > 0;
    int area = g->width * g->height;
    if (area < 1) area = 1;
    int found = 0;
    for (int b = 0; b < g->batch; ++b)
        for (int i = 0; i < area; ++i) {
            const int row = i / g->width, col = i % g->width;
            for (int n = 0; n < g->num_masks; ++n) {
                const float objectness = predictions[yolo_entry(g, b, n * area + i, 4)];
                if (objectness < threshold) continue;
                const size_t box_index = yolo_entry(g, b, n * area + i, 0);
                float box[4];
                if (scaled) {
                    yolo_scaled_box(g, predictions, g->mask[n], box_index, col, row, image_width, image_height, box);
                } else {
                    /* yoloBox(...).rect(): left/top fall back to the centre for a non-positive size */
                    float c[4];
                    yolo_box(g, predictions, g->mask[n], box_index, col, row, c);
                    box[0] = c[2] > 0.0f ? c[0] - c[2] / 2.0f : c[0];
                    box[1] = c[3] > 0.0f ? c[1] - c[3] / 2.0f : c[1];
                    box[2] = c[2]; box[3] = c[3];
                }
                for (int j = 0; j < g->classes; ++j) {
                    const float prob = objectness * predictions[yolo_entry(g, b, n * area + i, 5 + j)];
                    if (prob >= threshold) {
                        if (found < capacity) {
                            pxo_detection* d = out + found;
                            d->x = box[0]; d->y = box[1]; d->w = box[2]; d->h = box[3];
                            d->prob = prob; d->batch = b; d->class_index = j;
                            d->order = (unsigned) ((((size_t) b * area + i) * g->num_masks + n) * g->classes + j);
                        }
                        ++found;
                    }
                }
            }
        }
    return found;
}

/* ------------------------------------------------------------------ */
/* non-maximum suppression -- src/Box.cpp                              */
/* ------------------------------------------------------------------ */

/* Box.cpp:47-54 */
static rect_f nms_normalized_rect(const pxo_detection* d)
{
    const float xe = d->x + d->w, ye = d->y + d->h;
    const float x1 = d->x < xe ? d->x : xe, y1 = d->y < ye ? d->y : ye;
    const float x2 = d->x < xe ? xe : d->x, y2 = d->y < ye ? ye : d->y;
    rect_f r;
    r.x = x1; r.y = y1;
    r.w = x2 - x1 > 0.0f ? x2 - x1 : 0.0f;
    r.h = y2 - y1 > 0.0f ? y2 - y1 : 0.0f;
    return r;
}

/* Box.cpp:25-45: areas and overlap are floats, the union is clamped at zero, and a quotient that is
 * not finite counts as no overlap */
static float nms_iou(rect_f a, rect_f b)
{
    const float inter = rect_intersection_area(a, b);
    float uni = a.w * a.h + b.w * b.h - inter;
    if (!(0.0f < uni)) uni = 0.0f;
    const float q = inter / uni;
    if (isnan(q) || isinf(q)) return 0.0f;
    return q;
}

typedef struct nms_item {
    const pxo_detection* det;
    int position;           /* place in the input sequence */
} nms_item;

static int nms_by_prob(const void* pa, const void* pb)
{
    const nms_item* a = (const nms_item*) pa;
    const nms_item* b = (const nms_item*) pb;
    if (a->det->prob > b->det->prob) return -1;
    if (b->det->prob > a->det->prob) return 1;
    return a->position < b->position ? -1 : (a->position > b->position ? 1 : 0);   /* stable */
}

typedef struct nms_member {
    unsigned long long key;     /* image << 32 | class */
    int sorted;                 /* place in the sequence sorted by probability */
} nms_member;

static int nms_by_group(const void* pa, const void* pb)
{
    const nms_member* a = (const nms_member*) pa;
    const nms_member* b = (const nms_member*) pb;
    if (a->key != b->key) return a->key < b->key ? -1 : 1;
    return a->sorted < b->sorted ? -1 : (a->sorted > b->sorted ? 1 : 0);
}

/* Box.cpp:56-147.  The reference finds the earlier boxes of a group through an R-tree query for
 * intersecting rectangles and then tests their overlap ratio; a ratio above a non-negative
 * threshold implies a positive overlap, so testing every earlier kept box of the group decides the
 * same.  Only the first 1024 members of a group (in sorted order, counting those the first pass
 * discarded) are visited; later ones stay. */
int pxo_nms(const pxo_detection* detections, int count, float threshold, pxo_detection* out)
{
    if (count <= 0) return 0;
    nms_item* items = (nms_item*) malloc(sizeof(nms_item) * (size_t) count);
    rect_f* rects = (rect_f*) malloc(sizeof(rect_f) * (size_t) count);
    char* discard = (char*) calloc((size_t) count, 1);
    nms_member* members = (nms_member*) malloc(sizeof(nms_member) * (size_t) count);
    int* kept = (int*) malloc(sizeof(int) * 1024);
    for (int i = 0; i < count; ++i) { items[i].det = detections + i; items[i].position = i; }
    qsort(items, (size_t) count, sizeof(nms_item), nms_by_prob);
    for (int i = 0; i < count; ++i) rects[i] = nms_normalized_rect(items[i].det);

    /* near-identical boxes of different classes in one image: the strongest stays (65-88) */
    for (int i = 0; i < count; ++i)
        for (int j = 0; j < i; ++j) {
            if (discard[j] || items[i].det->batch != items[j].det->batch ||
                items[i].det->class_index == items[j].det->class_index)
                continue;
            if (nms_iou(rects[i], rects[j]) > 0.9f) { discard[i] = 1; break; }
        }

    /* greedy suppression inside each (image, class) group (90-136) */
    for (int i = 0; i < count; ++i) {
        members[i].key = ((unsigned long long) (unsigned) items[i].det->batch << 32) |
                         (unsigned) items[i].det->class_index;
        members[i].sorted = i;
    }
    qsort(members, (size_t) count, sizeof(nms_member), nms_by_group);
    for (int start = 0; start < count;) {
        int end = start;
        while (end < count && members[end].key == members[start].key) ++end;
        const int visit = end - start < 1024 ? end - start : 1024;
        int n_kept = 0;
        for (int p = 0; p < visit; ++p) {
            const int i = members[start + p].sorted;
            if (discard[i]) continue;
            int suppressed = 0;
            for (int k = 0; k < n_kept && !suppressed; ++k)
                if (nms_iou(rects[i], rects[kept[k]]) > threshold) suppressed = 1;
            if (suppressed) discard[i] = 1;
            else kept[n_kept++] = i;
        }
        start = end;
    }

    int n_out = 0;
    for (int i = 0; i < count; ++i)
        if (!discard[i]) out[n_out++] = *items[i].det;
    free(items); free(rects); free(discard); free(members); free(kept);
    return n_out;
}
