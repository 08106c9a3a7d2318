/*
 * px_oracle.h -- CPU restatement of PixieNN's non-convolution CPU layer math.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker the HIP kernels are
 * compared with (and the CPU baseline bench.py times).  Nothing in the product
 * package links, loads or calls it.
 *
 * Every function restates, in plain single-threaded C, the arithmetic of the
 * reference CPU path, including the places where the reference promotes to
 * double or rounds to float between passes.  Citations are
 * <file>:<lines> inside the reference tree.
 *
 * Build: gcc -O2 -ffp-contract=off (no FMA contraction: the reference is
 * built for baseline x86-64 where the compiler cannot fuse).
 */
#ifndef PX_ORACLE_H
#define PX_ORACLE_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* include/ActivationTypes.h:19-30 */
enum pxo_activation {
    PXO_LEAKY = 0, PXO_LINEAR, PXO_LOGGY, PXO_LOGISTIC, PXO_MISH,
    PXO_RELU, PXO_SOFTPLUS, PXO_SWISH, PXO_TANH
};

/* ---- activations: include/Activation.h:40-228, 292-324 ---- */
float pxo_act_apply(int type, float x);
float pxo_act_gradient(int type, float x);
void pxo_activate(int type, float* x, size_t n);
void pxo_gradient(int type, const float* x, size_t n, float* delta);

/* ---- per-channel primitives: src/CpuUtil.cpp:178-219, 248-342 ---- */
void pxo_add_bias(float* out, const float* bias, int batch, int n, int size);
void pxo_backward_bias(float* bias_updates, const float* delta, int batch, int n, int size);
void pxo_backward_scale(const float* xnorm, const float* delta, int batch, int n, int size,
                        float* scale_updates);
float pxo_sum_array(const float* a, int n);
float pxo_mag_array(const float* a, size_t n);
void pxo_mean(const float* x, int batch, int filters, int spatial, float* mean);
void pxo_variance(const float* x, const float* mean, int batch, int filters, int spatial, float* var);
void pxo_normalize(float* x, const float* mean, const float* var, int batch, int filters, int spatial);
void pxo_scale_bias(float* out, const float* scales, int batch, int n, int size);
void pxo_mean_delta(const float* delta, const float* var, int batch, int filters, int spatial,
                    float* mean_delta);
void pxo_variance_delta(const float* x, const float* delta, const float* mean, const float* var,
                        int batch, int filters, int spatial, float* var_delta);
void pxo_normalize_delta(const float* x, const float* mean, const float* var, const float* mean_delta,
                         const float* var_delta, int batch, int filters, int spatial, float* delta);
void pxo_constrain(int n, float alpha, float* x);

/* ---- batch norm: src/BatchNorm.cpp:24-96 ----
 * wide != 0 selects the tie-breaker variant: identical arithmetic except that
 * the per-channel running sums are carried in double.  It is NOT what the
 * reference computes; tests use it to measure how far the reference's own
 * sequential fp32 accumulation sits from the exact sums. */
void pxo_batchnorm_forward(int training, int batch, int channels, int height, int width,
                           const float* input, float* output, float* mean, float* var,
                           float* rolling_mean, float* rolling_var, const float* scales,
                           const float* biases, float* x, float* xnorm, int wide);
void pxo_batchnorm_backward(int batch, int channels, int height, int width, float* delta,
                            const float* mean, const float* var, float* mean_delta, float* var_delta,
                            const float* scales, float* scale_updates, float* bias_updates,
                            const float* x, const float* xnorm, int wide);

/* ---- conv-layer epilogue (everything after the GEMM): include/ConvLayer.h:227-252 ---- */
void pxo_conv_epilogue_forward(int batch_normalize, int training, int act, int batch, int channels,
                               int height, int width, float* output /* conv result in, activation out */,
                               float* pre_activation, float* mean, float* var, float* rolling_mean,
                               float* rolling_var, const float* scales, const float* biases,
                               float* x, float* xnorm, int wide);
void pxo_conv_epilogue_backward(int batch_normalize, int act, int batch, int channels, int height,
                                int width, float* delta, const float* pre_activation, const float* mean,
                                const float* var, float* mean_delta, float* var_delta,
                                const float* scales, float* scale_updates, float* bias_updates,
                                const float* x, const float* xnorm, int wide);

/* ---- max-pool: include/MaxPoolLayer.h:51-71 (geometry), 88-135, 137-158 ---- */
int pxo_maxpool_out_dim(int in, int kernel, int stride, int padding);
void pxo_maxpool_forward(const float* in, float* out, int* indexes, int batch, int channels,
                         int ih, int iw, int oh, int ow, int kernel, int stride, int padding);
void pxo_maxpool_backward(const float* delta, const int* indexes, float* grad, size_t size);

/* ---- upsample: include/UpsampleLayer.h:97-121 ---- */
void pxo_upsample(const float* in, int w, int h, int c, int batch, int stride, int forward,
                  float scale, float* acc, float* out);

/* ---- shortcut: include/ShortcutLayer.h:84-141 ---- */
int pxo_shortcut(int batch, int w1, int h1, int c1, const float* add, int w2, int h2, int c2,
                 float out_scale, float add_scale, float* out);
void pxo_shortcut_forward(int act, int batch, int w, int h, int c, const float* input,
                          const float* from_output, float alpha, float beta, float* output,
                          float* pre_activation);
void pxo_shortcut_backward(int act, int batch, int w, int h, int c, float* delta,
                           const float* pre_activation, float* from_delta, float* grad /* may be NULL */,
                           float alpha, float beta);

/* ---- boxes: src/DarkBox.cpp:84-151 + OpenCV >= 4.5.4 Rect_<float>::operator& ---- */
float pxo_box_intersection(const float a[4], const float b[4]);
float pxo_box_union(const float a[4], const float b[4]);
float pxo_box_iou(const float a[4], const float b[4]);

/* ---- YOLO head: include/YoloLayer.h:164-239, 390-547, 562-599, 637-651, 730-767 ----
 * truths: [batch][max_truth][5] = x, y, w, h, class; truth_counts[batch].
 * stats[12]: 0 sum IoU, 1 recall@.5, 2 recall@.75, 3 sum class prob, 4 sum obj at positives,
 *            5 sum obj over all slots, 6 count, 7 class count, 8 box, 9 obj, 10 no-obj, 11 class cost
 * (slot meaning of the reference's stats vector, include/cuda/YoloLayer.h:133-146). */
typedef struct pxo_yolo_cfg {
    int batch, width, height, classes;
    int num_masks, num_anchors;
    const int* mask;      /* [num_masks] */
    const int* anchors;   /* [2*num_anchors], integer pixels */
    int net_width, net_height;
    float ignore_thresh, truth_thresh;
    float coord_scale, object_scale, noobject_scale, class_scale;
} pxo_yolo_cfg;

void pxo_yolo_decode(const pxo_yolo_cfg* cfg, const float* input, float* output);
void pxo_yolo_forward(const pxo_yolo_cfg* cfg, const float* input, const float* truths,
                      const int* truth_counts, int max_truth, float* output, float* delta,
                      float* cost, float* stats);
/* src/YoloTargetBuilder.cpp:21-62, one image */
int pxo_yolo_build_targets(const pxo_yolo_cfg* cfg, const float* truths, int count,
                           int* classes, int* anchors, float* boxes);
void pxo_axpy(size_t n, float alpha, const float* x, float* y);

/* ---- route (channel concat): include/RouteLayer.h:91-137.  Parity pinned by construction only:
 * a copy and an alpha = 1 saxpy per image; the reference holds no test for this layer. ---- */
void pxo_route_forward(const float* layer_output, float* route_output, int batch, int layer_outputs,
                       int route_outputs, int offset);
void pxo_route_backward(const float* route_delta, float* layer_delta, int batch, int layer_outputs,
                        int route_outputs, int offset);

/* ---- Adam: include/cuda/Adam.h:49-90 + src/Adam.cu:26-37.  apply_decay: 0 none, 1 the reference's L2 term
 * (folded into the update before the moments), 2 decoupled (no counterpart in the reference; pinned by the
 * fp64 AdamW recurrence and its closed form at t = 1). ---- */
void pxo_adam_update(size_t n, float* w, float* d, float* m, float* v, int batch, int t, float lr,
                     float beta1, float beta2, float eps, float decay, int apply_decay);

/* ---- detections of a decoded head: include/YoloLayer.h:601-698 (addDetects, yoloBox, scaledYoloBox).
 * image_width/height > 0 selects the letterbox-corrected integer pixel boxes, else the relative
 * DarkBox rectangle (left, top, w, h).  Records come in the reference's order: image, cell, mask,
 * class.  Returns the number found; at most `capacity` are written.  Parity unpinned by reference
 * tests (they need downloaded weights); pinned by hand-computed cases and brute force. */
typedef struct pxo_detection {
    float x, y, w, h;
    float prob;
    int batch;
    int class_index;
    unsigned order;      /* ((image*area + cell)*masks + mask)*classes + class */
} pxo_detection;
int pxo_yolo_detections(const pxo_yolo_cfg* cfg, const float* predictions, float threshold,
                        int image_width, int image_height, pxo_detection* out, int capacity);

/* ---- nms, src/Box.cpp:56-147: stable sort by probability (descending), near-identical boxes
 * (overlap ratio > 0.9) of different classes in one image keep the strongest, then greedy
 * suppression above `threshold` (>= 0) inside each (image, class) group over its first 1024
 * members.  `out` needs room for `count` records; returns the number kept, in sorted order.
 * Pinned by the reference's tests/src/box.cpp:25-101 and by brute-force restatements. */
int pxo_nms(const pxo_detection* detections, int count, float threshold, pxo_detection* out);

/* ---- SGD with momentum: include/ConvLayer.h:309-311.  Parity unpinned by reference tests (no
 * numeric test of update() exists); pinned by the closed form of one step and an fp64 recurrence. */
void pxo_sgd_update(size_t n, float* w, float* d, int batch, float lr, float momentum, float decay,
                    int apply_decay);

/* ---- gradient rescale + clip: include/Layer.h:385-397, 479-499.  cblas_snrm2's internal summation
 * is implementation defined; the norm is carried in double here (pxo_mag_array). */
float pxo_rescale_clip(float* x, size_t n, float threshold, float clip);

#ifdef __cplusplus
}
#endif
#endif
