/*
 * pixienn_hip.h -- C ABI of the MI355X (gfx950) non-convolution layer kernels.
 *
 * Drop-in boundary for PixieNN's kernel entry points (the free functions the
 * reference declares in its include/<Name>.cuh headers and calls from the layers
 * under include/cuda/).
 * Each function cites the reference interface it replaces as <file>:<lines>.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless its name starts with "host_";
 *     tensors are fp32, NCHW, contiguous: index = ((n*C + c)*H + y)*W + x;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *     no function synchronises the device, callers order work through the
 *     stream (the reference's cudaDeviceSynchronize() calls are not kept);
 *   - return value: PXH_OK (0); PXH_ERR_* (< 0) for a rejected call, nothing
 *     was launched; > 0 is the hipError_t of a failed launch.
 *     pxh_last_error() gives the message of the calling thread's last failure;
 *   - buffers are caller owned.  Aliasing is only allowed where a function
 *     says so ("in place").
 */
#ifndef PIXIENN_HIP_H
#define PIXIENN_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PXH_OK 0
#define PXH_ERR_INVALID_ARGUMENT (-1)
#define PXH_ERR_UNSUPPORTED (-2)
#define PXH_ERR_WORKSPACE (-3)

/* include/ActivationTypes.h:19-30 (same numbering) */
enum pxh_activation {
    PXH_LEAKY = 0, PXH_LINEAR, PXH_LOGGY, PXH_LOGISTIC, PXH_MISH,
    PXH_RELU, PXH_SOFTPLUS, PXH_SWISH, PXH_TANH
};

const char* pxh_last_error(void);
/* library version, bumped when a signature changes or a declaration leaves this header
 * (2: the test hooks moved to a private header; the tensor tables, the norm-from-the-writer entry
 * points, pxh_reserve_workspace and pxh_bn_train_act_forward_static were added) */
int pxh_abi_version(void);

/* Entry points that take `(workspace, workspace_bytes)` use a per-device buffer owned by the library
 * when given NULL.  That buffer grows when a call needs more than it holds, which allocates device
 * memory and is therefore refused (PXH_ERR_WORKSPACE) while the call's stream is being captured into a
 * graph.  pxh_reserve_workspace makes the current device's buffer hold at least `bytes` (the largest
 * *_workspace_bytes() of the calls to come) ahead of time -- it allocates, so it is a call for BEFORE a
 * capture, not inside one; when the buffer grows it at least doubles, and blocks handed out earlier stay
 * allocated, so addresses that queued work or captured graphs hold remain valid (what is left behind adds
 * up to less than the live block).  The buffer is shared by every
 * NULL-workspace call on the device: calls that may overlap (several streams or threads) must pass
 * workspaces of their own.  No counterpart in the reference (cuDNN and cuBLAS own their scratch). */
int pxh_reserve_workspace(size_t bytes);

/* ------------------------------------------------------------------------
 * Conv-layer epilogue, forward.
 * ---------------------------------------------------------------------- */

/* BN-inference + activation in one pass:
 *   y = act( ((x - rolling_mean[c]) / (sqrt(rolling_var[c]) + 1e-5)) * scale[c] + bias[c] )
 * with the rounding sequence of the CPU layer (subtract, divide, scale, add
 * each rounded to fp32).  pre_activation (nullable) receives the value before
 * act.  In place allowed (y == x).
 * Two launches: the per-channel constants are folded into `workspace`
 * (pxh_bn_folded_bytes(channels) bytes, or NULL for the library's per-device buffer), then the
 * tensor is streamed once.
 * Replaces, for an inferring ConvLayer/BatchNormLayer: cudnnBatchNormalizationForwardInference
 * + preActivation_.copy + activate(), include/cuda/ConvLayer.h:284-307; CPU semantics
 * src/BatchNorm.cpp:24-67 (training == false), include/ConvLayer.h:227-236. */
int pxh_bn_infer_act_forward(const float* x, float* y, float* pre_activation,
                             const float* rolling_mean, const float* rolling_var,
                             const float* scale, const float* bias,
                             int batch, int channels, int spatial, int activation,
                             void* workspace, size_t workspace_bytes, void* stream);

/* The same, split for a layer whose weights do not change between calls: fold once (after
 * loading or updating the weights), then every forward is the single streaming launch.
 * `folded` is a caller-owned, 16-byte aligned device buffer of pxh_bn_folded_bytes(channels).
 * No counterpart in the reference, whose cuDNN call re-derives the constants on every forward. */
size_t pxh_bn_folded_bytes(int channels);
int pxh_bn_fold(const float* rolling_mean, const float* rolling_var, const float* scale,
                const float* bias, int channels, void* folded, void* stream);
int pxh_bn_folded_act_forward(const float* x, float* y, float* pre_activation, const void* folded,
                              int batch, int channels, int spatial, int activation, void* stream);

/* bias + activation in one pass: y = act(x + bias[c]); pre_activation nullable; in place allowed.
 * Replaces addBiasGpu (include/BiasKernels.cuh:21) + preActivation_.copy + activate()
 * (include/Activation.cuh:26) for a ConvLayer without batch_normalize. */
int pxh_bias_act_forward(const float* x, float* y, float* pre_activation, const float* bias,
                         int batch, int channels, int spatial, int activation, void* stream);

/* Bytes of device workspace the BN training entry points need for this shape. */
size_t pxh_bn_workspace_bytes(int batch, int channels, int spatial);

/* BN-training forward + activation:
 *   mean[c], var[c] (population variance) over N*H*W; rolling = 0.99*rolling + 0.01*stat;
 *   x_hat = (x - mean)/(sqrt(var) + 1e-5); pre = x_hat*scale + bias; y = act(pre).
 * Outputs x_saved, x_norm, pre_activation are each nullable (not materialised when NULL);
 * y == x is allowed when x_saved is NULL or distinct from x.
 * workspace: pxh_bn_workspace_bytes() bytes, or NULL to use a per-device buffer the
 * library allocates on first use and keeps.
 * Replaces cudnnBatchNormalizationForwardTraining + the x_/preActivation_ copies + activate(),
 * include/cuda/ConvLayer.h:284-307, include/cuda/BatchNormLayer.h:59-92; CPU semantics
 * src/BatchNorm.cpp:47-66, src/CpuUtil.cpp:248-301. */
int pxh_bn_train_act_forward(const float* x, float* y, float* pre_activation, float* x_saved,
                             float* x_norm, float* mean, float* var, float* rolling_mean,
                             float* rolling_var, const float* scale, const float* bias,
                             int batch, int channels, int spatial, int activation,
                             void* workspace, size_t workspace_bytes, void* stream);

/* A convolution's epilogue with the ShortcutLayer that follows it in the same pass, for a shortcut with
 * a linear activation over tensors of one shape (every residual block of the shipped YOLOv3 graphs):
 *   y = alpha * act(pre) + beta * from      (two products and one sum, each rounded)
 * i.e. what pxh_shortcut_forward(in = the epilogue's result, from, out = y, alpha, beta, PXH_LINEAR) would
 * leave, without the epilogue's result ever reaching memory: the shortcut's pass (12 bytes per element)
 * becomes one more stream read by the epilogue (4).  Everything else -- statistics, rolling averages,
 * x_saved, x_norm, pre_activation (the CONVOLUTION's pre-activation) -- as in the call without the
 * shortcut.  `from` may be y itself (read before it is written, element by element) but no other output.
 * The layer's own output is not materialised: only for a layer whose output nothing but the shortcut
 * reads (a route or a second shortcut that names the convolution needs the two separate calls), and
 * the layer's backward must not need its output (pxh_bn_act_backward recomputes from x).  In the
 * backward pass the convolution's delta is alpha times the shortcut's.
 * Replaces include/cuda/ConvLayer.h:284-307 followed by include/cuda/ShortcutLayer.h:23-37. */
int pxh_bn_train_act_shortcut_forward(const float* x, float* y, float* pre_activation, float* x_saved,
                                      float* x_norm, float* mean, float* var, float* rolling_mean,
                                      float* rolling_var, const float* scale, const float* bias,
                                      const float* from, float alpha, float beta, int batch, int channels,
                                      int spatial, int activation, void* workspace, size_t workspace_bytes,
                                      void* stream);
/* The same for inference, on constants folded by pxh_bn_fold (pxh_bn_folded_act_forward + shortcut). */
int pxh_bn_folded_act_shortcut_forward(const float* x, float* y, float* pre_activation, const void* folded,
                                       const float* from, float alpha, float beta, int batch, int channels,
                                       int spatial, int activation, void* stream);

/* A convolution's inference epilogue with the MaxPoolLayer that follows it in the same pass, for the
 * 2 x 2 window at stride 2 over planes of even height and width (five of the six pools of YOLOv3-tiny):
 *   pooled[n][c][i][j] = max over the window of act(bn(x)), compared in the pool's own order
 * i.e. what pxh_bn_folded_act_forward followed by pxh_maxpool_forward (kernel 2, stride 2, padding 1)
 * leaves in the pool's output, to the bit, without the layer's output reaching memory and without the
 * indexes, which only a backward pass reads: 5 bytes per element of x instead of 8 + 6.
 *   y       nullable: the layer's own output, for a layer that something else reads as well (a route);
 *   pooled  batch x channels x height/2 x width/2.
 * PXH_ERR_UNSUPPORTED for an odd height or width, or for tensors off a 16-byte boundary: take the two calls.
 * Replaces include/cuda/ConvLayer.h:284-307 (inference) followed by include/cuda/MaxPoolLayer.h:23-37. */
int pxh_bn_folded_act_maxpool_forward(const float* x, float* y, float* pooled, const void* folded, int batch,
                                      int channels, int height, int width, int activation, void* stream);

/* pxh_bn_train_act_forward for callers that cannot allocate device memory and have no workspace
 * to pass (code under HIP graph capture, serving loops, harnesses that forbid hipMalloc): same
 * arguments without the workspace, same kernels, same results.  The partial sums and per-channel
 * constants go into a buffer of PXH_BN_STATIC_SCRATCH_BYTES built into the library's device code
 * (each GPU holds its copy until the process ends); the call allocates and frees nothing.  A shape
 * for which pxh_bn_workspace_bytes() exceeds that size is rejected with PXH_ERR_WORKSPACE before
 * anything is launched.  All calls on one GPU share the buffer: two that overlap in time (different
 * streams or threads) race; order them, or use the workspace form.  The first call on a device looks
 * up the buffer's address, make it outside a capture.
 * No counterpart in the reference (its cuDNN calls own their scratch). */
#define PXH_BN_STATIC_SCRATCH_BYTES ((size_t) 1 << 20)
int pxh_bn_train_act_forward_static(const float* x, float* y, float* pre_activation, float* x_saved,
                                    float* x_norm, float* mean, float* var, float* rolling_mean,
                                    float* rolling_var, const float* scale, const float* bias,
                                    int batch, int channels, int spatial, int activation, void* stream);

/* Per-channel batch statistics only (first half of the above). */
int pxh_bn_stats(const float* x, float* mean, float* var, int batch, int channels, int spatial,
                 void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------
 * Conv-layer epilogue, backward.
 * ---------------------------------------------------------------------- */

/* Activation gradient + BN backward:
 *   d' = delta * act'(pre);  bias_updates[c] += sum d';  scale_updates[c] += sum d' * x_hat;
 *   d'' = d' * scale[c];  mean_delta, var_delta as src/CpuUtil.cpp:303-327;
 *   delta <- d''/sqrt(var+1e-5) + var_delta*2*(x-mean)/(N*HW) + mean_delta/(N*HW)   (in place)
 * x is the saved conv output (x_saved of the forward).  pre_activation may be NULL: it is then
 * recomputed from x exactly as the forward computed it.  mean_delta / var_delta are outputs
 * (nullable).  workspace as for the forward.
 * Replaces gradient() + cudnnBatchNormalizationBackward, include/cuda/ConvLayer.h:315-338;
 * CPU semantics include/ConvLayer.h:244-252, src/BatchNorm.cpp:69-96. */
int pxh_bn_act_backward(float* delta, const float* x, const float* pre_activation,
                        const float* mean, const float* var, const float* scale, const float* bias,
                        float* scale_updates, float* bias_updates, float* mean_delta, float* var_delta,
                        int batch, int channels, int spatial, int activation,
                        void* workspace, size_t workspace_bytes, void* stream);

/* Activation gradient + bias backward for a ConvLayer without batch_normalize:
 *   delta *= act'(pre) (in place);  bias_updates[c] += sum over N*HW of delta.
 * Replaces gradient() (include/Activation.cuh:27) + backwardBiasGpu (include/BiasKernels.cuh:22). */
int pxh_bias_act_backward(float* delta, const float* pre_activation, float* bias_updates,
                          int batch, int channels, int spatial, int activation,
                          void* workspace, size_t workspace_bytes, void* stream);

/* Layer::backward's gradient rescale + clip (include/Layer.h:385-397: scaleTensor when the norm of
 * the delta is beyond `threshold`, then clipDelta at +-`clip`; either is off when its figure is <= 0)
 * and the ConvLayer::backward epilogue that follows it (include/ConvLayer.h:238-252) in one call:
 * the same results as pxh_rescale_clip(delta, ...) followed by pxh_bn_act_backward(delta, ...), but the
 * delta is not read once just for its norm -- the first pass of the backward carries the sum of
 * squares and the largest magnitude, the decision is taken on the device, and when nothing has to
 * change (the usual case with the shipped thresholds) the call costs what pxh_bn_act_backward
 * costs plus launches that leave at once.  *norm_out (nullable, device) receives the norm of the
 * delta as it came.  When the delta is rescaled and the clamp moves nothing (in the one-launch
 * backward: nothing in a channel), the sums are not formed again from the rounded factor * delta: they
 * are linear in the delta and are multiplied by the factor instead -- within rounding of the two-call
 * sequence, not bit-identical to it.  When nothing changes the results are those of
 * pxh_bn_act_backward to the bit.
 * workspace: pxh_bn_clipped_workspace_bytes(), or NULL for the library's. */
size_t pxh_bn_clipped_workspace_bytes(int batch, int channels, int spatial);
int pxh_bn_act_backward_clipped(float* delta, const float* x, const float* pre_activation,
                                const float* mean, const float* var, const float* scale, const float* bias,
                                float* scale_updates, float* bias_updates, float* mean_delta, float* var_delta,
                                int batch, int channels, int spatial, int activation,
                                float threshold, float clip, float* norm_out,
                                void* workspace, size_t workspace_bytes, void* stream);

/* The same in front of pxh_bias_act_backward (a ConvLayer without batch_normalize): delta is left
 * rescaled, clamped and multiplied by act'(pre), as the two calls leave it; with a linear activation
 * and nothing to change it is only read.  workspace: pxh_bn_clipped_workspace_bytes(). */
int pxh_bias_act_backward_clipped(float* delta, const float* pre_activation, float* bias_updates,
                                  int batch, int channels, int spatial, int activation,
                                  float threshold, float clip, float* norm_out,
                                  void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------
 * Stand-alone pieces with the reference's own signatures.
 * ---------------------------------------------------------------------- */

/* include/Activation.cuh:26-27 */
int pxh_activate(int activation, float* x, size_t n, void* stream);
int pxh_gradient(int activation, const float* x, size_t n, float* delta, void* stream);
/* include/BiasKernels.cuh:21-22 (bias_updates accumulates) */
int pxh_add_bias(float* output, const float* bias, int batch, int n, int size, void* stream);
int pxh_backward_bias(float* bias_updates, const float* delta, int batch, int n, int size,
                      void* workspace, size_t workspace_bytes, void* stream);
/* include/CudaUtils.cuh:27-31 */
int pxh_fill_f32(float* x, size_t n, float value, void* stream);
/* pxh_fill_f32 for many tensors in a few launches (x, n: HOST arrays of `count` device pointers and
 * element counts): the deltas of all layers, which Layer::forward clears one by one
 * (include/Layer.h:378-383), at the start of a pass. */
int pxh_fill_f32_multi(int count, float* const* x, const size_t* n, float value, void* stream);
int pxh_fill_i32(int* x, size_t n, int value, void* stream);
int pxh_constrain(int n, float alpha, float* x, void* stream);
int pxh_mul(int n, const float* x, float* y, void* stream);          /* y[i] = x[i]*y[i]; x == y allowed */
/* cublasSaxpy as used for "grad += delta", include/cuda/YoloLayer.h:163, cuda/ShortcutLayer.h:49 */
int pxh_axpy(size_t n, float alpha, const float* x, float* y, void* stream);

/* ------------------------------------------------------------------------
 * Route (channel concatenation).  CPU semantics include/RouteLayer.h:91-137 (cblas_scopy /
 * cblas_saxpy per image), device path include/cuda/RouteLayer.h:23-71 (one cudaMemcpy or
 * cublasSaxpy per image and source layer; here one launch per source layer).
 * Image b of the source layer (layer_outputs floats, packed) corresponds to
 * route + b*route_outputs + offset.  forward copies the layer's output into the route's output;
 * backward adds the route's delta slice into the layer's delta.  batch*route_outputs < 2^31.
 * ---------------------------------------------------------------------- */
int pxh_route_forward(const float* layer_output, float* route_output, int batch, int layer_outputs,
                      int route_outputs, int offset, void* stream);
int pxh_route_backward(const float* route_delta, float* layer_delta, int batch, int layer_outputs,
                       int route_outputs, int offset, void* stream);

/* ------------------------------------------------------------------------
 * Max-pool.  include/MaxPoolKernels.cuh:5-7, CPU semantics include/MaxPoolLayer.h:88-158.
 * ---------------------------------------------------------------------- */

/* Writes every element of out and indexes (no prior zero fill needed).  indexes hold the flat
 * NCHW input index of the first strict maximum in row-major window order, or -1. */
int pxh_maxpool_forward(const float* in, float* out, int* indexes, int batch, int channels,
                        int ih, int iw, int oh, int ow, int kernel, int stride, int padding,
                        void* stream);
/* grad[indexes[i]] += delta[i] in ascending i order for every input cell, i.e. bit-identical to
 * the sequential CPU loop also when windows overlap (stride < kernel).  No atomics. */
int pxh_maxpool_backward(const float* delta, const int* indexes, float* grad, int batch, int channels,
                         int ih, int iw, int oh, int ow, int kernel, int stride, int padding,
                         void* stream);
/* The reference's geometry-free signature (maxPoolBackwardGpu).  Float atomics: bit-exact only
 * when no two outputs share an index (stride >= kernel). */
int pxh_maxpool_backward_scatter(const float* delta, const int* indexes, float* grad, int size,
                                 void* stream);

/* ------------------------------------------------------------------------
 * Upsample.  include/UpsampleKernels.cuh:21-22, CPU semantics include/UpsampleLayer.h:97-121.
 * forward != 0: out[b,k,j,i] = scale * in[b,k,j/stride,i/stride]   (plain store, every element)
 * forward == 0: acc[in] += scale * out[...] for the stride^2 covered cells in raster order.
 * ---------------------------------------------------------------------- */
int pxh_upsample(const float* in, int w, int h, int c, int batch, int stride, int forward,
                 float scale, float* acc, float* out, void* stream);
/* The same with the large tensor (`out`) being a channel slice of a wider one: image n of it starts at
 * out + n * out_image_stride (elements, >= c*h*w*stride^2).  With `out` pointing at a channel offset
 * inside the buffer of the route layer that follows (include/RouteLayer.h:91-137), the upsampled
 * tensor lands directly in the concatenation and the route copy of this source is not needed;
 * backward reads the route's delta slice in place. */
int pxh_upsample_strided(const float* in, int w, int h, int c, int batch, int stride, int forward,
                         float scale, float* acc, float* out, long long out_image_stride,
                         void* stream);

/* ------------------------------------------------------------------------
 * Shortcut.  include/ShortcutKernel.cuh:21-22, CPU semantics include/ShortcutLayer.h:84-141.
 * ---------------------------------------------------------------------- */

/* The reference's index-mapped blend: out[oi] = s1*out[oi] + s2*add[ai]. */
int pxh_shortcut(int batch, int w1, int h1, int c1, const float* add, int w2, int h2, int c2,
                 float s1, float s2, float* out, void* stream);
/* Whole ShortcutLayer::forward in one pass (same-shape operands):
 *   pre = alpha*input + beta*from_output; output = act(pre); pre_activation nullable. */
int pxh_shortcut_forward(const float* input, const float* from_output, float* output,
                         float* pre_activation, size_t n, float alpha, float beta, int activation,
                         void* stream);
/* Whole ShortcutLayer::backward in one pass:
 *   delta *= act'(pre_activation) (in place; skipped for linear, pre_activation may then be NULL);
 *   from_delta = 1*from_delta + beta*delta;  grad += alpha*delta (grad nullable). */
int pxh_shortcut_backward(float* delta, const float* pre_activation, float* from_delta, float* grad,
                          size_t n, float alpha, float beta, int activation, void* stream);
/* The same for the call that is the FIRST in a backward pass to write both targets: they are
 * overwritten (from_delta = beta*delta', grad = alpha*delta') instead of accumulated into, which is
 * what accumulating into cleared tensors gives (up to the sign of a zero), so neither needs the
 * zero-fill of Layer::forward (include/Layer.h:378-383) and neither is read: 12 B per element
 * instead of 20 + 8.  In a residual block the shortcut is that call for the delta of the layer in
 * front of it and of its `from` layer (the only other reader of the latter comes earlier in the
 * network, so later in the backward pass).  No counterpart in the reference, which always clears
 * and accumulates; the caller vouches for the order. */
int pxh_shortcut_backward_first(float* delta, const float* pre_activation, float* from_delta,
                                float* grad, size_t n, float alpha, float beta, int activation,
                                void* stream);

/* ------------------------------------------------------------------------
 * YOLO head.  include/YoloKernels.cuh:7-17, CPU semantics include/YoloLayer.h:164-239, 390-547.
 * Layout: [batch][mask][5+classes][area]; entries 0..3 box, 4 objectness, 5.. classes.
 * truths: [batch][max_truth][5] = x, y, w, h, class id (as float); truth_counts[batch].
 * stats[12] (accumulated into, as the reference does): 0 sum IoU, 1 #IoU>.5, 2 #IoU>.75,
 *   3 sum class prob, 4 sum obj at positives, 5 sum obj over all slots, 6 count, 7 class count;
 *   8 box, 9 object, 10 no-object, 11 class sum of squared delta (overwritten).
 * ---------------------------------------------------------------------- */

/* yoloActivateGpu: logistic on entries 0, 1, 4.., copy of entries 2, 3.  In place allowed. */
int pxh_yolo_activate(const float* input, float* output, int batch, int masks, int classes,
                      int area, void* stream);

/* yoloLossGpu with its argument list: region pass over every slot, then the host-assigned
 * positive slots, then cost (sum of squared delta, ADDED to *cost) and loss components.
 * delta must be zero on entry, as in the reference. */
int pxh_yolo_loss(const float* output, float* delta, const float* truths, const int* truth_counts,
                  int max_truth, const int* assigned_classes, const int* assigned_anchors,
                  const float* assigned_boxes, const int* masks, const float* anchors,
                  float* stats, float* cost, int batch, int mask_count, int anchor_count,
                  int classes, int width, int height, int net_width, int net_height,
                  float ignore_thresh, float truth_thresh, float coord_scale, float object_scale,
                  float noobject_scale, float class_scale, void* workspace, size_t workspace_bytes,
                  void* stream);

/* All heads of a model in one pass.  The engine runs each YoloLayer where it sits in the graph
 * (include/Model.h:1740-1759, include/YoloLayer.h:164-239), but nothing reads a head's output delta,
 * cost or statistics before the backward pass: a host that defers its heads to the end of forward
 * hands them over together, and the small heads -- each of which alone is one long chain of dependent
 * steps on a mostly idle machine -- run under the class rows of the large one: two launches for all
 * heads.  Per head the results are those of pxh_yolo_forward_train on that head (output and delta to
 * the bit; the sums are added in another grouping).  Heads share the batch, the truths, the anchor
 * list, the class count and the network size, as the YoloLayers of one model do.
 * masks: host memory; stats[12] / cost[1]: device, nullable.  At most 4 heads per call.
 * workspace: pxh_yolo_heads_workspace_bytes(), or NULL for the library's. */
typedef struct pxh_yolo_head {
    const float* input;
    float* output;
    float* delta;
    const int* masks;
    int mask_count;
    int width, height;
    float ignore_thresh, truth_thresh, coord_scale, object_scale, noobject_scale, class_scale;
    float* stats;
    float* cost;
} pxh_yolo_head;
size_t pxh_yolo_heads_workspace_bytes(int count, const pxh_yolo_head* heads, int batch);
int pxh_yolo_forward_train_heads(int count, const pxh_yolo_head* heads, const float* truths,
                                 const int* truth_counts, int max_truth, const int* host_anchors,
                                 int anchor_count, int batch, int classes, int net_width, int net_height,
                                 void* workspace, size_t workspace_bytes, void* stream);

/* Detections of a decoded head without copying the head to the host: YoloLayer::addDetects
 * (include/YoloLayer.h:601-698) as a thresholded compaction on the device.  A slot passes when its
 * objectness is not below `threshold`; each of its classes with objectness * probability >=
 * threshold gives one record.  image_width/height > 0 selects scaledYoloBox (integer pixel box of
 * the letterboxed image, x/y = left/top), else yoloBox(...).rect() (relative left, top, w, h).
 * *count (device int, cleared by the call) receives the number found, which may exceed `capacity`;
 * only the first `capacity` places are written.  Records are in no particular order; `order` is the
 * position in the reference's emission order (image, cell, mask, class), sort by it to restore it.
 * No counterpart among the reference's device kernels: its CUDA path copies the head to the host. */
typedef struct pxh_detection {
    float x, y, w, h;
    float prob;
    int batch;
    int class_index;
    unsigned order;
} pxh_detection;
int pxh_yolo_detections(const float* predictions, int batch, const int* host_masks, int mask_count,
                        const int* host_anchors, int anchor_count, int classes, int width, int height,
                        int net_width, int net_height, int image_width, int image_height,
                        float threshold, pxh_detection* out, int capacity, int* count, void* stream);
/* The same without clearing *count: the records of this head go behind those already there, and
 * `order_base` is added to their `order` -- with the number of (slot, class) pairs of the heads
 * before it, the orders of a model's heads continue as in Model::detections (include/Model.h:
 * 1078-1088), which asks one YOLO layer after the other. */
int pxh_yolo_detections_append(const float* predictions, int batch, const int* host_masks,
                               int mask_count, const int* host_anchors, int anchor_count, int classes,
                               int width, int height, int net_width, int net_height, int image_width,
                               int image_height, float threshold, unsigned order_base,
                               pxh_detection* out, int capacity, int* count, void* stream);

/* nms (src/Box.cpp:56-147) on records that never leave the device.  The input sequence of the
 * reference is the records' `order` (unique; ties in probability keep it, as its stable sort does).
 * *count (device) says how many of records[capacity] are there (more than capacity = capacity).
 * Records must name images in [0, batch) and classes in [0, classes).  kept[capacity] receives the
 * survivors sorted by descending probability, *kept_count (device) their number.  threshold >= 0.
 * Steps: near-identical boxes (overlap ratio > 0.9) of different classes in one image keep the
 * strongest; then greedy suppression above `threshold` inside each (image, class) group over its
 * first 1024 members.  Workspace: pxh_nms_workspace_bytes(capacity), or NULL for the library's.
 * A capacity of at most 512 (an inference pass) runs as one launch and needs no workspace. */
size_t pxh_nms_workspace_bytes(int capacity);
int pxh_nms(const pxh_detection* records, const int* count, int capacity, int batch, int classes,
            float threshold, pxh_detection* kept, int* kept_count, void* workspace,
            size_t workspace_bytes, void* stream);

size_t pxh_yolo_workspace_bytes(int batch, int mask_count, int classes, int width, int height,
                                int max_truth);

/* Whole YoloLayer::forward of a loss-computing pass in one sweep over the head: decode, dense
 * delta (every element written, no prior fill), positives assigned on the device from the
 * truths with the CPU layer's rule (best anchor over all anchors, later truth overwrites),
 * cost = sum(delta^2) (written to *cost, not divided by batch) and stats[12] (overwritten).
 * host_masks[mask_count], host_anchors[2*anchor_count] are HOST int arrays (layer constants).  * A workspace serves one stream at a time: the one-launch form of the pass counts its workgroups in at
 * device counters kept per workspace address (zero whenever no launch is using them), so two calls that
 * may overlap -- two streams, two threads -- must pass workspaces of their own, and a launch that never
 * completes (a device fault, a destroyed stream) leaves its counters unusable for that address.
 * pxh_yolo_forward_train_heads uses no such counters. */
int pxh_yolo_forward_train(const float* input, float* output, float* delta, const float* truths,
                           const int* truth_counts, int max_truth, const int* host_masks,
                           const int* host_anchors, float* stats, float* cost, int batch,
                           int mask_count, int anchor_count, int classes, int width, int height,
                           int net_width, int net_height, float ignore_thresh, float truth_thresh,
                           float coord_scale, float object_scale, float noobject_scale,
                           float class_scale, void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------
 * SGD with momentum.  The three BLAS calls of ConvLayer::update for one parameter tensor
 * (include/ConvLayer.h:309-321, include/cuda/ConvLayer.h:388-413) in one pass:
 *   if apply_decay d += (-decay*batch)*w;  w += (lr/batch)*d;  d *= momentum.
 * The reference applies the decay to the weights only, not to biases and scales.
 * ---------------------------------------------------------------------- */
int pxh_sgd_update(size_t n, float* w, float* d, int batch, float lr, float momentum, float decay,
                   int apply_decay, void* stream);

/* ... and for every parameter tensor of a model at once, as pxh_adam_update_multi does for Adam
 * (SGD is the optimiser of every shipped preset). */
int pxh_sgd_update_multi(int count, float* const* w, float* const* d, const size_t* n,
                         const int* apply_decay, int batch, float lr, float momentum, float decay,
                         void* stream);

/* ------------------------------------------------------------------------
 * Gradient rescale and clip, the two helpers Layer::backward runs on delta before a layer's own
 * backward (include/Layer.h:385-397, 479-499; include/cuda/Layer.h:24-39: cublasSnrm2 +
 * cublasSscal, then constrainGpu) without the host round trip of the norm:
 *   norm = |x|_2;  if (threshold > 0 && norm > 0 && norm > threshold) x *= threshold/norm;
 *   if (clip > 0) x = clamp(x, -clip, clip).
 * norm_out (nullable, device) receives the norm before rescaling.  When nothing has to change,
 * the tensor is read once and not written.  workspace: pxh_rescale_workspace_bytes() bytes or
 * NULL for the library's per-device buffer.
 * ---------------------------------------------------------------------- */
size_t pxh_rescale_workspace_bytes(void);
int pxh_rescale_clip(float* x, size_t n, float threshold, float clip, float* norm_out,
                     void* workspace, size_t workspace_bytes, void* stream);

/* The same for many tensors in a few launches: Layer::update's hooks pass every update buffer of
 * every layer through these helpers (include/Layer.h:400-411, ConvLayer.h:323-340: weights, biases,
 * scales), each with its own norm.  x and n are HOST arrays of `count` device pointers / element
 * counts; norms, if not NULL, is a DEVICE array of `count` floats that receives each tensor's norm
 * (an empty tensor's entry is left alone).  Every tensor ends up exactly as pxh_rescale_clip leaves
 * it.  Workspace: pxh_rescale_multi_workspace_bytes(), or NULL for the library's. */
size_t pxh_rescale_multi_workspace_bytes(void);
int pxh_rescale_clip_multi(int count, float* const* x, const size_t* n, float threshold, float clip,
                           float* norms, void* workspace, size_t workspace_bytes, void* stream);

/* Norm and largest magnitude from the kernel that writes the delta.  Layer::backward opens with the
 * two helpers above on the layer's own delta (include/Layer.h:385-397), which costs a read of the
 * tensor just for the norm.  Where one of this library's kernels is the LAST to write that delta
 * before its layer's backward -- the convolution in front of a shortcut receives its whole delta
 * from the shortcut's backward (include/ShortcutLayer.h:98-111), the layer in front of a YOLO head
 * from the head's `grad += delta` (include/YoloLayer.h:741-750) -- that kernel can leave behind, per
 * group of 256 values, the sum of squares and the largest magnitude of what it wrote (8 bytes per
 * KiB of tensor), and pxh_rescale_clip_from_groups starts from those instead of reading the tensor.
 * The sums are added in the order pxh_rescale_clip itself adds them: norm, verdict and rewritten
 * tensor are the same to the bit.
 *   groups: device buffer of pxh_norm_groups_bytes(n) bytes, 8-byte aligned, owned by the caller;
 *           it describes the tensor only until the tensor is written again.
 * A tensor that is not 16-byte aligned, or whose length is not a multiple of 4, has no group sums:
 * the producers then leave the buffer alone and pxh_rescale_clip_from_groups reads the tensor, so the
 * pair can be used without looking at the pointer.
 *   pxh_norm_groups               the group sums of a tensor as it is (one read)
 *   pxh_axpy_norm                 pxh_axpy, + the group sums of y
 *   pxh_shortcut_backward_norm    pxh_shortcut_backward (first == 0) or pxh_shortcut_backward_first
 *                                 (first != 0), + the group sums of grad, which is required */
size_t pxh_norm_groups_bytes(size_t n);
int pxh_norm_groups(const float* x, size_t n, void* groups, void* stream);
int pxh_axpy_norm(size_t n, float alpha, const float* x, float* y, void* y_groups, void* stream);
int pxh_shortcut_backward_norm(float* delta, const float* pre_activation, float* from_delta,
                               float* grad, size_t n, float alpha, float beta, int activation,
                               int first, void* grad_groups, void* stream);
int pxh_rescale_clip_from_groups(float* x, size_t n, float threshold, float clip, float* norm_out,
                                 const void* groups, void* workspace, size_t workspace_bytes,
                                 void* stream);

/* A ShortcutLayer's whole backward: Layer::backward's rescale + clip of its delta (include/Layer.h:385-397,
 * 474-499), then the shortcut's own backward (include/ShortcutLayer.h:98-111) --
 *   pxh_rescale_clip(delta, n, threshold, clip, norm_out, ...), then
 *   first ? pxh_shortcut_backward_first(delta, ...) : pxh_shortcut_backward(delta, ...)
 * with the values of that sequence to the bit.  For a first writer (first != 0) with a linear activation
 * over 16-byte aligned tensors of a multiple of four values -- every shortcut of the shipped YOLOv3 graph
 * once its targets are known to be written here first -- the two run as two launches that read the
 * delta once when nothing has to change (the common case: the pass that adds up the norm writes both
 * targets as well, the second launch forms the verdict and leaves; otherwise it rewrites the delta and
 * both targets from it): 8 or 12 bytes per element where the sequence moves 12 or 16.  Every other case
 * runs the sequence itself.  delta must not alias from_delta or grad; grad is nullable.
 * workspace: pxh_rescale_workspace_bytes() bytes or NULL. */
int pxh_shortcut_backward_clipped(float* delta, const float* pre_activation, float* from_delta,
                                  float* grad, size_t n, float alpha, float beta, int activation,
                                  int first, float threshold, float clip, float* norm_out,
                                  void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------
 * Adam.  include/Adam.cuh:21, include/cuda/Adam.h:49-90.
 * ---------------------------------------------------------------------- */

/* adamGpu: x += rate * (m/(1-b1^t)) / (sqrt(v/(1-b2^t)) + eps) */
int pxh_adam(int n, float* x, const float* m, const float* v, float beta1, float beta2, float rate,
             float eps, int t, void* stream);
/* Whole Adam<CUDA>::update in one pass, same per-element operation order:
 *   d *= 1/batch; if apply_decay d += -decay*w; m = b1*m + (1-b1)*d; v = b2*v + (1-b2)*d*d;
 *   w += lr * (m/(1-b1^t)) / (sqrt(v/(1-b2^t)) + eps);  d = 0.
 * (apply_decay == 1: L2 decay folded into the update before the moments, as the reference does.)
 * apply_decay == 2 is the decoupled form, which the reference does not have: the moments are formed from
 * the plain update and the weight also shrinks by lr * decay of its old value,
 *   w = (w + lr * (m/(1-b1^t)) / (sqrt(v/(1-b2^t)) + eps)) + (-(lr * decay)) * w,
 * each operation rounded to fp32.  Other values of apply_decay are rejected.  The many-tensor forms
 * below take the reference's form only. */
int pxh_adam_update(size_t n, float* w, float* d, float* m, float* v, int batch, int t, float lr,
                    float beta1, float beta2, float eps, float decay, int apply_decay, void* stream);

/* The same for every parameter tensor of a model in as few launches as possible (the engine updates
 * its layers one by one, cuda/ConvLayer.h:370-386: three tensors per convolution, most of them a few
 * hundred values).  w, d, m, v and n are HOST arrays of `count` device pointers / element counts;
 * apply_decay is a host array of flags (weights: 1, biases and scales: 0) or NULL for none.  Each
 * element gets exactly what pxh_adam_update gives it.  Tensors of length 0 are skipped. */
int pxh_adam_update_multi(int count, float* const* w, float* const* d, float* const* m,
                          float* const* v, const size_t* n, const int* apply_decay, int batch, int t,
                          float lr, float beta1, float beta2, float eps, float decay, void* stream);

/* ------------------------------------------------------------------------
 * The many-tensor operations over a table kept in device memory: ONE launch for all parameter
 * tensors of a model (two for rescale + clip), where the host-array forms above take one launch per
 * 32 tensors.  A model builds its tables once, after its layers exist (the engine's counterpart
 * would be Model::update, include/Model.h:1772-1792, gathering what ConvLayer::update,
 * include/cuda/ConvLayer.h:370-413, and Layer::update, include/Layer.h:400-411, step one by one).
 *
 * pxh_tensor_table_create: `buffers` is a HOST array of streams * count device pointers, stream after
 * stream (buffers[k * count + i] = buffer k of tensor i); streams = 1 (fill, rescale + clip: x),
 * 2 (SGD: w, d) or 4 (Adam: w, d, m, v); n[count] element counts; apply_decay[count] flags or NULL.
 * Tensors of length 0 are left out; at most 2048 tensors.  Allocates device memory and uploads the
 * table with a blocking copy: call it at set-up, not under graph capture.  The table belongs to the
 * device that was current; destroy it with pxh_tensor_table_destroy.  A table with more buffers per
 * tensor than an operation needs serves it too (an Adam table can be filled or rescaled: buffer 0).
 * Every tensor ends up exactly as the single-tensor call leaves it.  pxh_rescale_clip_table keeps
 * its partial sums inside the table, so two calls on one table must not overlap in time; `norms`
 * (nullable, device) receives one norm per tensor of the table, in table order.
 * No counterpart in the reference.
 * ---------------------------------------------------------------------- */
typedef struct pxh_tensor_table pxh_tensor_table;
int pxh_tensor_table_create(int count, int streams, float* const* buffers, const size_t* n,
                            const int* apply_decay, pxh_tensor_table** table);
void pxh_tensor_table_destroy(pxh_tensor_table* table);
/* tensors in the table (those of length 0 are not counted) */
int pxh_tensor_table_count(const pxh_tensor_table* table);
int pxh_adam_update_table(const pxh_tensor_table* table, int batch, int t, float lr, float beta1,
                          float beta2, float eps, float decay, void* stream);
int pxh_sgd_update_table(const pxh_tensor_table* table, int batch, float lr, float momentum, float decay,
                         void* stream);
int pxh_fill_f32_table(const pxh_tensor_table* table, float value, void* stream);
int pxh_rescale_clip_table(const pxh_tensor_table* table, float threshold, float clip, float* norms,
                           void* stream);

#ifdef __cplusplus
}
#endif
#endif
