/*
 * libaether_hip.so -- C ABI of the MI355X (gfx950) convolution hot path.
 *
 * The reference framework has no FFI: its boundary is the duck-typed layer
 * protocol that Model drives (CNN/models/CNN_model_cupy.py:153-193).  Each entry
 * point below replaces the array-library calls one reference method makes, and
 * cites that method.  The Python classes in aether/layers.py keep the reference
 * class API and call these through ctypes.
 *
 * Conventions
 *   - every function returns 0 on success or a negative AETH_E_* code;
 *     aeth_last_error() returns a thread-local message for the last failure.
 *     Nothing aborts the process.
 *   - every pointer is a DEVICE pointer obtained from aeth_malloc unless its
 *     name starts with host_.
 *   - tensors are dense, C-contiguous: activations NHWC [S,H,W,C], filters
 *     [fH,fW,C,D] (the reference's filter_weights layout), dense weights
 *     [n_in,n_out] row-major, all float32 unless the name says bf16 (uint16_t
 *     holding the upper 16 bits of a float32, rounded to nearest even).
 *   - element counts fit int32; byte counts are int64.  A convolution whose
 *     batch-sized tensors reach 2^31 bytes (up to the 2^31 elements, 8 GiB of
 *     float32) is run in several launches over runs of whole samples; results
 *     are the same bits as for the samples handed in separately (wgrad: the
 *     runs' sums are added in run order).
 *   - one process-wide context bound to one GPU with one stream; calls are
 *     asynchronous on that stream, aeth_sync() and the d2h copy are the sync
 *     points.  Not re-entrant: one caller thread at a time.
 *   - convolution geometry: Ho = (H + 2*pH - fH)/sH + 1, Wo likewise, the caller
 *     passes pH = pW = P where P = (fH-1)/2 for "same" and 0 for "valid"
 *     (CNN/models/CNN_classes_cupy.py:78-85).
 */
#ifndef AETHER_HIP_H
#define AETHER_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AETH_OK          0
#define AETH_E_INVALID  -1   /* bad shape / NULL pointer / unsupported argument */
#define AETH_E_HIP      -2   /* a HIP runtime call failed                       */
#define AETH_E_NOMEM    -3   /* device allocation failed                        */
#define AETH_E_STATE    -4   /* aeth_init not called, or called twice on different devices */

/* ---- lifetime -------------------------------------------------------------- */
int aeth_init(int device);
int aeth_shutdown(void);
const char* aeth_last_error(void);
/* "arch=gfx950;cus=256;clock_mhz=2400;mem_clock_mhz=...;hbm_bytes=...;lds_bytes=..." */
int aeth_device_info(char* host_buf, int n);

/* Kernel-choice overrides for tests and measurements; no counterpart in the reference.
 * Every dispatch decision follows from the problem's shape; a switch lets a test reach a
 * kernel with an input smaller than the shapes it is chosen for, or run a problem on a
 * second, independently scheduled kernel.  -1 restores "decide from the shape";
 * host_name == NULL resets every switch.  Names: gather_bm, gather_kc, gather_nloop,
 * gather_halo, gather_split, gather_sa, gather_direct_b, gather_clip, gather_merge, gather_border, gather_pairs,
 * gather_runs, gather_bkn, gather_wide, gather_res, narrow, dense_res, direct, wgrad_halo, wgrad_wide, wgrad_cw,
 * wgrad_br, wgrad_rounds, wgrad_swap, pair_bwd.  May be called before aeth_init.  The
 * same switches can be given once through the environment variable AETHER_TUNE
 * ("name=value,name=value"), read by aeth_init; the library reads no other variable. */
int aeth_debug_set(const char* host_name, int value);

/* ---- memory (replaces cp.zeros / cp.asarray / .get(), cupy array ownership) - */
int aeth_malloc(void** host_out_ptr, int64_t bytes);
int aeth_free(void* p);
int aeth_memcpy_h2d(void* dst, const void* host_src, int64_t bytes);
int aeth_memcpy_d2h(void* host_dst, const void* src, int64_t bytes);   /* synchronises */
/* A small device-to-host copy in two halves, for callers that want the bytes later (a training loop that reads
 * a step's loss while the next step already runs; no counterpart in the reference, whose arrays synchronise on
 * every read).  aeth_d2h_begin queues the copy of at most 256 KB into pinned memory of the library, behind
 * what is queued so far, and returns a ticket at once; aeth_d2h_end waits for THAT copy (not for work queued
 * after it) and hands over the first `bytes` bytes.  At most 8 copies may be pending; every ticket must be
 * ended (bytes = 0 drops it).  Not possible while recording. */
int aeth_d2h_begin(const void* src, int64_t bytes, int* host_out_ticket);
int aeth_d2h_end(int ticket, void* host_dst, int64_t bytes);
int aeth_memcpy_d2d(void* dst, const void* src, int64_t bytes);
int aeth_fill_f32(float* dst, float value, int64_t n);
int aeth_sync(void);

/* ---- timing on the library's own stream (used by the benchmark) ------------ */
int aeth_event_create(void** host_out_event);
int aeth_event_destroy(void* event);
int aeth_event_record(void* event);
int aeth_event_elapsed_ms(void* start, void* stop, float* host_out_ms);  /* synchronises on stop */

/* ---- convolution, fp32 in / fp32 accumulate on MFMA ----------------------------
 * fprop  : Conv_Layer.forward, CNN/models/CNN_classes_cupy.py:70-120
 *          (cp.pad :92, as_strided :101, einsum 'shwxyc,xycd->shwd' :115, bias :116)
 *          y[s,h,w,d] = bias[d] + sum_{x,y,c} xpad[s,h*sH+x,w*sW+y,c] * w[x,y,c,d]
 *          bias may be NULL.
 * dgrad  : Conv_Layer.backward, :136-153 (einsum 'shwd,xycd->shwxyc' :138 and the
 *          atomicAdd scatter kernel :4-35, :141-146, crop :149-153).  Writes every
 *          element of the UNPADDED dx [S,H,W,C]; positions no tap reaches get 0.
 * wgrad  : Conv_Layer.backward, :132 (dbiases = sum over s,h,w) and :134
 *          (einsum 'shwxyc,shwd->xycd').  dbias may be NULL.  Deterministic.
 */
int aeth_conv_fprop_f32(const float* x, const float* w, const float* bias, float* y,
                        int S, int H, int W, int C, int D,
                        int fH, int fW, int sH, int sW, int pH, int pW);
int aeth_conv_dgrad_f32(const float* dy, const float* w, float* dx,
                        int S, int H, int W, int C, int D,
                        int fH, int fW, int sH, int sW, int pH, int pW);
int aeth_conv_wgrad_f32(const float* x, const float* dy, float* dw, float* dbias,
                        int S, int H, int W, int C, int D,
                        int fH, int fW, int sH, int sW, int pH, int pW);

/* Conv_Layer.backward :122-153 in one call: the wgrad and the dgrad above, bit for bit.  The two
 * products do not depend on each other, and where neither fills the GPU (the layers of a small
 * network: unit stride, a few hundred workgroups each) they go out as ONE launch whose
 * workgroups are shared between them, and their split sums as one more; everywhere else the
 * call is the two calls above in a row.  dbias may be NULL. */
int aeth_conv_bwd_f32(const float* x, const float* dy, const float* w, float* dw, float* dbias, float* dx,
                      int S, int H, int W, int C, int D,
                      int fH, int fW, int sH, int sW, int pH, int pW);

/* aeth_conv_fprop_f32 for callers that cannot allocate (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same arguments, same kernels, bit-identical results; the packed filter and
 * the split-K partial tiles go to a fixed array of AETH_NOALLOC_SCRATCH_BYTES that each
 * GPU holds until the process ends, instead of the library's growing workspace, and the
 * call makes no hipMalloc / hipFree.  Shapes whose scratch does not fit fail with
 * AETH_E_INVALID (the message states both sizes).  Every call on a GPU shares that
 * GPU's array: calls that overlap on one GPU race (the library's single stream
 * serialises its own). */
#define AETH_NOALLOC_SCRATCH_BYTES (8 << 20)
int aeth_conv_fprop_f32_noalloc(const float* x, const float* w, const float* bias, float* y,
                                int S, int H, int W, int C, int D,
                                int fH, int fW, int sH, int sW, int pH, int pW);

/* ---- convolution, bf16 in / fp32 accumulate / fp32 out --------------------------
 * Same three contractions with x, w, dy given as bf16.  No reference counterpart
 * (the reference is fp32 only); the inputs are produced by aeth_cast_f32_to_bf16.
 */
int aeth_cast_f32_to_bf16(const float* src, uint16_t* dst, int64_t n);
int aeth_conv_fprop_bf16(const uint16_t* x, const uint16_t* w, const float* bias, float* y,
                         int S, int H, int W, int C, int D,
                         int fH, int fW, int sH, int sW, int pH, int pW);
int aeth_conv_dgrad_bf16(const uint16_t* dy, const uint16_t* w, float* dx,
                         int S, int H, int W, int C, int D,
                         int fH, int fW, int sH, int sW, int pH, int pW);
int aeth_conv_wgrad_bf16(const uint16_t* x, const uint16_t* dy, float* dw, float* dbias,
                         int S, int H, int W, int C, int D,
                         int fH, int fW, int sH, int sW, int pH, int pW);

/* ---- dense layer ------------------------------------------------------------------
 * fprop : Layer_Dense.forward, CNN_classes_cupy.py:328-331   y = x.w + bias
 * dgrad : Layer_Dense.backward :354                           dx = dy.w^T
 * wgrad : Layer_Dense.backward :334-335                       dw = x^T.dy, dbias = sum_rows dy
 * x [M,n_in], w [n_in,n_out], bias [n_out], y/dy [M,n_out].  bias/dbias may be NULL.
 * axpy and l1_grad implement the regulariser terms of :337-351
 * (y += alpha*x ;  dw += lambda * (w < 0 ? -1 : +1)).
 */
int aeth_dense_fprop_f32(const float* x, const float* w, const float* bias, float* y,
                         int M, int n_in, int n_out);
int aeth_dense_dgrad_f32(const float* dy, const float* w, float* dx,
                         int M, int n_in, int n_out);
int aeth_dense_wgrad_f32(const float* x, const float* dy, float* dw, float* dbias,
                         int M, int n_in, int n_out);
/* A dense layer together with the ReLU / Leaky_ReLU next to it (:406-428), for callers that
 * know the neighbour: the same values as the separate calls, fewer launches on small layers.
 * aeth_dense_fprop_act_f32 also writes act_y = y > 0 ? y : alpha * y (alpha = 0: ReLU), the
 * activation's output; where K is split over workgroups, the reduction of the split writes
 * both.  aeth_dense_bwd_f32 is Layer_Dense.backward :333-354 in one call (dw, dbias, dx;
 * regulariser terms stay with the caller) and, with act_in / act_dx not NULL, the backward
 * pass of the activation IN FRONT of the layer on the way: act_dx = act_in < 0 ? alpha * dx
 * : dx (act_in = that activation's input).  A layer of at most 16 outputs on at most 1024
 * rows goes out as one launch; a wider layer on a small batch shares one launch between its
 * weight gradient and its input gradient, as aeth_conv_bwd_f32 does. */
int aeth_dense_fprop_act_f32(const float* x, const float* w, const float* bias, float* y, float* act_y,
                             float alpha, int M, int n_in, int n_out);
int aeth_dense_bwd_f32(const float* x, const float* dy, const float* w, float* dw, float* dbias, float* dx,
                       const float* act_in /* may be NULL */, float* act_dx /* NULL with act_in */, float alpha,
                       int M, int n_in, int n_out);
int aeth_axpy_f32(float alpha, const float* x, float* y, int64_t n);
int aeth_l1_grad_f32(float lambda, const float* w, float* dw, int64_t n);
/* out[0] = sum |x| (mode 0) or sum x*x (mode 1): Loss.regularization_loss :593-609 */
int aeth_reduce_f32(const float* x, int64_t n, int mode, float* out);

/* ---- layers either side of the path (so activations stay on the GPU) -------------
 * rows = product of the leading axes, C = channels (last axis).
 * bn_fwd_train : Batch_Norm.forward training branch :467-476 (biased variance,
 *                running = momentum*running + (1-momentum)*batch).  Saves batch mean
 *                and 1/sqrt(var+eps) for the backward pass.
 * bn_fwd_infer : :478-480.       bn_bwd : Batch_Norm.backward :484-508.
 */
int aeth_bn_fwd_train_f32(const float* x, const float* gamma, const float* beta,
                          float* running_mean, float* running_var,
                          float* save_mean, float* save_invstd, float* y,
                          int rows, int C, float eps, float momentum);
int aeth_bn_fwd_infer_f32(const float* x, const float* gamma, const float* beta,
                          const float* running_mean, const float* running_var, float* y,
                          int rows, int C, float eps);
int aeth_bn_bwd_f32(const float* x, const float* dy, const float* gamma,
                    const float* save_mean, const float* save_invstd,
                    float* dx, float* dgamma, float* dbeta, int rows, int C);
/* ReLU (alpha = 0) :406-415 and Leaky_ReLU :417-428.
 * fwd: y = x > 0 ? x : alpha*x ;  bwd: dx = x < 0 ? alpha*dy : dy  (strict <). */
int aeth_relu_fwd_f32(const float* x, float* y, float alpha, int64_t n);
int aeth_relu_bwd_f32(const float* x, const float* dy, float* dx, float alpha, int64_t n);
/* Producers that also leave a bfloat16 copy of what they write, for a bf16 convolution that
 * reads it next (no counterpart in the reference, which is fp32 only): the copy costs 2
 * bytes per element inside the producing kernel instead of a cast pass of 6.
 * relu_fwd_twin = relu_fwd with y_bf16; bn_bwd_twin = bn_bwd with dx_bf16 (declared below,
 * same arguments otherwise).  The fused block entry points take the same kind of optional
 * last argument (pool_out_bf16, bn_dx_bf16; NULL = none). */
int aeth_relu_fwd_twin_f32(const float* x, float* y, uint16_t* y_bf16, float alpha, int64_t n);
int aeth_bn_bwd_twin_f32(const float* x, const float* dy, const float* gamma,
                         const float* save_mean, const float* save_invstd,
                         float* dx, uint16_t* dx_bf16, float* dgamma, float* dbeta, int rows, int C);
/* Pooling "max"/"valid" :212-273 and :275-300.  idx holds the flat window index
 * fh*fW+fw of the FIRST maximum in row-major window order. */
int aeth_maxpool_fwd_f32(const float* x, float* y, uint8_t* idx,
                         int S, int H, int W, int C, int fH, int fW, int sH, int sW);
int aeth_maxpool_bwd_f32(const float* dy, const uint8_t* idx, float* dx,
                         int S, int H, int W, int C, int fH, int fW, int sH, int sW);
/* One pass over a convolution block's Batch_Norm (training branch, as bn_fwd_train),
 * ReLU / Leaky_ReLU and 2x2 stride-2 "valid" max pooling: writes the three outputs
 * the layers would have written one after the other (:467-476, :406-428, :212-273)
 * and the pooling indices.  x is [S,H,W,C] with even H and W and C % 4 == 0, all
 * pointers 16-byte aligned; AETH_E_INVALID otherwise (callers then use the three
 * separate entry points).  maxpool2_relu_bwd is the backward pass of the pooling
 * and the activation of such a block (:275-300, :412-415): pool_dx = Pooling.dinputs,
 * relu_dx = ReLU.dinputs, relu_in = the activation's input (Batch_Norm's output). */
int aeth_bn_relu_maxpool2_fwd_f32(const float* x, const float* gamma, const float* beta,
                                  float* running_mean, float* running_var,
                                  float* save_mean, float* save_invstd,
                                  float* bn_out, float* relu_out, float* pool_out, uint8_t* idx,
                                  int S, int H, int W, int C, float eps, float momentum, float alpha);
int aeth_maxpool2_relu_bwd_f32(const float* dy, const uint8_t* idx, const float* relu_in,
                               float* pool_dx, float* relu_dx,
                               int S, int H, int W, int C, float alpha);
/* The same with Batch_Norm.backward (:484-508) behind it: the column sums of the
 * batch norm are taken while the activation's gradient is written.  x is the batch
 * norm's input, bn_dx its dinputs.  Additionally needs C / 4 to divide 256. */
int aeth_maxpool2_relu_bn_bwd_f32(const float* dy, const uint8_t* idx, const float* relu_in,
                                  const float* x, const float* gamma,
                                  const float* save_mean, const float* save_invstd,
                                  float* pool_dx, float* relu_dx, float* bn_dx,
                                  float* dgamma, float* dbeta,
                                  int S, int H, int W, int C, float alpha);
/* The two fused calls above with a bfloat16 copy (round to nearest even) of pool_out / bn_dx written beside the
 * float32 tensor, for a bf16 convolution that takes it as input / upstream gradient (as aeth_relu_fwd_twin_f32
 * and aeth_bn_bwd_twin_f32 do for the separate layers).  No counterpart in the reference. */
int aeth_bn_relu_maxpool2_fwd_twin_f32(const float* x, const float* gamma, const float* beta,
                                       float* running_mean, float* running_var,
                                       float* save_mean, float* save_invstd,
                                       float* bn_out, float* relu_out, float* pool_out, uint16_t* pool_out_bf16,
                                       uint8_t* idx,
                                       int S, int H, int W, int C, float eps, float momentum, float alpha);
int aeth_maxpool2_relu_bn_bwd_twin_f32(const float* dy, const uint8_t* idx, const float* relu_in,
                                       const float* x, const float* gamma,
                                       const float* save_mean, const float* save_invstd,
                                       float* pool_dx, float* relu_dx, float* bn_dx, uint16_t* bn_dx_bf16,
                                       float* dgamma, float* dbeta,
                                       int S, int H, int W, int C, float alpha);
/* Pooling "average" :267-268 and the scatter kernel :163-202. */
int aeth_avgpool_fwd_f32(const float* x, float* y,
                         int S, int H, int W, int C, int fH, int fW, int sH, int sW);
int aeth_avgpool_bwd_f32(const float* dy, float* dx,
                         int S, int H, int W, int C, int fH, int fW, int sH, int sW);
/* Dropout masks :375-377, :397-399: y[i] = x[i] * mask[i % mask_n]
 * (mask_n = n for Layer_Dropout, = C for Layer_Dropout_Spatial). */
int aeth_mul_mask_f32(const float* x, const float* mask, float* y, int64_t n, int64_t mask_n);
/* SoftMax.forward :542-547 and SoftMax.backward :549-560
 * (dx = (diag(p) - p p^T) dy per row = p * (dy - sum_j p_j dy_j)). */
int aeth_softmax_f32(const float* logits, float* probs, int rows, int K);
int aeth_softmax_bwd_f32(const float* probs, const float* dy, float* dx, int rows, int K);
/* Loss_CategoricalCrossEntropy.forward :615-632 on probabilities (clip to
 * [1e-7, 1-1e-7], label smoothing) -> per-sample loss; pred[i] = argmax_k probs[i][k]
 * (first maximum), which is what SoftMax.predictions :562-563 returns. */
int aeth_cce_fwd_f32(const float* probs, const int32_t* labels, float label_smoothing,
                     float* sample_loss, int32_t* pred, int rows, int K);
/* Activation_Softmax_Loss_CategoricalCrossEntropy.backward :666-680:
 * dlogits = (probs - smooth(onehot)) / rows. */
int aeth_softmax_cce_bwd_f32(const float* probs, const int32_t* labels, float label_smoothing,
                             float* dlogits, int rows, int K);
/* The classifier head of a training step in one launch: SoftMax.forward :542-547, the loss and predictions of
 * aeth_cce_fwd_f32 and the gradient of aeth_softmax_cce_bwd_f32, with their operations in their order (same bits). */
int aeth_softmax_cce_train_f32(const float* logits, const int32_t* labels, float label_smoothing, float* probs,
                               float* sample_loss, int32_t* pred, float* dlogits, int rows, int K);
/* The three calls above for a 2-D y_true that is not one-hot: soft or already smoothed targets, which the
 * reference multiplies in as given (:622-626, :672-676).  targets[rows][K] takes the place of the labels;
 * label smoothing is applied to it as to the one-hot rows, t (1 - ls) + ls / K (:626-628).  For one-hot rows
 * the results are bit-identical to the index forms. */
int aeth_cce_fwd_dense_f32(const float* probs, const float* targets, float label_smoothing,
                           float* sample_loss, int32_t* pred, int rows, int K);
int aeth_softmax_cce_bwd_dense_f32(const float* probs, const float* targets, float label_smoothing,
                                   float* dlogits, int rows, int K);
int aeth_softmax_cce_train_dense_f32(const float* logits, const float* targets, float label_smoothing, float* probs,
                                     float* sample_loss, int32_t* pred, float* dlogits, int rows, int K);
/* Optimizer_Adam.update_parameters for one tensor :702-734; t = iterations (0-based). */
int aeth_adam_f32(float* theta, const float* grad, float* m, float* v, int64_t n,
                  float lr, float beta1, float beta2, float eps, int t);
/* The same update for `count` (1..32) tensors in ONE launch: the loop over
 * trainable layers of Model.train (CNN_model_cupy.py:124-125) with each layer's
 * weights and biases as separate entries.  The five host_ arrays have `count`
 * entries; the pointers they hold are device pointers. */
int aeth_adam_multi_f32(int count, float* const* host_theta, const float* const* host_grad,
                        float* const* host_m, float* const* host_v, const int64_t* host_n,
                        float lr, float beta1, float beta2, float eps, int t);

/* Adam with the step state on the device, for recorded steps (below) that cannot take a
 * new step number from the host: state[4] doubles = {iterations, beta1^iterations,
 * beta2^iterations, learning rate of the current step}.  aeth_adam_state_step does
 * pre_update_parameters :693-697 and post_update_parameters :735-736 for one step
 * (learning-rate decay from the old iteration count, then iterations += 1 and the two
 * powers advance); aeth_adam_multi_dev_f32 is aeth_adam_multi_f32 reading lr and the bias
 * corrections 1 - beta^iterations from `state`. */
int aeth_adam_state_step(double* state, double lr, double decay, double beta1, double beta2);
int aeth_adam_multi_dev_f32(int count, float* const* host_theta, const float* const* host_grad,
                            float* const* host_m, float* const* host_v, const int64_t* host_n,
                            float beta1, float beta2, float eps, const double* state);

/* ---- recorded steps -------------------------------------------------------------------
 * No counterpart in the reference (CuPy launches every kernel from Python each step).
 * Between aeth_graph_begin and aeth_graph_end the library's stream records instead of
 * executing: every launch and device-to-device copy of the calls made in between
 * becomes a node of a HIP graph; nothing runs.  aeth_graph_launch replays the whole
 * sequence with one host call.  Blocks returned by aeth_malloc while recording stay
 * reserved for the graph until aeth_graph_destroy, also after aeth_free, because replays
 * write to them.  While recording, calls that wait for the device (aeth_sync, host
 * copies, a workspace that has to grow) fail with AETH_E_STATE: run the step once
 * normally first.  Arguments are frozen at recording time: feed new data by copying
 * into the buffers the recorded step reads. */
int aeth_graph_begin(void);
int aeth_graph_end(void** host_out_graph);
int aeth_graph_launch(void* graph);
int aeth_graph_destroy(void* graph);

#ifdef __cplusplus
}
#endif
#endif /* AETHER_HIP_H */
