/*
 * C ABI of libpytorch_loss_hip.so: the fused "V3" loss kernels of pytorch-loss,
 * written for AMD MI355X (gfx950).  This is the boundary that replaces the
 * reference's four pybind11 extension modules (lsr_cpp, focal_cpp,
 * large_margin_cpp, lovasz_softmax_cpp).
 *
 * Conventions for every entry point
 *   - plain device pointers, sizes and scalars; no framework types;
 *   - logits (and the logits gradient) are fp32, fp16 or bf16 as named by `dtype`
 *     (PLH_DTYPE_*), laid out (n_size, dimsize, m_size) row-major, i.e. NCHW
 *     with the spatial dims flattened into m_size (the reference flattens the
 *     same way, csrc/lsr_kernel.cu:199-202); integer labels are int64 (n_size, m_size);
 *   - `stream` is a hipStream_t (NULL = the default stream); launches are
 *     asynchronous and the library never synchronises, allocates or frees
 *     device memory, reads no environment variable and keeps no state between calls
 *     (re-entrant; the one exception, plh_lsr_forward_reduced_static, says so);
 *   - the caller sets the current device to the one that owns the pointers;
 *   - return value: PLH_OK (0), a negative PLH_ERR_* for rejected arguments
 *     (nothing was launched), or a positive hipError_t from the launch;
 *   - sizes of 0 elements return PLH_OK without launching
 *     (csrc/lsr_kernel.cu:207-210 does the same).
 *
 * Upstream gradients: the reference returns dloss/dlogits and lets Python do
 * `grad.mul_(grad_output...)` in a second pass over the tensor
 * (pytorch_loss/label_smooth.py:143-144).  Here the multiply is fused:
 *   grad_output == NULL          -> unit upstream gradient (the reference's raw result)
 *   grad_output_stride == 0      -> one fp32 scalar in device memory, broadcast
 *   grad_output_stride == 1      -> one fp32 value per loss element, contiguous
 */
#ifndef PYTORCH_LOSS_HIP_H
#define PYTORCH_LOSS_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PLH_ABI_VERSION 5

#define PLH_OK 0
#define PLH_ERR_NULL_POINTER (-1)   /* a required pointer is NULL */
#define PLH_ERR_BAD_SIZE (-2)       /* negative size, or numel beyond the supported range */
#define PLH_ERR_BAD_STRIDE (-3)     /* grad_output_stride not 0 or 1 */
#define PLH_ERR_TOO_MANY_CLASSES (-4) /* Lovasz: dimsize >= 512 (csrc/lovasz_softmax.cu:665) */
#define PLH_ERR_WORKSPACE (-5)      /* workspace missing, misaligned or smaller than plh_*_workspace_bytes() */
#define PLH_ERR_MISALIGNED (-6)     /* a pointer is not aligned to its element size */
#define PLH_ERR_BAD_DTYPE (-7)      /* dtype is not one of PLH_DTYPE_* */

/* Element type of the logits and of the logits gradient (`dtype` argument; both tensors of one call
 * share it). Arithmetic is fp32 whatever the storage type; losses, upstream gradients and the Lovasz
 * jacc tensor are always fp32. The reference dispatches the same three floating types
 * (AT_DISPATCH_FLOATING_TYPES_AND_HALF, e.g. csrc/lsr_kernel.cu:215) but computes in the storage
 * type; computing in fp32 is what its autocast wrapper asks for (custom_fwd(cast_inputs=float32)). */
#define PLH_DTYPE_F32 0
#define PLH_DTYPE_F16 1
#define PLH_DTYPE_BF16 2

int plh_abi_version(void);

/* Text for any value an entry point can return (PLH_ERR_* or hipError_t). */
const char *plh_error_string(int code);

/* ---- label-smoothed softmax cross entropy -----------------------------------
 * Replaces lsr_cpp.lsr_forward / lsr_cpp.lsr_backward
 * (csrc/lsr_kernel.cu:296-305, 307-317; kernels :65-185; host :191-293).
 * losses: (n_size, m_size) fp32, 0 at ignored pixels.
 * grad_logits: shape of logits, 0 at ignored pixels.
 */
int plh_lsr_forward(const void *logits, int32_t dtype, const int64_t *labels, float *losses,
                    int64_t n_size, int64_t dimsize, int64_t m_size,
                    int64_t ignore_index, float smooth, void *stream);

int plh_lsr_backward(const void *logits, int32_t dtype, const int64_t *labels,
                     const float *grad_output, int64_t grad_output_stride,
                     void *grad_logits,
                     int64_t n_size, int64_t dimsize, int64_t m_size,
                     int64_t ignore_index, float smooth, void *stream);

/* Module-level reduction fused into the forward (no counterpart in the reference's
 * extension, which leaves `losses.sum()` and `(labels != ignore).sum()` to ATen,
 * pytorch_loss/label_smooth.py:165-170).  The forward kernel leaves per-block partial
 * sums/counts in `workspace`; a one-block kernel adds them in a fixed order.
 *   losses      per-pixel losses, or NULL to skip writing them
 *   loss_out    1 fp32: the sum (mean == 0) or sum / n_valid (mean != 0; 0/0 = NaN)
 *   n_valid_out 1 int64: number of non-ignored pixels, or NULL
 *   workspace   at least plh_reduce_workspace_bytes(n_size*m_size) bytes, 16-byte aligned
 * plh_lsr_backward_scaled is the matching backward: the upstream gradient is the scalar
 * grad_scalar[0] * scale / divide_by[0] (divide_by NULL = 1), all read on the device.
 */
int64_t plh_reduce_workspace_bytes(int64_t units);

int plh_lsr_forward_reduced(const void *logits, int32_t dtype, const int64_t *labels, float *losses,
                            float *loss_out, int64_t *n_valid_out, int32_t mean,
                            void *workspace, int64_t workspace_bytes,
                            int64_t n_size, int64_t dimsize, int64_t m_size,
                            int64_t ignore_index, float smooth, void *stream);

int plh_lsr_backward_scaled(const void *logits, int32_t dtype, const int64_t *labels,
                            const float *grad_scalar, float scale, const int64_t *divide_by,
                            void *grad_logits,
                            int64_t n_size, int64_t dimsize, int64_t m_size,
                            int64_t ignore_index, float smooth, void *stream);

/* Loss ('mean' / 'sum') and its gradient under an upstream gradient of 1 from ONE pass over the logits, as
 * plh_lmargin_forward_backward_reduced does for the large-margin loss (no counterpart in the reference, whose LSR
 * module has no forward+backward Function; label_smooth.py:150-172 of the repository root runs lsr_forward, then
 * lsr_backward). The labels are counted first (n_valid_out: required), the pass writes grad_logits already divided by
 * the count (mean); plh_scale_unless_one is the backward. Up to 32 channels; beyond, and for (N, C) rows of more than
 * 32 classes, the entry point runs the forward and the backward kernels one after the other (same outputs). */
int plh_lsr_forward_backward_reduced(const void *logits, int32_t dtype, const int64_t *labels,
                                     float *loss_out, int64_t *n_valid_out, void *grad_logits, int32_t mean,
                                     void *workspace, int64_t workspace_bytes,
                                     int64_t n_size, int64_t dimsize, int64_t m_size,
                                     int64_t ignore_index, float smooth, void *stream);

/* The module step on channel planes that do not start on 128-byte lines (513 x 513, 769 x 769 crops; no counterpart in the reference, whose
 * backward recomputes the softmax, csrc/lsr_kernel.cu:139-225). plh_lsr_saves_lse says (1 / 0) whether it applies to
 * these sizes: fp32 logits and channel planes of at least 4096 pixels, with either a plane byte length that is no
 * multiple of 128 and dimsize up to 24 or from 33 (25..32 keep their kernels), or dimsize above 256 on any plane;
 * and (N, C) rows (m_size 1) of more than 32 classes, where the backward becomes elementwise over the flattened tensor
 * (bf16 (8192,32000): forward + backward 0.357 -> 0.275 ms), wherever that is the faster one: fp32 rows except those of a
 * multiple of 32 classes from 96 to 768 and those of 2049..4096 classes; 16-bit rows of more than 1024 classes, and of a
 * multiple of 8 classes up to 96.
 * Then plh_lsr_forward_reduced_lse is plh_lsr_forward_reduced that also leaves every pixel's
 * log-sum-exp in lse_out (n_size*m_size floats; it writes no per-pixel losses), and plh_lsr_backward_scaled_lse is
 * plh_lsr_backward_scaled that forms the gradient from it, sumw*exp(x - lse) - w, plane by plane in each plane's own
 * cache lines (`kept`: optional byte mask as in plh_lsr_backward_kept, else NULL). The gradient equals the
 * recomputing kernels' to rounding (relative 1e-6; 1e-5 beyond 512 channels, whose sums are longer). When logits and grad_logits do not sit at the same offset into a
 * 128-byte line the recomputing kernel runs and `lse` is not read. PLH_ERR_BAD_SIZE for sizes that
 * plh_lsr_saves_lse answers with 0. */
int plh_lsr_saves_lse(int32_t dtype, int64_t n_size, int64_t dimsize, int64_t m_size);

int plh_lsr_forward_reduced_lse(const void *logits, int32_t dtype, const int64_t *labels, float *lse_out,
                                float *loss_out, int64_t *n_valid_out, int32_t mean,
                                void *workspace, int64_t workspace_bytes,
                                int64_t n_size, int64_t dimsize, int64_t m_size,
                                int64_t ignore_index, float smooth, void *stream);

int plh_lsr_backward_scaled_lse(const void *logits, int32_t dtype, const int64_t *labels, const float *lse,
                                const uint8_t *kept, const float *grad_scalar, float scale, const int64_t *divide_by,
                                void *grad_logits,
                                int64_t n_size, int64_t dimsize, int64_t m_size,
                                int64_t ignore_index, float smooth, void *stream);

/* plh_lsr_forward_reduced for callers that cannot allocate device memory or bring a workspace
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc). It has no
 * counterpart in the reference. Same arguments and results as plh_lsr_forward_reduced, without the
 * workspace: the per-block partials live in a 2 MiB device array that is part of the library's
 * code object (each GPU that the library runs on holds its own copy until the process ends); its
 * address is looked up on the first call on each device (hipGetSymbolAddress, under a mutex: make that
 * first call outside a stream capture). The call allocates and frees nothing.
 * Limit: n_size * m_size <= 2^24 pixels, else PLH_ERR_BAD_SIZE. All calls on one GPU share the one
 * array: calls that overlap on one GPU (different streams or threads) race; calls on one stream
 * are ordered and need no clearing in between.
 */
int plh_lsr_forward_reduced_static(const void *logits, int32_t dtype, const int64_t *labels, float *losses,
                                   float *loss_out, int64_t *n_valid_out, int32_t mean,
                                   int64_t n_size, int64_t dimsize, int64_t m_size,
                                   int64_t ignore_index, float smooth, void *stream);

/* ---- sigmoid focal loss -------------------------------------------------------
 * Replaces focal_cpp.focalloss_forward / focalloss_backward /
 * focalloss_forward_backward (csrc/focal_kernel.cu:301-335; kernels :29-164).
 * labels have the logits' shape and element type (soft labels allowed).  Argument order
 * (gamma, alpha) follows the reference's C++ side (csrc/focal_kernel.cu:301-303).
 */
int plh_focal_forward(const void *logits, int32_t dtype, const void *labels, float *losses,
                      int64_t numel, float gamma, float alpha, void *stream);

int plh_focal_backward(const void *logits, int32_t dtype, const void *labels,
                       const float *grad_output, int64_t grad_output_stride,
                       void *grad_logits,
                       int64_t numel, float gamma, float alpha, void *stream);

/* Reduction fused into the forward, as for LSR (replaces `loss.mean()` / `loss.sum()` of
 * focal_loss.py:196-199): loss_out = sum, or sum / numel when mean != 0; workspace of
 * plh_reduce_workspace_bytes(numel) bytes. The matching backward takes the upstream
 * gradient grad_scalar[0] * scale (scale = 1/numel for a mean). */
int plh_focal_forward_reduced(const void *logits, int32_t dtype, const void *labels, float *losses,
                              float *loss_out, int32_t mean, void *workspace, int64_t workspace_bytes,
                              int64_t numel, float gamma, float alpha, void *stream);

int plh_focal_backward_scaled(const void *logits, int32_t dtype, const void *labels,
                              const float *grad_scalar, float scale, void *grad_logits,
                              int64_t numel, float gamma, float alpha, void *stream);

/* One pass producing both the losses and dloss/dlogits under a unit upstream gradient. */
int plh_focal_forward_backward(const void *logits, int32_t dtype, const void *labels,
                               float *losses, void *grad_logits,
                               int64_t numel, float gamma, float alpha, void *stream);

/* The module step of the repository root's FocalLossV3 (focal_loss.py:196-200: FocalSigmoidLossFuncV3FB.apply, then
 * loss.mean() / loss.sum()) in ONE pass: the kernel leaves the partial sums of the losses and writes grad_logits
 * already divided by numel (mean) - the gradient under an upstream gradient of 1; plh_scale_unless_one is its backward.
 * loss_out: the sum or the mean. Workspace as for plh_focal_forward_reduced. */
int plh_focal_forward_backward_reduced(const void *logits, int32_t dtype, const void *labels, float *loss_out,
                                       void *grad_logits, int32_t mean, void *workspace, int64_t workspace_bytes,
                                       int64_t numel, float gamma, float alpha, void *stream);

/* ---- large-margin softmax -------------------------------------------------------
 * Replaces large_margin_cpp.l_margin_forward / l_margin_backward /
 * l_margin_forward_backward (csrc/large_margin_kernel.cu:796-831; kernels :140-599).
 * valid_cnt (forward_backward only): one int64 that receives the number of
 * non-ignored pixels; the call overwrites it (no need to clear it first).
 */
int plh_lmargin_forward(const void *logits, int32_t dtype, const int64_t *labels, float *losses,
                        int64_t n_size, int64_t dimsize, int64_t m_size,
                        int64_t ignore_index, float lam, void *stream);

int plh_lmargin_backward(const void *logits, int32_t dtype, const int64_t *labels,
                         const float *grad_output, int64_t grad_output_stride,
                         void *grad_logits,
                         int64_t n_size, int64_t dimsize, int64_t m_size,
                         int64_t ignore_index, float lam, void *stream);

/* Reduction fused into the forward and the matching backward, as for LSR
 * (replaces large_margin_softmax.py:169-173 of the packaged copy). */
int plh_lmargin_forward_reduced(const void *logits, int32_t dtype, const int64_t *labels, float *losses,
                                float *loss_out, int64_t *n_valid_out, int32_t mean,
                                void *workspace, int64_t workspace_bytes,
                                int64_t n_size, int64_t dimsize, int64_t m_size,
                                int64_t ignore_index, float lam, void *stream);

int plh_lmargin_backward_scaled(const void *logits, int32_t dtype, const int64_t *labels,
                                const float *grad_scalar, float scale, const int64_t *divide_by,
                                void *grad_logits,
                                int64_t n_size, int64_t dimsize, int64_t m_size,
                                int64_t ignore_index, float lam, void *stream);

int plh_lmargin_forward_backward(const void *logits, int32_t dtype, const int64_t *labels,
                                 float *losses, void *grad_logits, int64_t *valid_cnt,
                                 int64_t n_size, int64_t dimsize, int64_t m_size,
                                 int64_t ignore_index, float lam, void *stream);

/* The module step with fb=True and reduction 'mean' / 'sum' in ONE pass over the logits (replaces, in
 * large_margin_softmax.py:198-229 of the repository root, l_margin_forward_backward followed by losses.sum() / valid_cnt,
 * whose backward then multiplies the kept gradient by a per-pixel upstream tensor). The labels are counted first
 * (n_valid_out: labels other than ignore_index; required), then one kernel reads the logits, leaves the partial sums of
 * the losses and writes grad_logits already divided by that count (mean) - the gradient under an upstream gradient of 1.
 * loss_out: the sum or the mean (0/0 = NaN when nothing is valid). Workspace as for plh_lmargin_forward_reduced. */
int plh_lmargin_forward_backward_reduced(const void *logits, int32_t dtype, const int64_t *labels,
                                         float *loss_out, int64_t *n_valid_out, void *grad_logits, int32_t mean,
                                         void *workspace, int64_t workspace_bytes,
                                         int64_t n_size, int64_t dimsize, int64_t m_size,
                                         int64_t ignore_index, float lam, void *stream);

/* (N, C) rows (m_size 1) of more than 2048 classes, and shorter ones of more than 32 wherever the elementwise backward is
 * the faster one (16-bit logits: all of them; fp32: a class count that is no multiple of 32, or below 96, or above 1536):
 * the forward leaves eight floats of statistics per row
 * (stats_out: n_size * 8 floats on a 16-byte boundary) and the backward forms the gradient from them elementwise over the
 * flattened tensor instead of sweeping every row for them again (no counterpart in the reference, whose backward
 * recomputes: csrc/large_margin_kernel.cu:387-599). plh_lmargin_saves_stats says (1 / 0) whether the sizes qualify;
 * the other two are plh_lmargin_forward_reduced and plh_lmargin_backward_scaled / _kept (`kept`: optional byte mask, else
 * NULL) with that one more argument, and return PLH_ERR_BAD_SIZE for sizes that do not qualify. When logits or
 * grad_logits do not sit on 16-byte boundaries the recomputing kernel runs and `stats` is not read. */
int plh_lmargin_saves_stats(int32_t dtype, int64_t n_size, int64_t dimsize, int64_t m_size);
int plh_lmargin_forward_reduced_stats(const void *logits, int32_t dtype, const int64_t *labels, float *stats_out,
                                      float *loss_out, int64_t *n_valid_out, int32_t mean,
                                      void *workspace, int64_t workspace_bytes,
                                      int64_t n_size, int64_t dimsize, int64_t m_size,
                                      int64_t ignore_index, float lam, void *stream);
int plh_lmargin_backward_scaled_stats(const void *logits, int32_t dtype, const int64_t *labels,
                                      const float *stats, const uint8_t *kept,
                                      const float *grad_scalar, float scale, const int64_t *divide_by,
                                      void *grad_logits,
                                      int64_t n_size, int64_t dimsize, int64_t m_size,
                                      int64_t ignore_index, float lam, void *stream);

/* data[i] *= *scalar in place for numel elements of `dtype`, except that nothing is read or written when *scalar is exactly
 * 1: the backward of a kept gradient (replaces logits_grads.mul_(grad_output), large_margin_softmax.py:189 of the
 * repository root, for a scalar upstream gradient, which loss.backward() makes 1). `data` on a 16-byte boundary. */
int plh_scale_unless_one(void *data, int32_t dtype, int64_t numel, const float *scalar, void *stream);

/* ---- Lovasz-softmax ---------------------------------------------------------------
 * Replaces lovasz_softmax_cpp.lovasz_softmax_forward / lovasz_softmax_backward
 * (csrc/lovasz_softmax.cu:778-797; pipeline :495-773; csrc/cumsum.hpp:113-150).
 * losses: (dimsize) fp32, one Lovasz loss per class.
 * jacc:   (dimsize, n_size*m_size) fp32, the Jaccard differences scattered back to
 *         pixel order (pixel i = n*m_size + m); the forward writes every element
 *         and the backward only reads it.
 * workspace: scratch device memory of at least plh_lovasz_workspace_bytes() bytes,
 *         256-byte aligned, owned by the caller; contents are undefined afterwards.
 * Limits: dimsize < 512 and n_size*dimsize*m_size < 2^31 (csrc/lovasz_softmax.cu:664-665).
 */
int64_t plh_lovasz_workspace_bytes(int64_t n_size, int64_t dimsize, int64_t m_size);

int plh_lovasz_forward(const void *logits, int32_t dtype, const int64_t *labels,
                       float *losses, float *jacc,
                       void *workspace, int64_t workspace_bytes,
                       int64_t n_size, int64_t dimsize, int64_t m_size,
                       int64_t ignore_index, void *stream);

/* The same forward with the sort passes in their decoupled look-back form (tile descriptors and chained waits instead
 * of a histogram kernel and a row scan in front of every pass; no counterpart in the reference, whose scan is
 * csrc/cumsum.hpp:82-108). Results are those of plh_lovasz_forward bit for bit; it needs the larger workspace that
 * plh_lovasz_lookback_workspace_bytes() names, n_size*m_size < 2^30, and is the slower of the two on MI355X: it is
 * kept to be measured against the default. */
int64_t plh_lovasz_lookback_workspace_bytes(int64_t n_size, int64_t dimsize, int64_t m_size);

int plh_lovasz_forward_lookback(const void *logits, int32_t dtype, const int64_t *labels,
                                float *losses, float *jacc,
                                void *workspace, int64_t workspace_bytes,
                                int64_t n_size, int64_t dimsize, int64_t m_size,
                                int64_t ignore_index, void *stream);

int plh_lovasz_backward(const float *grad_output, const void *logits, int32_t dtype, const int64_t *labels,
                        const float *jacc, void *grad_logits,
                        int64_t n_size, int64_t dimsize, int64_t m_size,
                        int64_t ignore_index, void *stream);

/* ---- online hard example mining by score ---------------------------------------------
 * Replaces ohem_cpp.score_ohem_label (csrc/ohem_label_kernel.cu:171-276), the relabelling step
 * that pytorch_loss/ohem_loss.py:22-27 and :40-45 run before their loss: with the pixels ordered
 * by score = softmax(logits)[label] ascending (ignored pixels score 1, ties in pixel order),
 * every pixel at position >= n_min whose score exceeds score_thresh gets ignore_index as its
 * label; n_min >= n_size*m_size leaves the labels as they are (:189).
 *
 * plh_ohem_scores        scores (n_size*m_size fp32) only               (:112-151)
 * plh_ohem_select_labels the relabelling for given scores in [0, 1]     (:155-168, :247-262);
 *                        out_labels may be the labels buffer itself
 * plh_ohem_score_label   both; `scores` is scratch of n_size*m_size floats
 * workspace: at least plh_ohem_workspace_bytes(n_size*m_size) bytes, 256-byte aligned, owned by
 * the caller, contents undefined afterwards. Limit: n_size*m_size <= 2^31 - 1024.
 */
int64_t plh_ohem_workspace_bytes(int64_t n_pixels);

int plh_ohem_scores(const void *logits, int32_t dtype, const int64_t *labels, float *scores,
                    int64_t n_size, int64_t dimsize, int64_t m_size,
                    int64_t ignore_index, void *stream);

int plh_ohem_select_labels(const float *scores, const int64_t *labels, int64_t *out_labels,
                           void *workspace, int64_t workspace_bytes, int64_t n_pixels,
                           int64_t ignore_index, float score_thresh, int64_t n_min, void *stream);

int plh_ohem_score_label(const void *logits, int32_t dtype, const int64_t *labels,
                         int64_t *out_labels, float *scores,
                         void *workspace, int64_t workspace_bytes,
                         int64_t n_size, int64_t dimsize, int64_t m_size,
                         int64_t ignore_index, float score_thresh, int64_t n_min, void *stream);

/* OhemCELoss.forward in one call (pytorch_loss/ohem_loss.py:22-30: score_ohem_label, then
 * nn.CrossEntropyLoss(ignore_index, reduction='mean') on the new labels). The score pass already
 * holds each pixel's log-sum-exp and target logit, so it also writes the pixel's cross entropy
 * (pixel_ce, scratch of n_size*m_size floats like `scores`), and the relabelling pass adds up the
 * kept pixels': the forward reads the logits once instead of twice. out_labels: the new labels
 * (what the backward needs; plh_lsr_backward_scaled with smooth = 0 and divide_by = n_valid_out is
 * the matching gradient). loss_out: fp32 mean over the pixels whose new label is not ignore_index
 * (NaN if there are none), n_valid_out (may be NULL): their number. n_min >= n_size*m_size keeps
 * every label. workspace: plh_ohem_ce_workspace_bytes(n_size*m_size) bytes, 256-byte aligned.
 */
int64_t plh_ohem_ce_workspace_bytes(int64_t n_pixels);

int plh_ohem_ce_forward(const void *logits, int32_t dtype, const int64_t *labels,
                        int64_t *out_labels, float *scores, float *pixel_ce,
                        float *loss_out, int64_t *n_valid_out,
                        void *workspace, int64_t workspace_bytes,
                        int64_t n_size, int64_t dimsize, int64_t m_size,
                        int64_t ignore_index, float score_thresh, int64_t n_min, void *stream);

/* OhemLargeMarginLoss.forward in one call (pytorch_loss/ohem_loss.py:33-45: score_ohem_label, then
 * LargeMarginSoftmaxV3(ignore_index, reduction='mean') on the new labels). The large-margin forward
 * kernel holds the full softmax of every pixel, so it also writes the pixel's score; the relabelling
 * pass then adds up the kept pixels' losses (pixel_loss, scratch of n_size*m_size floats like
 * `scores`): one pass over the logits instead of two. plh_lmargin_backward_scaled on out_labels with
 * divide_by = n_valid_out is the matching gradient. Sizes, outputs and workspace as for
 * plh_ohem_ce_forward (plh_ohem_ce_workspace_bytes).
 */
int plh_ohem_lmargin_forward(const void *logits, int32_t dtype, const int64_t *labels,
                             int64_t *out_labels, float *scores, float *pixel_loss,
                             float *loss_out, int64_t *n_valid_out,
                             void *workspace, int64_t workspace_bytes,
                             int64_t n_size, int64_t dimsize, int64_t m_size,
                             int64_t ignore_index, float lam, float score_thresh, int64_t n_min, void *stream);

/* The two forwards above for callers that keep the selection as a mask rather than as new labels (no counterpart in
 * the reference; what OhemCELoss / OhemLargeMarginLoss of this package call): `kept` receives one byte per pixel,
 * 1 where the pixel keeps a label other than ignore_index and 0 elsewhere (4-byte aligned, n_size*m_size bytes). The
 * relabelling pass then neither reads the labels again nor writes new ones (9 instead of 24 bytes per pixel).
 * plh_lsr_backward_kept (smooth = 0) and plh_lmargin_backward_kept are the matching gradients: plh_*_backward_scaled
 * on the ORIGINAL labels, with an upstream gradient of 0 for every pixel whose byte in `kept` is 0. Everything else
 * as for plh_ohem_ce_forward / plh_ohem_lmargin_forward; `scores` holds 2 instead of 1 for pixels without a target.
 * On logits of up to 32 channels both also have their score pass leave mask, sum and count of the rule "drop what
 * scores above the threshold", which is the whole selection whenever n_min or more pixels score within the
 * threshold; the kernels of the selection then return at once. The loss then is a sum over other blocks than the
 * relabelling pass's: equal to plh_ohem_ce_forward's / plh_ohem_lmargin_forward's to rounding, not bit for bit.
 */
int plh_ohem_ce_forward_kept(const void *logits, int32_t dtype, const int64_t *labels,
                             uint8_t *kept, float *scores, float *pixel_ce,
                             float *loss_out, int64_t *n_valid_out,
                             void *workspace, int64_t workspace_bytes,
                             int64_t n_size, int64_t dimsize, int64_t m_size,
                             int64_t ignore_index, float score_thresh, int64_t n_min, void *stream);

int plh_ohem_lmargin_forward_kept(const void *logits, int32_t dtype, const int64_t *labels,
                                  uint8_t *kept, float *scores, float *pixel_loss,
                                  float *loss_out, int64_t *n_valid_out,
                                  void *workspace, int64_t workspace_bytes,
                                  int64_t n_size, int64_t dimsize, int64_t m_size,
                                  int64_t ignore_index, float lam, float score_thresh, int64_t n_min, void *stream);

int plh_lsr_backward_kept(const void *logits, int32_t dtype, const int64_t *labels, const uint8_t *kept,
                          const float *grad_scalar, float scale, const int64_t *divide_by,
                          void *grad_logits,
                          int64_t n_size, int64_t dimsize, int64_t m_size,
                          int64_t ignore_index, float smooth, void *stream);

int plh_lmargin_backward_kept(const void *logits, int32_t dtype, const int64_t *labels, const uint8_t *kept,
                              const float *grad_scalar, float scale, const int64_t *divide_by,
                              void *grad_logits,
                              int64_t n_size, int64_t dimsize, int64_t m_size,
                              int64_t ignore_index, float lam, void *stream);

/* ---- one-hot / label-smoothed targets -------------------------------------------------
 * Replaces one_hot_cpp.label_one_hot (csrc/one_hot_kernel.cu:265-350).
 * labels (n_size, m_size) int64 -> one_hot (n_size, dimsize, m_size) fp32: 0 in every channel of an
 * ignored pixel, else 1 - smooth at the label and smooth / dimsize elsewhere (:305-306).
 * range_flags: NULL, or two int32 in device memory that the call clears and then sets:
 *   [0] = 1 if some non-ignored label is >= dimsize, [1] = 1 if some is negative
 * (the reference finds max and min and synchronises to refuse such input, :301-304; here the
 * caller decides when to look). Labels outside [0, dimsize) match no channel and address nothing.
 */
int plh_onehot(const int64_t *labels, float *one_hot, int32_t *range_flags,
               int64_t n_size, int64_t dimsize, int64_t m_size,
               int64_t ignore_index, float smooth, void *stream);

/* ---- Taylor softmax ------------------------------------------------------------------
 * Replaces taylor_softmax_cpp.taylor_softmax_forward / taylor_softmax_backward
 * (csrc/taylor_softmax.cu:270-417). The tensor is (n_size, dimsize, m_size) around the dimension
 * the softmax runs over; feat, out, grad_output and grad_feat share `dtype`.
 *   f(x) = sum_{i=0..order} x^i / i!   (order even, 2..64),   S = sum_j f(x_j)
 *   out = f(x_j) / S, or log f(x_j) - log S with use_log               (:50-86)
 *   grad_feat from grad_output as in :140-192.
 */
int plh_taylor_softmax_forward(const void *feat, int32_t dtype, void *out,
                               int64_t n_size, int64_t dimsize, int64_t m_size,
                               int64_t order, int32_t use_log, void *stream);

int plh_taylor_softmax_backward(const void *grad_output, const void *feat, int32_t dtype,
                                void *grad_feat,
                                int64_t n_size, int64_t dimsize, int64_t m_size,
                                int64_t order, int32_t use_log, void *stream);

/* Cross entropy on the logarithmic Taylor softmax in one kernel per direction: what
 * TaylorCrossEntropyLossV3 composes from the Function above and F.nll_loss
 * (pytorch_loss/taylor_softmax.py:175-198). loss_i = log S - log f(x_y), 0 at ignored pixels.
 * forward: losses (n_size*m_size fp32) and/or, with loss_out != NULL, the 'sum' (mean = 0) or the
 *   mean over the non-ignored pixels (mean = 1) in *loss_out and their count in *n_valid_out
 *   (may be NULL); the reduced form needs a workspace of plh_reduce_workspace_bytes(n_size*m_size).
 * backward: grad_logits = dloss/dlogits * grad_output[i * stride] * scale / *divide_by
 *   (grad_output NULL = 1, stride 0 = one scalar; divide_by NULL = 1).
 */
int plh_taylor_ce_forward(const void *logits, int32_t dtype, const int64_t *labels, float *losses,
                          float *loss_out, int64_t *n_valid_out, int32_t mean,
                          void *workspace, int64_t workspace_bytes,
                          int64_t n_size, int64_t dimsize, int64_t m_size,
                          int64_t order, int64_t ignore_index, void *stream);

int plh_taylor_ce_backward(const void *logits, int32_t dtype, const int64_t *labels,
                           const float *grad_output, int64_t grad_output_stride, float scale,
                           const int64_t *divide_by, void *grad_logits,
                           int64_t n_size, int64_t dimsize, int64_t m_size,
                           int64_t order, int64_t ignore_index, void *stream);

/* (N, C) rows (m_size 1) of more than 32 classes wherever the elementwise backward is the faster one (fp32 rows except
 * those of a multiple of 32 classes from 96 to 768; 16-bit rows of more than 1024 classes, and of a multiple of 8 classes
 * up to 96), and fp32 channel planes (NCHW) of 4096 pixels or more that do not start on 128-byte lines, with up to 24
 * channels or 33..256 (513 x 513, 769 x 769 crops), and 257..512 channels on any plane of that size (orders 2 and 4, other
 * orders leave sums_out unwritten and recompute): the reduced
 * forward leaves each row's (pixel's) S = sum_j f(x_j)
 * (sums_out: n_size floats) and the backward forms the gradient from it elementwise over the flattened tensor instead of
 * summing every row again (no counterpart in the reference, where autograd keeps the log-softmax output between
 * TaylorSoftmaxFunc and F.nll_loss: pytorch_loss/taylor_softmax.py:175-198). plh_taylor_ce_saves_sums says (1 / 0)
 * whether the sizes qualify; the other two are plh_taylor_ce_forward with loss_out (no per-row losses) and
 * plh_taylor_ce_backward with one scalar upstream gradient, each with that one more argument, and return
 * PLH_ERR_BAD_SIZE for sizes that do not qualify. When logits or grad_logits do not sit on 16-byte boundaries (rows), or
 * not at the same offset into a 128-byte line (planes), the recomputing kernel runs and `sums` is not read. */
int plh_taylor_ce_saves_sums(int32_t dtype, int64_t n_size, int64_t dimsize, int64_t m_size);
int plh_taylor_ce_forward_reduced_sums(const void *logits, int32_t dtype, const int64_t *labels,
                                       float *sums_out, float *loss_out, int64_t *n_valid_out, int32_t mean,
                                       void *workspace, int64_t workspace_bytes,
                                       int64_t n_size, int64_t dimsize, int64_t m_size,
                                       int64_t order, int64_t ignore_index, void *stream);
int plh_taylor_ce_backward_scaled_sums(const void *logits, int32_t dtype, const int64_t *labels,
                                       const float *sums, const float *grad_scalar, float scale,
                                       const int64_t *divide_by, void *grad_logits,
                                       int64_t n_size, int64_t dimsize, int64_t m_size,
                                       int64_t order, int64_t ignore_index, void *stream);

/* ---- soft dice loss ---------------------------------------------------------------------
 * Replaces soft_dice_cpp.soft_dice_forward / soft_dice_backward (csrc/soft_dice_kernel_v2.cu:258-436).
 * logits and labels are (batchsize, sample_size) tensors of one floating type (`dtype`); with
 * q = sigmoid(logits): numer = 2 sum(q y) + smooth, denor = sum(q^p + y) + smooth per row
 * (the label is not raised to p, csrc/soft_dice_kernel_v2.cu:90; equal to y^p for binary labels),
 * losses[n] = 1 - numer / denor (fp32).
 * forward also leaves (numer, denor) per row in stats (batchsize x 2 fp32), which the backward
 * reads instead of reducing the rows again; workspace: plh_soft_dice_workspace_bytes() bytes,
 * 256-byte aligned. backward: grad_logits[n, l] = grad_output[n] * dloss_n/dlogits[n, l].
 * Limit: batchsize <= 65535.
 */
int64_t plh_soft_dice_workspace_bytes(int64_t batchsize, int64_t sample_size);

int plh_soft_dice_forward(const void *logits, int32_t dtype, const void *labels,
                          float *losses, float *stats,
                          void *workspace, int64_t workspace_bytes,
                          int64_t batchsize, int64_t sample_size,
                          float p, float smooth, void *stream);

int plh_soft_dice_backward(const float *grad_output, const void *logits, int32_t dtype,
                           const void *labels, const float *stats, void *grad_logits,
                           int64_t batchsize, int64_t sample_size, float p, void *stream);

/* ---- layer norm over the channel dimension --------------------------------------------
 * Replaces layer_norm_cpp.layer_norm_forward / layer_norm_backward (csrc/layer_norm.cu:377-393;
 * kernels :53-257). x, out, grad_output, grad_x: (n_size, dimsize, m_size) contiguous in `dtype`.
 * forward: out = (x - mean) * rsqrt(var + eps), mean and population variance over dimsize for
 * each (n, m). backward returns what the reference's kernel returns (:212-216),
 *   -rsqrt(v) * (1/C + (x - mean) * (x - 1/C) * mean * v) * grad_output,  v = var + eps.
 * Arithmetic is fp32 for every dtype. Limit: n_size * m_size <= 64 * (2^31 - 1).
 */
int plh_layer_norm_forward(const void *x, int32_t dtype, void *out,
                           int64_t n_size, int64_t dimsize, int64_t m_size,
                           float eps, void *stream);

int plh_layer_norm_backward(const void *grad_output, const void *x, int32_t dtype, void *grad_x,
                            int64_t n_size, int64_t dimsize, int64_t m_size,
                            float eps, void *stream);

/* ---- measurement aid ----------------------------------------------------------------
 * Plain fp32 device-to-device copy kernel of known traffic (4*numel bytes read,
 * 4*numel written), used to calibrate hardware byte counters and to measure the
 * achievable copy bandwidth.  No counterpart in the reference.
 */
int plh_stream_copy(const float *src, float *dst, int64_t numel, void *stream);

#ifdef __cplusplus
}
#endif

#endif /* PYTORCH_LOSS_HIP_H */
