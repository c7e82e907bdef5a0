// Large-margin softmax cross entropy for gfx950: the C entry points. The kernels live in
// lmargin_kernels.hpp and are compiled per element type and direction (lmargin_f32_fwd.hip, ...).
#include "lmargin_kernels.hpp"

namespace plh {

PLH_LM_EXTERN(float)
PLH_LM_EXTERN(f16)
PLH_LM_EXTERN(bf16)

// The partial sums (part.sum) and the count of valid pixels (cnt) are produced when their pointers are given: the
// kernels test the pointers, so the reduced forward shares its kernels with the plain one.
template <class T>
static unsigned lmargin_run_typed(int variant, const T *x, const int64_t *lab, const Upstream &up, float *loss, T *grad,
                                  unsigned long long *cnt, Partials part, const LmParams &p, hipStream_t st) {
    switch (variant) {
        case kLmForward:
        case kLmForwardReduced: return launch_typed<T, true, false>(x, lab, up, loss, grad, cnt, part, p, st);
        case kLmBackward: return launch_typed<T, false, true>(x, lab, up, loss, grad, cnt, part, p, st);
        default: return launch_typed<T, true, true>(x, lab, up, loss, grad, cnt, part, p, st);
    }
}

// Launches one direction (or the fused pair). blocks_out: blocks that wrote partials (Reduce only).
static int launch(int variant, const void *x, int32_t dtype, const int64_t *lab, const Upstream &up, float *loss, void *grad,
                  int64_t *valid_cnt, Partials part, unsigned *blocks_out, int64_t n_size, int64_t dimsize,
                  int64_t m_size, int64_t ignore, float lam, void *stream, float *scores = nullptr,
                  float no_target_score = 1.f, const OhemEarly *early = nullptr, float *saved = nullptr) {
    const bool WantLoss = variant != kLmBackward, WantGrad = variant >= kLmBackward;
    const bool WantCount = variant == kLmForwardBackwardCount;
    const bool Reduce = variant == kLmForwardReduced || variant == kLmForwardBackwardReduced;
    if (blocks_out) *blocks_out = 0;
    if (!dtype_ok(dtype)) return PLH_ERR_BAD_DTYPE;
    const size_t es = dtype_size(dtype);
    const bool out_is_loss = WantLoss && !Reduce;
    const void *out = out_is_loss ? (const void *)loss : (WantGrad ? (const void *)grad : x);
    int rc = check_slice_args(x, lab, out, n_size, dimsize, m_size, es, out_is_loss ? 4 : es);
    if (rc != PLH_OK) return rc;
    if (up.gout && up.stride == 1 && misaligned(up.gout, 4)) return PLH_ERR_MISALIGNED;
    if (WantCount && (!valid_cnt || misaligned(valid_cnt, 8))) return valid_cnt ? PLH_ERR_MISALIGNED : PLH_ERR_NULL_POINTER;
    hipStream_t st = (hipStream_t)stream;
    unsigned long long *cnt = reinterpret_cast<unsigned long long *>(valid_cnt);
    if (WantCount) hipLaunchKernelGGL(lm_zero_count, dim3(1), dim3(1), 0, st, cnt);
    if (n_size * dimsize * m_size == 0) return check_launch();
    // the fused pair's count of valid pixels comes from a pass over the labels (256 atomics): with the fused kernel
    // counting, one atomic per wavefront on the one address, the call took 0.81 ms at (8,19,1024,1024) fp32 and 0.76 ms
    // at (65536,1000); now 0.26 and 0.085 ms
    if (WantCount) {
        count_valid_total(lab, n_size * m_size, ignore, cnt, st);
        cnt = nullptr;
    }
    if (WantLoss && WantGrad && (!grad || misaligned(grad, es))) return grad ? PLH_ERR_MISALIGNED : PLH_ERR_NULL_POINTER;
    if (loss && misaligned(loss, 4)) return PLH_ERR_MISALIGNED;

    LmParams p;
    p.P = n_size * m_size;
    p.m_size = m_size;
    p.C = (int)dimsize;
    p.ignore = ignore;
    p.half_lam = lam / 2.f;                          // csrc/large_margin_kernel.cu:188
    p.coeff = 1.f / (float)(dimsize - 1);            // csrc/large_margin_kernel.cu:404
    p.xcd_run = xcd_run_for(es, m_size);
    p.scores = scores;
    p.no_target_score = no_target_score;
    p.saved = saved;
    if (early) {
        p.early_kept = early->kept;
        p.early_below = early->below;
        p.early_thresh = early->thresh;
    }
    unsigned blocks = 0;
    dispatch_dtype(dtype, [&](auto tag) {
        using T = decltype(tag);
        blocks = lmargin_run_typed<T>(variant, static_cast<const T *>(x), lab, up, loss, static_cast<T *>(grad), cnt,
                                      part, p, st);
    });
    if (blocks_out) *blocks_out = blocks;
    return check_launch();
}

static const Partials kNoPartials{nullptr, nullptr};

// Declared in plh_common.hpp for the OHEM entry point: the per-pixel forward that also leaves each
// pixel's score.
// With `early` (see OhemEarly) the launch is a reduced forward whose partial sums run over the pixels of the threshold
// rule; *early_blocks is the number of blocks that left them, 0 when the launch shape took none of it (the
// per-pixel losses and scores are written either way).
int lmargin_forward_with_scores(const void *logits, int32_t dtype, const int64_t *labels, float *losses, float *scores,
                                int64_t n_size, int64_t dimsize, int64_t m_size, int64_t ignore_index, float lam,
                                hipStream_t stream, float no_target_score, const OhemEarly *early, unsigned *early_blocks) {
    const Upstream up{nullptr, 0, nullptr, 1.f};
    if (early_blocks) *early_blocks = 0;
    // up to kMaxRegsChannels channels every forward runs in the register-resident kernels (pick_shape), the ones that
    // take LmParams::early_*; their partial sums come from at most one block per 256 pixels, which is what `early` holds
    const bool regs = early && early->kept && early_blocks && dimsize <= kMaxRegsChannels;
    if (regs) {
        unsigned blocks = 0;
        const int rc = launch(kLmForwardReduced, logits, dtype, labels, up, losses, nullptr, nullptr,
                              Partials{early->sum, early->cnt}, &blocks, n_size, dimsize, m_size, ignore_index, lam, stream,
                              scores, no_target_score, early);
        if (rc == PLH_OK && (blocks & kLmTookEarly)) *early_blocks = blocks & ~kLmTookEarly;
        return rc;
    }
    return launch(kLmForward, logits, dtype, labels, up, losses, nullptr, nullptr, kNoPartials, nullptr, n_size, dimsize,
                  m_size, ignore_index, lam, stream, scores, no_target_score);
}

}  // namespace plh

using namespace plh;

extern "C" int plh_lmargin_forward(const void *logits, int32_t dtype, const int64_t *labels, float *losses,
                                   int64_t n_size, int64_t dimsize, int64_t m_size,
                                   int64_t ignore_index, float lam, void *stream) {
    const Upstream up{nullptr, 0, nullptr, 1.f};
    return launch(kLmForward, logits, dtype, labels, up, losses, nullptr, nullptr, kNoPartials, nullptr,
                                             n_size, dimsize, m_size, ignore_index, lam, stream);
}

extern "C" int plh_lmargin_forward_reduced(const void *logits, int32_t dtype, const int64_t *labels, float *losses,
                                           float *loss_out, int64_t *n_valid_out, int32_t mean,
                                           void *workspace, int64_t workspace_bytes,
                                           int64_t n_size, int64_t dimsize, int64_t m_size,
                                           int64_t ignore_index, float lam, void *stream) {
    if (n_size < 0 || m_size < 0 || n_size > kMaxNumel || m_size > kMaxNumel) return PLH_ERR_BAD_SIZE;
    Partials part;
    int rc = carve_partials(workspace, workspace_bytes, n_size * m_size, loss_out, n_valid_out, part);
    if (rc != PLH_OK) return rc;
    const Upstream up{nullptr, 0, nullptr, 1.f};
    unsigned blocks = 0;
    rc = launch(kLmForwardReduced, logits, dtype, labels, up, losses, nullptr, nullptr, part, &blocks, n_size,
                                          dimsize, m_size, ignore_index, lam, stream);
    if (rc != PLH_OK) return rc;
    finish_partials(part, blocks, loss_out, n_valid_out, mean ? kFinishMeanOverCount : kFinishSum, 0,
                    (hipStream_t)stream);
    return check_launch();
}

extern "C" int plh_lmargin_backward(const void *logits, int32_t dtype, const int64_t *labels,
                                    const float *grad_output, int64_t grad_output_stride, void *grad_logits,
                                    int64_t n_size, int64_t dimsize, int64_t m_size,
                                    int64_t ignore_index, float lam, void *stream) {
    const int rc = check_gout(grad_output, grad_output_stride);
    if (rc != PLH_OK) return rc;
    const Upstream up{grad_output, grad_output_stride, nullptr, 1.f};
    return launch(kLmBackward, logits, dtype, labels, up, nullptr, grad_logits, nullptr, kNoPartials,
                                             nullptr, n_size, dimsize, m_size, ignore_index, lam, stream);
}

extern "C" int plh_lmargin_backward_scaled(const void *logits, int32_t dtype, const int64_t *labels,
                                           const float *grad_scalar, float scale, const int64_t *divide_by,
                                           void *grad_logits,
                                           int64_t n_size, int64_t dimsize, int64_t m_size,
                                           int64_t ignore_index, float lam, void *stream) {
    if (n_size * dimsize * m_size != 0 && !grad_scalar) return PLH_ERR_NULL_POINTER;
    if (misaligned(grad_scalar, 4) || misaligned(divide_by, 8)) return PLH_ERR_MISALIGNED;
    const Upstream up{grad_scalar, 0, divide_by, scale};
    return launch(kLmBackward, logits, dtype, labels, up, nullptr, grad_logits, nullptr, kNoPartials,
                                             nullptr, n_size, dimsize, m_size, ignore_index, lam, stream);
}

extern "C" int plh_lmargin_backward_kept(const void *logits, int32_t dtype, const int64_t *labels, const uint8_t *kept,
                                         const float *grad_scalar, float scale, const int64_t *divide_by,
                                         void *grad_logits,
                                         int64_t n_size, int64_t dimsize, int64_t m_size,
                                         int64_t ignore_index, float lam, void *stream) {
    if (n_size * dimsize * m_size != 0 && (!grad_scalar || !kept)) return PLH_ERR_NULL_POINTER;
    if (misaligned(grad_scalar, 4) || misaligned(divide_by, 8)) return PLH_ERR_MISALIGNED;
    const Upstream up{grad_scalar, 0, divide_by, scale, kept};
    return launch(kLmBackward, logits, dtype, labels, up, nullptr, grad_logits, nullptr, kNoPartials,
                                             nullptr, n_size, dimsize, m_size, ignore_index, lam, stream);
}

extern "C" int plh_lmargin_forward_backward(const void *logits, int32_t dtype, const int64_t *labels, float *losses,
                                            void *grad_logits, int64_t *valid_cnt,
                                            int64_t n_size, int64_t dimsize, int64_t m_size,
                                            int64_t ignore_index, float lam, void *stream) {
    const Upstream up{nullptr, 0, nullptr, 1.f};
    return launch(kLmForwardBackwardCount, logits, dtype, labels, up, losses, grad_logits, valid_cnt, kNoPartials,
                                           nullptr, n_size, dimsize, m_size, ignore_index, lam, stream);
}

extern "C" int plh_lmargin_forward_backward_reduced(const void *logits, int32_t dtype, const int64_t *labels,
                                                    float *loss_out, int64_t *n_valid_out, void *grad_logits, int32_t mean,
                                                    void *workspace, int64_t workspace_bytes,
                                                    int64_t n_size, int64_t dimsize, int64_t m_size,
                                                    int64_t ignore_index, float lam, void *stream) {
    if (n_size < 0 || m_size < 0 || n_size > kMaxNumel || m_size > kMaxNumel) return PLH_ERR_BAD_SIZE;
    if (!n_valid_out) return PLH_ERR_NULL_POINTER;
    Partials part;
    int rc = carve_partials(workspace, workspace_bytes, n_size * m_size, loss_out, n_valid_out, part);
    if (rc != PLH_OK) return rc;
    hipStream_t st = (hipStream_t)stream;
    const bool any = n_size * dimsize * m_size != 0;
    if (any && !labels) return PLH_ERR_NULL_POINTER;
    if (misaligned(labels, 8)) return PLH_ERR_MISALIGNED;
    // More than kMaxRegsChannels channels in NCHW: the fused kernel there has a lane walk its pixel's channels, and
    // the forward and the backward that share a pixel among wavefronts are faster one after the other than it is alone
    // ((8,150,512,512) fp32: 0.64 against 1.06 ms); same outputs, and the forward's own count divides the gradient.
    if (any && m_size > 1 && dimsize > kMaxRegsChannels) {
        if (!grad_logits) return PLH_ERR_NULL_POINTER;
        const Upstream unit{nullptr, 0, nullptr, 1.f};
        unsigned blocks = 0;
        rc = launch(kLmForwardReduced, logits, dtype, labels, unit, nullptr, nullptr, nullptr, part, &blocks, n_size, dimsize,
                    m_size, ignore_index, lam, stream);
        if (rc != PLH_OK) return rc;
        finish_partials(part, blocks, loss_out, n_valid_out, mean ? kFinishMeanOverCount : kFinishSum, 0, st);
        const Upstream up{nullptr, 0, mean ? n_valid_out : nullptr, 1.f};
        return launch(kLmBackward, logits, dtype, labels, up, nullptr, grad_logits, nullptr, kNoPartials, nullptr, n_size,
                      dimsize, m_size, ignore_index, lam, stream);
    }
    // the mean's divisor first: the one pass over the logits writes the gradient already divided by it
    if (any && mean) {
        const unsigned counted = count_valid_partials(labels, n_size * m_size, ignore_index, part, st);
        finish_partials(part, counted, loss_out, n_valid_out, kFinishSum, 0, st);
    }
    const Upstream up{nullptr, 0, mean ? n_valid_out : nullptr, 1.f};
    unsigned blocks = 0;
    rc = launch(kLmForwardBackwardReduced, logits, dtype, labels, up, nullptr, grad_logits, nullptr, part, &blocks, n_size,
                dimsize, m_size, ignore_index, lam, stream);
    if (rc != PLH_OK) return rc;
    finish_partials(part, blocks, loss_out, n_valid_out, mean ? kFinishMeanOverCount : kFinishSum, 0, st);
    return check_launch();
}

extern "C" int plh_lmargin_saves_stats(int32_t dtype, int64_t n_size, int64_t dimsize, int64_t m_size) {
    return dtype_ok(dtype) && n_size > 0 && dimsize > 0 && m_size > 0 && lm_saved_applies(dtype_size(dtype), dimsize, m_size) ? 1 : 0;
}

extern "C" int plh_lmargin_forward_reduced_stats(const void *logits, int32_t dtype, const int64_t *labels, float *stats_out,
                                                 float *loss_out, int64_t *n_valid_out, int32_t mean,
                                                 void *workspace, int64_t workspace_bytes,
                                                 int64_t n_size, int64_t dimsize, int64_t m_size,
                                                 int64_t ignore_index, float lam, void *stream) {
    if (n_size < 0 || m_size < 0 || n_size > kMaxNumel || m_size > kMaxNumel) return PLH_ERR_BAD_SIZE;
    if (!dtype_ok(dtype)) return PLH_ERR_BAD_DTYPE;
    if (!lm_saved_applies(dtype_size(dtype), dimsize, m_size)) return PLH_ERR_BAD_SIZE;
    if (!stats_out && n_size * dimsize * m_size != 0) return PLH_ERR_NULL_POINTER;
    if (misaligned(stats_out, 16)) return PLH_ERR_MISALIGNED;
    Partials part;
    int rc = carve_partials(workspace, workspace_bytes, n_size * m_size, loss_out, n_valid_out, part);
    if (rc != PLH_OK) return rc;
    const Upstream up{nullptr, 0, nullptr, 1.f};
    unsigned blocks = 0;
    rc = launch(kLmForwardReduced, logits, dtype, labels, up, nullptr, nullptr, nullptr, part, &blocks, n_size, dimsize,
                m_size, ignore_index, lam, stream, nullptr, 1.f, nullptr, stats_out);
    if (rc != PLH_OK) return rc;
    finish_partials(part, blocks, loss_out, n_valid_out, mean ? kFinishMeanOverCount : kFinishSum, 0,
                    (hipStream_t)stream);
    return check_launch();
}

extern "C" int plh_lmargin_backward_scaled_stats(const void *logits, int32_t dtype, const int64_t *labels,
                                                 const float *stats, const uint8_t *kept,
                                                 const float *grad_scalar, float scale, const int64_t *divide_by,
                                                 void *grad_logits,
                                                 int64_t n_size, int64_t dimsize, int64_t m_size,
                                                 int64_t ignore_index, float lam, void *stream) {
    if (!dtype_ok(dtype)) return PLH_ERR_BAD_DTYPE;
    if (!lm_saved_applies(dtype_size(dtype), dimsize, m_size)) return PLH_ERR_BAD_SIZE;
    if (n_size * dimsize * m_size != 0 && (!grad_scalar || !stats)) return PLH_ERR_NULL_POINTER;
    if (misaligned(grad_scalar, 4) || misaligned(divide_by, 8) || misaligned(stats, 16)) return PLH_ERR_MISALIGNED;
    const Upstream up{grad_scalar, 0, divide_by, scale, kept};
    return launch(kLmBackward, logits, dtype, labels, up, nullptr, grad_logits, nullptr, kNoPartials, nullptr, n_size,
                  dimsize, m_size, ignore_index, lam, stream, nullptr, 1.f, nullptr, const_cast<float *>(stats));
}
