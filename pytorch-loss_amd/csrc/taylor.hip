// Taylor softmax and the cross entropy on its logarithm: the C entry points. Kernels live in
// taylor_kernels.hpp and are compiled per element type and kind (taylor_f32_fwd.hip, ...).
#include "taylor_kernels.hpp"

namespace plh {

PLH_TAYLOR_EXTERN(float)
PLH_TAYLOR_EXTERN(f16)
PLH_TAYLOR_EXTERN(bf16)

template <class T>
static unsigned taylor_run_typed(int kind, const T *x, const T *g, const int64_t *lab, const Upstream &up, T *out,
                                 float *loss, Partials part, const TaylorParams &p, hipStream_t st) {
    switch (kind) {
        case kTaylorFwd: return taylor_launch<T, kTaylorFwd>(x, g, lab, up, out, loss, part, p, st);
        case kTaylorBwd: return taylor_launch<T, kTaylorBwd>(x, g, lab, up, out, loss, part, p, st);
        case kTaylorCeFwd: return taylor_launch<T, kTaylorCeFwd>(x, g, lab, up, out, loss, part, p, st);
        default: return taylor_launch<T, kTaylorCeBwd>(x, g, lab, up, out, loss, part, p, st);
    }
}

// Size and pointer checks of the label-free entry points: `in` and `out` hold elem-byte elements.
static int check_pair(const void *in, const void *out, int64_t n_size, int64_t dimsize, int64_t m_size, size_t elem) {
    static const int64_t aligned_dummy[1] = {0};       // stands in for the labels check_slice_args expects
    return check_slice_args(in, (n_size * dimsize * m_size != 0) ? aligned_dummy : nullptr, out, n_size, dimsize, m_size,
                            elem, elem);
}

static int check_order(int64_t order) { return (order < 2 || order > 64 || (order & 1)) ? PLH_ERR_BAD_SIZE : PLH_OK; }

static TaylorParams make_taylor(int64_t n_size, int64_t dimsize, int64_t m_size, int64_t order, int use_log,
                                int64_t ignore, size_t elem) {
    TaylorParams p;
    p.P = n_size * m_size;
    p.m_size = m_size;
    p.C = (int)dimsize;
    p.order = (int)order;
    p.use_log = use_log ? 1 : 0;
    p.ignore = ignore;
    p.xcd_run = xcd_run_for(elem, m_size);
    return p;
}

static unsigned run(int kind, int32_t dtype, const void *x, const void *g, const int64_t *lab,
                    const Upstream &up, void *out, float *loss, Partials part, const TaylorParams &p, hipStream_t st) {
    unsigned blocks = 0;
    dispatch_dtype(dtype, [&](auto tag) {
        using T = decltype(tag);
        blocks = taylor_run_typed<T>(kind, static_cast<const T *>(x), static_cast<const T *>(g), lab, up,
                                     static_cast<T *>(out), loss, part, p, st);
    });
    return blocks;
}

}  // namespace plh

using namespace plh;

static const Partials kNone{nullptr, nullptr};
static const Upstream kUnit{nullptr, 0, nullptr, 1.f};

extern "C" int plh_taylor_softmax_forward(const void *feat, int32_t dtype, void *out,
                                          int64_t n_size, int64_t dimsize, int64_t m_size,
                                          int64_t order, int32_t use_log, void *stream) {
    if (!dtype_ok(dtype)) return PLH_ERR_BAD_DTYPE;
    int rc = check_order(order);
    if (rc != PLH_OK) return rc;
    const size_t es = dtype_size(dtype);
    rc = check_pair(feat, out, n_size, dimsize, m_size, es);
    if (rc != PLH_OK) return rc;
    if (n_size * dimsize * m_size == 0) return PLH_OK;
    run(kTaylorFwd, dtype, feat, nullptr, nullptr, kUnit, out, nullptr, kNone,
        make_taylor(n_size, dimsize, m_size, order, use_log, 0, es), (hipStream_t)stream);
    return check_launch();
}

extern "C" int plh_taylor_softmax_backward(const void *grad_output, const void *feat, int32_t dtype, void *grad_feat,
                                           int64_t n_size, int64_t dimsize, int64_t m_size,
                                           int64_t order, int32_t use_log, void *stream) {
    if (!dtype_ok(dtype)) return PLH_ERR_BAD_DTYPE;
    int rc = check_order(order);
    if (rc != PLH_OK) return rc;
    const size_t es = dtype_size(dtype);
    rc = check_pair(feat, grad_feat, n_size, dimsize, m_size, es);
    if (rc != PLH_OK) return rc;
    if (n_size * dimsize * m_size == 0) return PLH_OK;
    if (!grad_output) return PLH_ERR_NULL_POINTER;
    if (misaligned(grad_output, es)) return PLH_ERR_MISALIGNED;
    run(kTaylorBwd, dtype, feat, grad_output, nullptr, kUnit, grad_feat, nullptr, kNone,
        make_taylor(n_size, dimsize, m_size, order, use_log, 0, es), (hipStream_t)stream);
    return check_launch();
}

extern "C" int plh_taylor_ce_forward(const void *logits, int32_t dtype, const int64_t *labels, float *losses,
                                     float *loss_out, int64_t *n_valid_out, int32_t mean,
                                     void *workspace, int64_t workspace_bytes,
                                     int64_t n_size, int64_t dimsize, int64_t m_size,
                                     int64_t order, int64_t ignore_index, void *stream) {
    if (!dtype_ok(dtype)) return PLH_ERR_BAD_DTYPE;
    int rc = check_order(order);
    if (rc != PLH_OK) return rc;
    const size_t es = dtype_size(dtype);
    const bool reduce = loss_out != nullptr;
    if (!reduce && !losses && n_size * dimsize * m_size != 0) return PLH_ERR_NULL_POINTER;
    rc = check_slice_args(logits, labels, reduce ? (const void *)loss_out : (const void *)losses, n_size, dimsize, m_size,
                          es, 4);
    if (rc != PLH_OK) return rc;
    if (losses && misaligned(losses, 4)) return PLH_ERR_MISALIGNED;
    Partials part = kNone;
    if (reduce) {
        rc = carve_partials(workspace, workspace_bytes, n_size * m_size, loss_out, n_valid_out, part);
        if (rc != PLH_OK) return rc;
    }
    hipStream_t st = (hipStream_t)stream;
    unsigned blocks = 0;
    if (n_size * dimsize * m_size != 0)
        blocks = run(kTaylorCeFwd, dtype, logits, nullptr, labels, kUnit, nullptr, losses, part,
                     make_taylor(n_size, dimsize, m_size, order, 1, ignore_index, es), st);
    if (reduce) finish_partials(part, blocks, loss_out, n_valid_out, mean ? kFinishMeanOverCount : kFinishSum, 0, st);
    return check_launch();
}

extern "C" int plh_taylor_ce_backward(const void *logits, int32_t dtype, const int64_t *labels,
                                      const float *grad_output, int64_t grad_output_stride, float scale,
                                      const int64_t *divide_by, void *grad_logits,
                                      int64_t n_size, int64_t dimsize, int64_t m_size,
                                      int64_t order, int64_t ignore_index, void *stream) {
    if (!dtype_ok(dtype)) return PLH_ERR_BAD_DTYPE;
    int rc = check_order(order);
    if (rc != PLH_OK) return rc;
    rc = check_gout(grad_output, grad_output_stride);
    if (rc != PLH_OK) return rc;
    if (misaligned(divide_by, 8)) return PLH_ERR_MISALIGNED;
    const size_t es = dtype_size(dtype);
    rc = check_slice_args(logits, labels, grad_logits, n_size, dimsize, m_size, es, es);
    if (rc != PLH_OK) return rc;
    if (n_size * dimsize * m_size == 0) return PLH_OK;
    const Upstream up{grad_output, grad_output_stride, divide_by, scale};
    run(kTaylorCeBwd, dtype, logits, nullptr, labels, up, grad_logits, nullptr, kNone,
        make_taylor(n_size, dimsize, m_size, order, 1, ignore_index, es), (hipStream_t)stream);
    return check_launch();
}

extern "C" int plh_taylor_ce_saves_sums(int32_t dtype, int64_t n_size, int64_t dimsize, int64_t m_size) {
    return dtype_ok(dtype) && n_size > 0 && dimsize > 0 && m_size > 0 &&
                   taylor_sums_apply(dtype_size(dtype), dimsize, m_size) ? 1 : 0;
}

extern "C" int plh_taylor_ce_forward_reduced_sums(const void *logits, int32_t dtype, const int64_t *labels,
                                                  float *sums_out, float *loss_out, int64_t *n_valid_out, int32_t mean,
                                                  void *workspace, int64_t workspace_bytes,
                                                  int64_t n_size, int64_t dimsize, int64_t m_size,
                                                  int64_t order, int64_t ignore_index, void *stream) {
    if (!dtype_ok(dtype)) return PLH_ERR_BAD_DTYPE;
    int rc = check_order(order);
    if (rc != PLH_OK) return rc;
    if (n_size < 0 || m_size < 0 || n_size > kMaxNumel || m_size > kMaxNumel) return PLH_ERR_BAD_SIZE;
    if (!taylor_sums_apply(dtype_size(dtype), dimsize, m_size)) return PLH_ERR_BAD_SIZE;
    if (!loss_out) return PLH_ERR_NULL_POINTER;
    if (!sums_out && n_size * dimsize * m_size != 0) return PLH_ERR_NULL_POINTER;
    if (misaligned(sums_out, 4)) return PLH_ERR_MISALIGNED;
    const size_t es = dtype_size(dtype);
    rc = check_slice_args(logits, labels, loss_out, n_size, dimsize, m_size, es, 4);
    if (rc != PLH_OK) return rc;
    Partials part = kNone;
    rc = carve_partials(workspace, workspace_bytes, n_size * m_size, loss_out, n_valid_out, part);
    if (rc != PLH_OK) return rc;
    hipStream_t st = (hipStream_t)stream;
    unsigned blocks = 0;
    if (n_size * dimsize * m_size != 0) {
        TaylorParams p = make_taylor(n_size, dimsize, m_size, order, 1, ignore_index, es);
        // (channel planes: the kernels that leave and use S per pixel are compiled for orders 2 and 4; other orders
        // leave sums_out unwritten and the backward recomputes)
        p.sums = (m_size > 1 && order > 4) ? nullptr : sums_out;
        blocks = run(kTaylorCeFwd, dtype, logits, nullptr, labels, kUnit, nullptr, nullptr, part, p, st);
    }
    finish_partials(part, blocks, loss_out, n_valid_out, mean ? kFinishMeanOverCount : kFinishSum, 0, st);
    return check_launch();
}

extern "C" int plh_taylor_ce_backward_scaled_sums(const void *logits, int32_t dtype, const int64_t *labels,
                                                  const float *sums, const float *grad_scalar, float scale,
                                                  const int64_t *divide_by, void *grad_logits,
                                                  int64_t n_size, int64_t dimsize, int64_t m_size,
                                                  int64_t order, int64_t ignore_index, void *stream) {
    if (!dtype_ok(dtype)) return PLH_ERR_BAD_DTYPE;
    int rc = check_order(order);
    if (rc != PLH_OK) return rc;
    if (!taylor_sums_apply(dtype_size(dtype), dimsize, m_size)) return PLH_ERR_BAD_SIZE;
    if (n_size * dimsize * m_size != 0 && (!grad_scalar || !sums)) return PLH_ERR_NULL_POINTER;
    if (misaligned(grad_scalar, 4) || misaligned(divide_by, 8) || misaligned(sums, 4)) return PLH_ERR_MISALIGNED;
    const size_t es = dtype_size(dtype);
    rc = check_slice_args(logits, labels, grad_logits, n_size, dimsize, m_size, es, es);
    if (rc != PLH_OK) return rc;
    if (n_size * dimsize * m_size == 0) return PLH_OK;
    const Upstream up{grad_scalar, 0, divide_by, scale};
    TaylorParams p = make_taylor(n_size, dimsize, m_size, order, 1, ignore_index, es);
    p.sums = (m_size > 1 && order > 4) ? nullptr : const_cast<float *>(sums);
    run(kTaylorCeBwd, dtype, logits, nullptr, labels, up, grad_logits, nullptr, kNone, p, (hipStream_t)stream);
    return check_launch();
}
