// Label-smoothed softmax cross entropy for gfx950: the C entry points. The kernels live in
// lsr_kernels.hpp and are compiled per element type and direction (lsr_f32_fwd.hip, lsr_f32_bwd.hip, ...).
#include <mutex>

#include "lsr_kernels.hpp"

namespace plh {

// Partials buffer of plh_lsr_forward_reduced_static: device memory that belongs to the loaded code
// object (every GPU the library runs on holds its own copy at its own address until the process ends).
// Host code never uses this name as an address; scratch_for_current_device() asks the runtime for it.
constexpr int64_t kStaticMaxPixels = (int64_t)1 << 24;
constexpr int64_t kStaticScratchBytes = 8 * (kStaticMaxPixels / 64);    // = 8 * partial_slots(kStaticMaxPixels) = 2 MiB
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;

// The device address of `scratch` on the current device, looked up once per device.
static int scratch_for_current_device(void **out) {
    static std::mutex mu;
    static void *ptrs[kMaxDevices] = {};
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return PLH_ERR_BAD_SIZE;
    std::lock_guard<std::mutex> lock(mu);
    if (!ptrs[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!p) return PLH_ERR_WORKSPACE;
        ptrs[dev] = p;
    }
    *out = ptrs[dev];
    return PLH_OK;
}

PLH_LSR_EXTERN(float)
PLH_LSR_EXTERN(f16)
PLH_LSR_EXTERN(bf16)

static int backward(const void *logits, int32_t dtype, const int64_t *labels, const Upstream &up, void *grad_logits,
                    int64_t n_size, int64_t dimsize, int64_t m_size, int64_t ignore_index, float smooth,
                    void *stream, const float *lse = nullptr) {
    if (!dtype_ok(dtype)) return PLH_ERR_BAD_DTYPE;
    const int rc = check_slice_args(logits, labels, grad_logits, n_size, dimsize, m_size, dtype_size(dtype),
                                    dtype_size(dtype));
    if (rc != PLH_OK) return rc;
    if (n_size * dimsize * m_size == 0) return PLH_OK;
    if (lse && (misaligned(lse, 4) || !lsr_lse_applies(dtype_size(dtype), dimsize, m_size))) return PLH_ERR_BAD_SIZE;
    LsrParams p = make_params(n_size, dimsize, m_size, ignore_index, smooth, dtype_size(dtype));
    p.lse = const_cast<float *>(lse);           // read only in the backward
    dispatch_dtype(dtype, [&](auto tag) {
        using T = decltype(tag);
        lsr_backward_typed<T>(static_cast<const T *>(logits), labels, up, static_cast<T *>(grad_logits), p,
                          (hipStream_t)stream);
    });
    return check_launch();
}

}  // namespace plh

using namespace plh;

extern "C" int plh_lsr_forward(const void *logits, int32_t dtype, const int64_t *labels, float *losses,
                               int64_t n_size, int64_t dimsize, int64_t m_size,
                               int64_t ignore_index, float smooth, void *stream) {
    if (!dtype_ok(dtype)) return PLH_ERR_BAD_DTYPE;
    const int rc = check_slice_args(logits, labels, losses, n_size, dimsize, m_size, dtype_size(dtype), 4);
    if (rc != PLH_OK) return rc;
    if (n_size * dimsize * m_size == 0) return PLH_OK;
    const LsrParams p = make_params(n_size, dimsize, m_size, ignore_index, smooth, dtype_size(dtype));
    dispatch_dtype(dtype, [&](auto tag) {
        using T = decltype(tag);
        lsr_forward_typed<T>(static_cast<const T *>(logits), labels, losses, Partials{nullptr, nullptr}, false, p,
                             (hipStream_t)stream);
    });
    return check_launch();
}

static int forward_reduced(const void *logits, int32_t dtype, const int64_t *labels, float *losses, float *lse_out,
                           float *loss_out, int64_t *n_valid_out, int32_t mean, void *workspace, int64_t workspace_bytes,
                           int64_t n_size, int64_t dimsize, int64_t m_size, int64_t ignore_index, float smooth,
                           void *stream) {
    if (!dtype_ok(dtype)) return PLH_ERR_BAD_DTYPE;
    if (lse_out && (misaligned(lse_out, 4) || !lsr_lse_applies(dtype_size(dtype), dimsize, m_size))) return PLH_ERR_BAD_SIZE;
    int rc = check_slice_args(logits, labels, loss_out, n_size, dimsize, m_size, dtype_size(dtype), 4);
    if (rc != PLH_OK) return rc;
    Partials part;
    rc = carve_partials(workspace, workspace_bytes, n_size * m_size, loss_out, n_valid_out, part);
    if (rc != PLH_OK) return rc;
    if (losses && misaligned(losses, 4)) return PLH_ERR_MISALIGNED;
    hipStream_t st = (hipStream_t)stream;
    unsigned blocks = 0;
    if (n_size * dimsize * m_size != 0) {
        LsrParams p = make_params(n_size, dimsize, m_size, ignore_index, smooth, dtype_size(dtype));
        p.lse = lse_out;
        dispatch_dtype(dtype, [&](auto tag) {
            using T = decltype(tag);
            blocks = lsr_forward_typed<T>(static_cast<const T *>(logits), labels, losses, part, true, p, st);
        });
    }
    finish_partials(part, blocks, loss_out, n_valid_out, mean ? kFinishMeanOverCount : kFinishSum, 0, st);
    return check_launch();
}

extern "C" int plh_lsr_forward_reduced(const void *logits, int32_t dtype, const int64_t *labels, float *losses,
                                       float *loss_out, int64_t *n_valid_out, int32_t mean,
                                       void *workspace, int64_t workspace_bytes,
                                       int64_t n_size, int64_t dimsize, int64_t m_size,
                                       int64_t ignore_index, float smooth, void *stream) {
    return forward_reduced(logits, dtype, labels, losses, nullptr, loss_out, n_valid_out, mean, workspace, workspace_bytes,
                           n_size, dimsize, m_size, ignore_index, smooth, stream);
}

extern "C" int plh_lsr_forward_backward_reduced(const void *logits, int32_t dtype, const int64_t *labels,
                                                float *loss_out, int64_t *n_valid_out, void *grad_logits, int32_t mean,
                                                void *workspace, int64_t workspace_bytes,
                                                int64_t n_size, int64_t dimsize, int64_t m_size,
                                                int64_t ignore_index, float smooth, void *stream) {
    if (!dtype_ok(dtype)) return PLH_ERR_BAD_DTYPE;
    if (!n_valid_out) return PLH_ERR_NULL_POINTER;
    const size_t es = dtype_size(dtype);
    int rc = check_slice_args(logits, labels, grad_logits, n_size, dimsize, m_size, es, es);
    if (rc != PLH_OK) return rc;
    Partials part;
    rc = carve_partials(workspace, workspace_bytes, n_size * m_size, loss_out, n_valid_out, part);
    if (rc != PLH_OK) return rc;
    hipStream_t st = (hipStream_t)stream;
    const FinishMode mode = mean ? kFinishMeanOverCount : kFinishSum;
    if (n_size * dimsize * m_size == 0) {
        finish_partials(part, 0, loss_out, n_valid_out, mode, 0, st);
        return check_launch();
    }
    const LsrParams p = make_params(n_size, dimsize, m_size, ignore_index, smooth, es);
    // One pass where the register-resident kernels run: the mean's divisor first (a count of the labels), so that the
    // pass writes the gradient already divided by it. The partials of the count are gone before the pass leaves its own.
    const bool one_pass = dimsize <= kMaxRegsChannels;
    if (one_pass && mean) {
        const unsigned counted = count_valid_partials(labels, n_size * m_size, ignore_index, part, st);
        finish_partials(part, counted, loss_out, n_valid_out, kFinishSum, 0, st);
    }
    const Upstream up{nullptr, 0, mean ? n_valid_out : nullptr, 1.f};
    unsigned blocks = 0;
    if (one_pass)
        dispatch_dtype(dtype, [&](auto tag) {
            using T = decltype(tag);
            blocks = lsr_fused_typed<T>(static_cast<const T *>(logits), labels, up, static_cast<T *>(grad_logits), part, p,
                                        st);
        });
    if (blocks != 0) {
        finish_partials(part, blocks, loss_out, n_valid_out, mode, 0, st);
        return check_launch();
    }
    // every other shape: the forward and the backward one after the other (same outputs; the forward's own count
    // divides the gradient - the count taken above, if any, is the same number)
    dispatch_dtype(dtype, [&](auto tag) {
        using T = decltype(tag);
        blocks = lsr_forward_typed<T>(static_cast<const T *>(logits), labels, nullptr, part, true, p, st);
    });
    finish_partials(part, blocks, loss_out, n_valid_out, mode, 0, st);
    dispatch_dtype(dtype, [&](auto tag) {
        using T = decltype(tag);
        lsr_backward_typed<T>(static_cast<const T *>(logits), labels, up, static_cast<T *>(grad_logits), p, st);
    });
    return check_launch();
}

extern "C" int plh_lsr_saves_lse(int32_t dtype, int64_t n_size, int64_t dimsize, int64_t m_size) {
    return dtype_ok(dtype) && n_size > 0 && dimsize > 0 && m_size > 0 &&
           lsr_lse_applies(dtype_size(dtype), dimsize, m_size) ? 1 : 0;
}

extern "C" int plh_lsr_forward_reduced_lse(const void *logits, int32_t dtype, const int64_t *labels, float *lse_out,
                                           float *loss_out, int64_t *n_valid_out, int32_t mean,
                                           void *workspace, int64_t workspace_bytes,
                                           int64_t n_size, int64_t dimsize, int64_t m_size,
                                           int64_t ignore_index, float smooth, void *stream) {
    if (!lse_out && n_size * dimsize * m_size != 0) return PLH_ERR_NULL_POINTER;
    return forward_reduced(logits, dtype, labels, nullptr, lse_out, loss_out, n_valid_out, mean, workspace, workspace_bytes,
                           n_size, dimsize, m_size, ignore_index, smooth, stream);
}

extern "C" int plh_lsr_forward_reduced_static(const void *logits, int32_t dtype, const int64_t *labels, float *losses,
                                              float *loss_out, int64_t *n_valid_out, int32_t mean,
                                              int64_t n_size, int64_t dimsize, int64_t m_size,
                                              int64_t ignore_index, float smooth, void *stream) {
    if (n_size < 0 || m_size < 0 || n_size > kStaticMaxPixels || m_size > kStaticMaxPixels ||
        n_size * m_size > kStaticMaxPixels)
        return PLH_ERR_BAD_SIZE;
    static_assert(8 * ((kStaticMaxPixels + 63) / 64) <= kStaticScratchBytes && kStaticMaxPixels / 64 >= kMinPartialSlots,
                  "the static buffer holds the partials of the largest accepted input");
    void *ws = nullptr;
    const int rc = scratch_for_current_device(&ws);
    if (rc != PLH_OK) return rc;
    // Every partial that the finishing kernel reads was written by this call's forward kernel, so
    // nothing has to be cleared between calls.
    return plh_lsr_forward_reduced(logits, dtype, labels, losses, loss_out, n_valid_out, mean, ws, kStaticScratchBytes,
                                   n_size, dimsize, m_size, ignore_index, smooth, stream);
}

extern "C" int plh_lsr_backward(const void *logits, int32_t dtype, const int64_t *labels,
                                const float *grad_output, int64_t grad_output_stride,
                                void *grad_logits,
                                int64_t n_size, int64_t dimsize, int64_t m_size,
                                int64_t ignore_index, float smooth, void *stream) {
    const int rc = check_gout(grad_output, grad_output_stride);
    if (rc != PLH_OK) return rc;
    const Upstream up{grad_output, grad_output_stride, nullptr, 1.f};
    return backward(logits, dtype, labels, up, grad_logits, n_size, dimsize, m_size, ignore_index, smooth, stream);
}

extern "C" int plh_lsr_backward_scaled(const void *logits, int32_t dtype, const int64_t *labels,
                                       const float *grad_scalar, float scale, const int64_t *divide_by,
                                       void *grad_logits,
                                       int64_t n_size, int64_t dimsize, int64_t m_size,
                                       int64_t ignore_index, float smooth, void *stream) {
    if (n_size * dimsize * m_size != 0 && !grad_scalar) return PLH_ERR_NULL_POINTER;
    if (misaligned(grad_scalar, 4) || misaligned(divide_by, 8)) return PLH_ERR_MISALIGNED;
    const Upstream up{grad_scalar, 0, divide_by, scale};
    return backward(logits, dtype, labels, up, grad_logits, n_size, dimsize, m_size, ignore_index, smooth, stream);
}

extern "C" int plh_lsr_backward_kept(const void *logits, int32_t dtype, const int64_t *labels, const uint8_t *kept,
                                     const float *grad_scalar, float scale, const int64_t *divide_by,
                                     void *grad_logits,
                                     int64_t n_size, int64_t dimsize, int64_t m_size,
                                     int64_t ignore_index, float smooth, void *stream) {
    if (n_size * dimsize * m_size != 0 && (!grad_scalar || !kept)) return PLH_ERR_NULL_POINTER;
    if (misaligned(grad_scalar, 4) || misaligned(divide_by, 8)) return PLH_ERR_MISALIGNED;
    const Upstream up{grad_scalar, 0, divide_by, scale, kept};
    return backward(logits, dtype, labels, up, grad_logits, n_size, dimsize, m_size, ignore_index, smooth, stream);
}

extern "C" int plh_lsr_backward_scaled_lse(const void *logits, int32_t dtype, const int64_t *labels, const float *lse,
                                           const uint8_t *kept, const float *grad_scalar, float scale,
                                           const int64_t *divide_by, void *grad_logits,
                                           int64_t n_size, int64_t dimsize, int64_t m_size,
                                           int64_t ignore_index, float smooth, void *stream) {
    if (n_size * dimsize * m_size != 0 && (!grad_scalar || !lse)) return PLH_ERR_NULL_POINTER;
    if (misaligned(grad_scalar, 4) || misaligned(divide_by, 8)) return PLH_ERR_MISALIGNED;
    const Upstream up{grad_scalar, 0, divide_by, scale, kept};
    return backward(logits, dtype, labels, up, grad_logits, n_size, dimsize, m_size, ignore_index, smooth, stream, lse);
}
