// Layer norm over the channel dimension: the C entry points. Kernels live in layernorm_kernels.hpp
// and are compiled once per element type (layernorm_f32.hip, layernorm_f16.hip, layernorm_bf16.hip).
#include "layernorm_kernels.hpp"

namespace plh {

PLH_LN_EXTERN(float)
PLH_LN_EXTERN(f16)
PLH_LN_EXTERN(bf16)

static int ln_check(const void *x, const void *out, int64_t n_size, int64_t dimsize, int64_t m_size, size_t es) {
    static const int64_t aligned_dummy[1] = {0};       // stands in for the labels check_slice_args expects
    int rc = check_slice_args(x, (n_size * dimsize * m_size != 0) ? aligned_dummy : nullptr, out, n_size, dimsize, m_size,
                              es, es);
    if (rc != PLH_OK) return rc;
    // a launch covers at most 2^31 - 1 pixel groups of 64 pixels
    if ((double)n_size * (double)m_size > 64.0 * 2147483647.0) return PLH_ERR_BAD_SIZE;
    return PLH_OK;
}

}  // namespace plh

using namespace plh;

extern "C" int plh_layer_norm_forward(const void *x, int32_t dtype, void *out, int64_t n_size, int64_t dimsize,
                                      int64_t m_size, float eps, void *stream) {
    if (!dtype_ok(dtype)) return PLH_ERR_BAD_DTYPE;
    const size_t es = dtype_size(dtype);
    const int rc = ln_check(x, out, n_size, dimsize, m_size, es);
    if (rc != PLH_OK) return rc;
    if (n_size * dimsize * m_size == 0) return PLH_OK;
    dispatch_dtype(dtype, [&](auto tag) {
        using T = decltype(tag);
        ln_run_typed<T>(false, static_cast<const T *>(x), nullptr, static_cast<T *>(out), n_size, dimsize, m_size, eps,
                        (hipStream_t)stream);
    });
    return check_launch();
}

extern "C" int plh_layer_norm_backward(const void *grad_output, const void *x, int32_t dtype, void *grad_x,
                                       int64_t n_size, int64_t dimsize, int64_t m_size, float eps, void *stream) {
    if (!dtype_ok(dtype)) return PLH_ERR_BAD_DTYPE;
    const size_t es = dtype_size(dtype);
    const int rc = ln_check(x, grad_x, n_size, dimsize, m_size, es);
    if (rc != PLH_OK) return rc;
    if (n_size * dimsize * m_size == 0) return PLH_OK;
    if (!grad_output) return PLH_ERR_NULL_POINTER;
    if (misaligned(grad_output, es)) return PLH_ERR_MISALIGNED;
    dispatch_dtype(dtype, [&](auto tag) {
        using T = decltype(tag);
        ln_run_typed<T>(true, static_cast<const T *>(x), static_cast<const T *>(grad_output), static_cast<T *>(grad_x),
                        n_size, dimsize, m_size, eps, (hipStream_t)stream);
    });
    return check_launch();
}
