// Sigmoid focal loss, forward / backward / fused forward+backward, for gfx950.
//
// Per element (x logit, y label in [0,1], csrc/focal_kernel.cu:39-51,65-83):
//   p      = sigmoid(x)
//   log p  = min(x,0) - log1p(exp(-|x|)),  log(1-p) = -max(x,0) - log1p(exp(-|x|))
//            (focal_loss.py:59-64; the CUDA kernel's log p - x loses digits for x << 0)
//   ce     = y*alpha*log p + (1-y)*(1-alpha)*log(1-p)
//   coeff  = -|y-p|^gamma,                  loss = coeff*ce
//   d_ce   = y*alpha - p*(1 - y - alpha + 2*y*alpha)
//   d_coef = gamma*|y-p|^(gamma-1)*p*(1-p), negated when y < p
//   grad   = (d_coef*ce + d_ce*coeff) * upstream
// Pure streaming: every thread moves one 128-bit vector per tensor; a scalar
// kernel finishes sizes that are not a multiple of 4 (or unaligned pointers).
#include "plh_common.hpp"

namespace plh {

enum GammaMode { kGammaTwo = 0, kGammaOne = 1, kGammaAny = 2 };

struct FocalParams {
    float gamma, alpha;
};

template <int Mode, bool WantLoss, bool WantGrad>
__device__ __forceinline__ void focal_point(float x, float y, const FocalParams p, float &loss, float &grad) {
    const float e = fast_exp(-fabsf(x));             // exp(-|x|) in [0, 1]: one exponential serves p and log p
    const float inv = __builtin_amdgcn_rcpf(1.f + e);
    const float prob = (x >= 0.f) ? inv : e * inv;
    const float l1p = fast_log1p_unit(e);
    const float log_p = fminf(x, 0.f) - l1p;
    const float log_1p = -fmaxf(x, 0.f) - l1p;       // formed directly: log_p - x cancels for x << 0
    const float ce = y * p.alpha * log_p + (1.f - y) * (1.f - p.alpha) * log_1p;
    const float a = fabsf(y - prob);
    float a_pow, a_pow_m1;                           // |y-p|^gamma and |y-p|^(gamma-1)
    if constexpr (Mode == kGammaTwo) {
        a_pow = a * a;
        a_pow_m1 = a;
    } else if constexpr (Mode == kGammaOne) {
        a_pow = a;
        a_pow_m1 = 1.f;
    } else {
        a_pow = powf(a, p.gamma);
        a_pow_m1 = WantGrad ? powf(a, p.gamma - 1.f) : 0.f;
    }
    const float coeff = -a_pow;
    if constexpr (WantLoss) loss = coeff * ce;
    if constexpr (WantGrad) {
        const float d_ce = y * p.alpha - prob * (1.f - y - p.alpha + 2.f * y * p.alpha);
        float d_coeff = p.gamma * a_pow_m1 * prob * (1.f - prob);
        if (y < prob) d_coeff = -d_coeff;
        grad = d_coeff * ce + d_ce * coeff;
    }
}

// One float4 per thread. Reduce: also leave the block's sum of losses in part.sum[slot0 + block].
template <class T, int Mode, bool WantLoss, bool WantGrad, bool Reduce>
__global__ __launch_bounds__(256) void focal_vec4(const T *__restrict__ x, const T *__restrict__ y,
                                                  const Upstream up, float *__restrict__ loss,
                                                  T *__restrict__ grad, float *__restrict__ partial,
                                                  int64_t n4, const FocalParams p) {
    __shared__ float red[4];
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const bool live = i < n4;
    if (!Reduce && !live) return;
    const int64_t at = live ? i * 4 : 0;
    float xs[4], ys[4], go[4], l[4], g[4];
    load_vec<4>(x + at, xs);
    load_vec<4>(y + at, ys);
    if constexpr (WantGrad) load_upstream<4>(up, at, go);
    float mine = 0.f;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        focal_point<Mode, WantLoss || Reduce, WantGrad>(xs[k], ys[k], p, l[k], g[k]);
        if constexpr (WantGrad) g[k] *= go[k];
        if constexpr (Reduce) mine += live ? l[k] : 0.f;
    }
    if (live) {
        if (WantLoss && loss) store_vec<4>(loss + at, l);
        if constexpr (WantGrad) store_vec<4>(grad + at, g);
    }
    if constexpr (Reduce) {
        const float bs = block_sum_256(mine, red);
        if (threadIdx.x == 0) partial[blockIdx.x] = bs;
    }
}

template <class T, int Mode, bool WantLoss, bool WantGrad, bool Reduce>
__global__ __launch_bounds__(256) void focal_scalar(const T *__restrict__ x, const T *__restrict__ y,
                                                    const Upstream up, float *__restrict__ loss,
                                                    T *__restrict__ grad, float *__restrict__ partial,
                                                    int64_t first, int64_t numel, const FocalParams p) {
    __shared__ float red[4];
    const int64_t i = first + (int64_t)blockIdx.x * 256 + threadIdx.x;
    const bool live = i < numel;
    if (!Reduce && !live) return;
    const int64_t at = live ? i : first;
    float l = 0.f, g = 0.f;
    focal_point<Mode, WantLoss || Reduce, WantGrad>(load_one(x + at), load_one(y + at), p, l, g);
    if (live) {
        if (WantLoss && loss) loss[at] = l;
        if constexpr (WantGrad) {
            float go[1];
            load_upstream<1>(up, at, go);
            store_one(grad + at, g * go[0]);
        }
    }
    if constexpr (Reduce) {
        const float bs = block_sum_256(live ? l : 0.f, red);
        if (threadIdx.x == 0) partial[blockIdx.x] = bs;
    }
}

// Returns the number of partial slots written (0 unless Reduce).
template <class T, int Mode, bool WantLoss, bool WantGrad, bool Reduce>
static unsigned launch_mode(const T *x, const T *y, const Upstream &up, float *loss, T *grad, float *partial,
                            int64_t numel, const FocalParams &p, hipStream_t st) {
    int64_t done = 0;
    unsigned slots = 0;
    const bool aligned = !misaligned(x, 4 * sizeof(T)) && !misaligned(y, 4 * sizeof(T)) &&
                         !(loss && misaligned(loss, 16)) && !(WantGrad && misaligned(grad, 4 * sizeof(T))) &&
                         !(WantGrad && up.gout && up.stride == 1 && misaligned(up.gout, 16));
    if (aligned && numel >= 4) {
        const int64_t n4 = numel / 4;
        const unsigned grid = (unsigned)ceil_div(n4, 256);
        hipLaunchKernelGGL((focal_vec4<T, Mode, WantLoss, WantGrad, Reduce>), dim3(grid), dim3(256), 0, st, x, y, up,
                           loss, grad, partial, n4, p);
        done = n4 * 4;
        slots = grid;
    }
    if (done < numel) {
        const unsigned grid = (unsigned)ceil_div(numel - done, 256);
        hipLaunchKernelGGL((focal_scalar<T, Mode, WantLoss, WantGrad, Reduce>), dim3(grid), dim3(256), 0, st, x, y, up,
                           loss, grad, Reduce ? partial + slots : nullptr, done, numel, p);
        slots += grid;
    }
    return Reduce ? slots : 0;
}

template <bool WantLoss, bool WantGrad, bool Reduce>
static int launch(const void *x, const void *y, int32_t dtype, const Upstream &up, float *loss, void *grad,
                  float *partial, unsigned *slots_out, int64_t numel, float gamma, float alpha, void *stream) {
    if (slots_out) *slots_out = 0;
    if (!dtype_ok(dtype)) return PLH_ERR_BAD_DTYPE;
    if (numel < 0 || numel > kMaxNumel) return PLH_ERR_BAD_SIZE;
    if (numel == 0) return PLH_OK;
    if (!x || !y || (WantLoss && !Reduce && !loss) || (WantGrad && !grad)) return PLH_ERR_NULL_POINTER;
    const size_t es = dtype_size(dtype);
    if (misaligned(x, es) || misaligned(y, es) || misaligned(loss, 4) || misaligned(grad, es)) return PLH_ERR_MISALIGNED;
    const FocalParams p{gamma, alpha};
    hipStream_t st = (hipStream_t)stream;
    unsigned slots = 0;
    dispatch_dtype(dtype, [&](auto tag) {
        using T = decltype(tag);
        const T *xt = static_cast<const T *>(x), *yt = static_cast<const T *>(y);
        T *gt = static_cast<T *>(grad);
        if (gamma == 2.f) slots = launch_mode<T, kGammaTwo, WantLoss, WantGrad, Reduce>(xt, yt, up, loss, gt, partial, numel, p, st);
        else if (gamma == 1.f) slots = launch_mode<T, kGammaOne, WantLoss, WantGrad, Reduce>(xt, yt, up, loss, gt, partial, numel, p, st);
        else slots = launch_mode<T, kGammaAny, WantLoss, WantGrad, Reduce>(xt, yt, up, loss, gt, partial, numel, p, st);
    });
    if (slots_out) *slots_out = slots;
    return check_launch();
}

}  // namespace plh

using namespace plh;

extern "C" int plh_focal_forward(const void *logits, int32_t dtype, const void *labels, float *losses,
                                 int64_t numel, float gamma, float alpha, void *stream) {
    const Upstream up{nullptr, 0, nullptr, 1.f};
    return launch<true, false, false>(logits, labels, dtype, up, losses, nullptr, nullptr, nullptr, numel, gamma, alpha,
                                      stream);
}

extern "C" int plh_focal_forward_reduced(const void *logits, int32_t dtype, const void *labels, float *losses,
                                         float *loss_out, int32_t mean, void *workspace, int64_t workspace_bytes,
                                         int64_t numel, float gamma, float alpha, void *stream) {
    if (numel < 0 || numel > kMaxNumel) return PLH_ERR_BAD_SIZE;
    Partials part;
    int rc = carve_partials(workspace, workspace_bytes, numel, loss_out, nullptr, part);
    if (rc != PLH_OK) return rc;
    const Upstream up{nullptr, 0, nullptr, 1.f};
    unsigned slots = 0;
    rc = launch<true, false, true>(logits, labels, dtype, up, losses, nullptr, part.sum, &slots, numel, gamma, alpha,
                                   stream);
    if (rc != PLH_OK) return rc;
    part.cnt = nullptr;
    finish_partials(part, slots, loss_out, nullptr, mean ? kFinishMeanOverFixed : kFinishSum, numel, (hipStream_t)stream);
    return check_launch();
}

extern "C" int plh_focal_backward(const void *logits, int32_t dtype, const void *labels,
                                  const float *grad_output, int64_t grad_output_stride, void *grad_logits,
                                  int64_t numel, float gamma, float alpha, void *stream) {
    const int rc = check_gout(grad_output, grad_output_stride);
    if (rc != PLH_OK) return rc;
    const Upstream up{grad_output, grad_output_stride, nullptr, 1.f};
    return launch<false, true, false>(logits, labels, dtype, up, nullptr, grad_logits, nullptr, nullptr, numel, gamma,
                                      alpha, stream);
}

extern "C" int plh_focal_backward_scaled(const void *logits, int32_t dtype, const void *labels,
                                         const float *grad_scalar, float scale, void *grad_logits,
                                         int64_t numel, float gamma, float alpha, void *stream) {
    if (numel > 0 && !grad_scalar) return PLH_ERR_NULL_POINTER;
    if (misaligned(grad_scalar, 4)) return PLH_ERR_MISALIGNED;
    const Upstream up{grad_scalar, 0, nullptr, scale};
    return launch<false, true, false>(logits, labels, dtype, up, nullptr, grad_logits, nullptr, nullptr, numel, gamma,
                                      alpha, stream);
}

extern "C" int plh_focal_forward_backward(const void *logits, int32_t dtype, const void *labels, float *losses,
                                          void *grad_logits, int64_t numel, float gamma, float alpha,
                                          void *stream) {
    const Upstream up{nullptr, 0, nullptr, 1.f};
    return launch<true, true, false>(logits, labels, dtype, up, losses, grad_logits, nullptr, nullptr, numel, gamma,
                                     alpha, stream);
}

extern "C" int plh_focal_forward_backward_reduced(const void *logits, int32_t dtype, const void *labels, float *loss_out,
                                                  void *grad_logits, int32_t mean, void *workspace,
                                                  int64_t workspace_bytes, int64_t numel, float gamma, float alpha,
                                                  void *stream) {
    if (numel < 0 || numel > kMaxNumel) return PLH_ERR_BAD_SIZE;
    Partials part;
    int rc = carve_partials(workspace, workspace_bytes, numel, loss_out, nullptr, part);
    if (rc != PLH_OK) return rc;
    // the mean's divisor is the element count, known here: the gradient is written already divided by it
    const Upstream up{nullptr, 0, nullptr, (mean && numel > 0) ? 1.f / (float)numel : 1.f};
    unsigned slots = 0;
    rc = launch<true, true, true>(logits, labels, dtype, up, nullptr, grad_logits, part.sum, &slots, numel, gamma, alpha,
                                  stream);
    if (rc != PLH_OK) return rc;
    part.cnt = nullptr;
    finish_partials(part, slots, loss_out, nullptr, mean ? kFinishMeanOverFixed : kFinishSum, numel, (hipStream_t)stream);
    return check_launch();
}
