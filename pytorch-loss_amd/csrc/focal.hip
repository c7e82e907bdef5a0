// Sigmoid focal loss, forward / backward / fused forward+backward, for gfx950.
//
// Per element (x logit, y label in [0,1], csrc/focal_kernel.cu:39-51,65-83):
//   p      = sigmoid(x)
//   log p  = min(x,0) - log1p(exp(-|x|)),  log(1-p) = log p - x
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
    const float e = expf(-fabsf(x));                 // exp(-|x|) in (0, 1]: one exponential serves p and log p
    const float inv = 1.f / (1.f + e);
    const float prob = (x >= 0.f) ? inv : e * inv;
    const float log_p = fminf(x, 0.f) - log1pf(e);
    const float log_1p = log_p - x;
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

// One float4 per thread. gout: nullptr = 1, gstride 0 = broadcast scalar, 1 = per element.
template <int Mode, bool WantLoss, bool WantGrad>
__global__ __launch_bounds__(256) void focal_vec4(const float4 *__restrict__ x4, const float4 *__restrict__ y4,
                                                  const float *__restrict__ gout, int64_t gstride,
                                                  float4 *__restrict__ loss4, float4 *__restrict__ grad4,
                                                  int64_t n4, const FocalParams p) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n4) return;
    const float4 xv = x4[i];
    const float4 yv = y4[i];
    float go[4];
    if constexpr (WantGrad) load_gout<4>(gout, gstride, i * 4, go);
    const float xs[4] = {xv.x, xv.y, xv.z, xv.w};
    const float ys[4] = {yv.x, yv.y, yv.z, yv.w};
    float l[4], g[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        focal_point<Mode, WantLoss, WantGrad>(xs[k], ys[k], p, l[k], g[k]);
        if constexpr (WantGrad) g[k] *= go[k];
    }
    if constexpr (WantLoss) loss4[i] = make_float4(l[0], l[1], l[2], l[3]);
    if constexpr (WantGrad) grad4[i] = make_float4(g[0], g[1], g[2], g[3]);
}

template <int Mode, bool WantLoss, bool WantGrad>
__global__ __launch_bounds__(256) void focal_scalar(const float *__restrict__ x, const float *__restrict__ y,
                                                    const float *__restrict__ gout, int64_t gstride,
                                                    float *__restrict__ loss, float *__restrict__ grad,
                                                    int64_t first, int64_t numel, const FocalParams p) {
    const int64_t i = first + (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= numel) return;
    float l, g;
    focal_point<Mode, WantLoss, WantGrad>(x[i], y[i], p, l, g);
    if constexpr (WantLoss) loss[i] = l;
    if constexpr (WantGrad) {
        float go[1];
        load_gout<1>(gout, gstride, i, go);
        grad[i] = g * go[0];
    }
}

template <int Mode, bool WantLoss, bool WantGrad>
static void launch_mode(const float *x, const float *y, const float *gout, int64_t gstride, float *loss,
                        float *grad, int64_t numel, const FocalParams &p, hipStream_t st) {
    int64_t done = 0;
    const bool aligned = !misaligned(x, 16) && !misaligned(y, 16) && !(WantLoss && misaligned(loss, 16)) &&
                         !(WantGrad && misaligned(grad, 16)) &&
                         !(WantGrad && gout && gstride == 1 && misaligned(gout, 16));
    if (aligned && numel >= 4) {
        const int64_t n4 = numel / 4;
        hipLaunchKernelGGL((focal_vec4<Mode, WantLoss, WantGrad>), dim3((unsigned)ceil_div(n4, 256)), dim3(256), 0, st,
                           reinterpret_cast<const float4 *>(x), reinterpret_cast<const float4 *>(y), gout, gstride,
                           reinterpret_cast<float4 *>(loss), reinterpret_cast<float4 *>(grad), n4, p);
        done = n4 * 4;
    }
    if (done < numel) {
        hipLaunchKernelGGL((focal_scalar<Mode, WantLoss, WantGrad>), dim3((unsigned)ceil_div(numel - done, 256)),
                           dim3(256), 0, st, x, y, gout, gstride, loss, grad, done, numel, p);
    }
}

template <bool WantLoss, bool WantGrad>
static int launch(const float *x, const float *y, const float *gout, int64_t gstride, float *loss, float *grad,
                  int64_t numel, float gamma, float alpha, void *stream) {
    if (numel < 0 || numel > kMaxNumel) return PLH_ERR_BAD_SIZE;
    if (numel == 0) return PLH_OK;
    if (!x || !y || (WantLoss && !loss) || (WantGrad && !grad)) return PLH_ERR_NULL_POINTER;
    if (misaligned(x, 4) || misaligned(y, 4) || misaligned(loss, 4) || misaligned(grad, 4)) return PLH_ERR_MISALIGNED;
    const int rc = check_gout(gout, gstride);
    if (rc != PLH_OK) return rc;
    const FocalParams p{gamma, alpha};
    hipStream_t st = (hipStream_t)stream;
    if (gamma == 2.f) launch_mode<kGammaTwo, WantLoss, WantGrad>(x, y, gout, gstride, loss, grad, numel, p, st);
    else if (gamma == 1.f) launch_mode<kGammaOne, WantLoss, WantGrad>(x, y, gout, gstride, loss, grad, numel, p, st);
    else launch_mode<kGammaAny, WantLoss, WantGrad>(x, y, gout, gstride, loss, grad, numel, p, st);
    return check_launch();
}

}  // namespace plh

extern "C" int plh_focal_forward(const float *logits, const float *labels, float *losses,
                                 int64_t numel, float gamma, float alpha, void *stream) {
    return plh::launch<true, false>(logits, labels, nullptr, 0, losses, nullptr, numel, gamma, alpha, stream);
}

extern "C" int plh_focal_backward(const float *logits, const float *labels,
                                  const float *grad_output, int64_t grad_output_stride, float *grad_logits,
                                  int64_t numel, float gamma, float alpha, void *stream) {
    return plh::launch<false, true>(logits, labels, grad_output, grad_output_stride, nullptr, grad_logits, numel,
                                    gamma, alpha, stream);
}

extern "C" int plh_focal_forward_backward(const float *logits, const float *labels, float *losses,
                                          float *grad_logits, int64_t numel, float gamma, float alpha,
                                          void *stream) {
    return plh::launch<true, true>(logits, labels, nullptr, 0, losses, grad_logits, numel, gamma, alpha, stream);
}
