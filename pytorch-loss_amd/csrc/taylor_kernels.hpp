// Taylor softmax (de Brebisson & Vincent; "Exploring Alternatives to Softmax Function") along one
// dimension, forward and backward, plus the cross entropy built on its logarithm, for gfx950.
//
// With f(x) = sum_{i=0..n} x^i / i!  (n even, so f > 0) and S = sum_j f(x_j) over the dimension:
//   y_j      = f(x_j) / S                    or, with use_log,  log f(x_j) - log S
//   backward = f'(x_k) * (g_k - sum_j g_j y_j) / S                          (plain)
//            = f'(x_k) * (g_k / f(x_k) - (sum_j g_j) / S)                   (log)
// where f' is the series of order n-1 (csrc/taylor_softmax.cu:24-33 series, :50-86 forward,
// :140-192 backward). The tensor is seen as (n_size, dimsize, m_size) around the chosen dimension.
// Cross entropy on the log form (what TaylorCrossEntropyLossV3 composes from the Function and
// F.nll_loss, pytorch_loss/taylor_softmax.py:175-198) in one kernel per direction:
//   loss_i = log S - log f(x_y),   grad_k = gout_i * (f'(x_k) / S - [k == y] f'(x_k) / f(x_k)).
#pragma once
#include "plh_common.hpp"

namespace plh {

struct TaylorParams {
    int64_t P;          // n_size * m_size
    int64_t m_size;
    int C;              // dimsize
    int order;          // n
    int use_log;
    int64_t ignore;     // cross entropy only
    unsigned xcd_run;
    // cross entropy of long rows: one float per row, the row's S. The reduced forward writes it beside its partial sums
    // and the backward reads it instead of sweeping the row for it (taylor_ce_bwd_flat_sums); see taylor_sums_apply
    float *sums = nullptr;
};

// Rows (m_size 1) whose backward is one elementwise pass over the flattened tensor with S kept (beyond what a wavefront's
// registers hold the other backward reads its row twice, S and then the gradient): row_backward_is_elementwise.
// Channel planes (NCHW) that do not start on 128-byte lines, fp32, 4096 pixels or more, up to 24 channels or 33 .. 256
// (odd crops: the forward is the per-image form of the register-resident kernel, or the split kernel in tiles per image,
// and leaves S per pixel; the backward walks every plane in its own lines, taylor_ce_bwd_planes): orders 2 and 4, which
// those kernels are compiled for.
inline bool taylor_sums_apply(size_t elem_bytes, int64_t dimsize, int64_t m_size) {
    if (m_size == 1) return row_backward_is_elementwise(elem_bytes, dimsize, 1024);
    if (elem_bytes != 4 || dimsize < 1 || m_size < 4096) return false;
    // 257 .. 512 channels on any plane: the recomputing kernels keep a pixel's slice in two halves per wavefront there
    if (dimsize > kMaxSplitChannels && dimsize <= kMaxDeepChannels) return true;
    if ((m_size * 4) % 128 == 0) return false;
    return image_form_pays<float>((int)dimsize, m_size) || (dimsize > kMaxRegsChannels && dimsize <= kMaxSplitChannels);
}

// 1 / i! for i = 0..33; 34! does not fit fp32 (the reference's running factorial becomes inf there and
// its terms vanish, which the zero past the end of the table reproduces).
struct InvFactorials {
    float v[36];
    constexpr InvFactorials() : v{} {
        double f = 1.0;
        for (int i = 0; i < 36; ++i) {
            if (i > 1) f *= (double)i;
            v[i] = (i <= 33) ? (float)(1.0 / f) : 0.f;
        }
    }
};
__device__ constexpr InvFactorials kInvFact{};

// f of order n (>= 2) and, as a by-product, of order n-1 (its derivative). The orders in common use
// (2, the modules' default, and 4; `order` is uniform, so the branch is scalar) are evaluated in nested form.
// The kernels that keep a slice or a row in registers are compiled for these two orders only (taylor_pair24, the
// order a compile-time constant of a body that is chosen once per launch): every evaluation is inlined into their
// unrolled sweeps, and a third, general form there made up a third of the library's code for orders nobody trains
// with; higher orders take the kernels that walk the slice
// (taylor_group, the block-per-row forms), which evaluate term by term upwards like the reference's
// recurrence (csrc/taylor_softmax.cu:24-33).
template <int ORD>
__device__ __forceinline__ void taylor_pair24(float x, float &f, float &df) {
    static_assert(ORD == 2 || ORD == 4, "the register-resident kernels are compiled for orders 2 and 4");
    if constexpr (ORD == 2) {
        df = 1.f + x;
        f = __builtin_fmaf(x * x, 0.5f, df);
    } else {
        const float x2 = x * x;
        df = __builtin_fmaf(x, __builtin_fmaf(x, __builtin_fmaf(x, 1.f / 6.f, 0.5f), 1.f), 1.f);
        f = __builtin_fmaf(x2 * x2, 1.f / 24.f, df);
    }
}

__device__ __forceinline__ void taylor_pair(float x, int order, float &f, float &df) {
    if (order == 2) {
        taylor_pair24<2>(x, f, df);
        return;
    }
    if (order == 4) {
        taylor_pair24<4>(x, f, df);
        return;
    }
    float res = 1.f + x, prev = 1.f, mid = x;
    for (int i = 2; i <= order; ++i) {
        prev = res;
        mid *= x;
        res = __builtin_fmaf(mid, kInvFact.v[i < 35 ? i : 35], res);
    }
    f = res;
    df = prev;
}

// ORD = 2 or 4: that order inlined; 0: the order at run time.
template <int ORD>
__device__ __forceinline__ void taylor_pair_as(float x, int order, float &f, float &df) {
    if constexpr (ORD == 0) taylor_pair(x, order, f, df);
    else taylor_pair24<ORD>(x, f, df);
}

// ---------------------------------------------------------------- regs ----

template <class T, int CP, int V, int Form>
__global__ __launch_bounds__(kRegsBlock) void taylor_fwd_regs(const T *__restrict__ x, T *__restrict__ out,
                                                             const TaylorParams p) {
    // the order is uniform over the grid: the body is compiled once per order and chosen here, so that no
    // evaluation of the series carries a test of its own
    auto run = [&](auto order_tag, auto log_tag) {
    constexpr int ORD = decltype(order_tag)::value;
    constexpr bool LOG = decltype(log_tag)::value;
    const PixelRef<V, Form> at(p.P, p.m_size, p.C, p.xcd_run);
    if (!at.live) return;
    typename Pack<T, V>::Raw raw[CP];
    at.load_slice(x, p.C, p.m_size, raw);
    // a pixel's results replace its inputs in the slice as soon as they are formed (one pixel at a time
    // for fp32, two for 16-bit elements, which share a dword): no second array
    using PK = Pack<T, V>;
#pragma unroll
    for (int k0 = 0; k0 < V; k0 += PK::kStep) {
        float y[CP][PK::kStep];
#pragma unroll
        for (int kk = 0; kk < PK::kStep; ++kk) {
            const int k = k0 + kk;
            float s = 0.f;
#pragma unroll
            for (int j = 0; j < CP; ++j)
                if (chan_ok<CP>(j, p.C)) {
                    float f, df;
                    taylor_pair24<ORD>(PK::get(raw[j], k), f, df);
                    y[j][kk] = f;
                    s += f;
                }
            const float inv = 1.f / s, ls = logf(s);
#pragma unroll
            for (int j = 0; j < CP; ++j)
                if (chan_ok<CP>(j, p.C)) y[j][kk] = LOG ? logf(y[j][kk]) - ls : y[j][kk] * inv;
        }
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (chan_ok<CP>(j, p.C)) PK::set(raw[j], k0 / PK::kStep, y[j]);
    }
    at.store_slice(out, p.C, p.m_size, raw);
    };
    if (p.order == 2 && p.use_log) run(std::integral_constant<int, 2>(), std::true_type());
    else if (p.order == 2) run(std::integral_constant<int, 2>(), std::false_type());
    else if (p.use_log) run(std::integral_constant<int, 4>(), std::true_type());
    else run(std::integral_constant<int, 4>(), std::false_type());
}

template <class T, int CP, int V, int Form>
__global__ __launch_bounds__(kRegsBlock) void taylor_bwd_regs(const T *__restrict__ g, const T *__restrict__ x,
                                                             T *__restrict__ gx, const TaylorParams p) {
    // the order is uniform over the grid: the body is compiled once per order and chosen here, so that no
    // evaluation of the series carries a test of its own
    auto run = [&](auto order_tag, auto log_tag) {
    constexpr int ORD = decltype(order_tag)::value;
    constexpr bool LOG = decltype(log_tag)::value;
    const PixelRef<V, Form> at(p.P, p.m_size, p.C, p.xcd_run);
    if (!at.live) return;
    typename Pack<T, V>::Raw raw[CP], graw[CP];
    at.load_slice(x, p.C, p.m_size, raw);
    at.load_slice(g, p.C, p.m_size, graw);
    // the series is cheap: it is evaluated again in the second sweep rather than kept in registers,
    // and the second sweep goes channel by channel so that only one packed result is live at a time
    float inv[V], mid[V];
#pragma unroll
    for (int k = 0; k < V; ++k) {
        float s = 0.f, dot = 0.f;
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (chan_ok<CP>(j, p.C)) {
                float f, df;
                taylor_pair24<ORD>(Pack<T, V>::get(raw[j], k), f, df);
                const float gj = Pack<T, V>::get(graw[j], k);
                s += f;
                dot += LOG ? gj : f * gj;
            }
        inv[k] = 1.f / s;
        mid[k] = LOG ? dot * inv[k] : dot * inv[k] * inv[k];     // csrc/taylor_softmax.cu:163-173
    }
#pragma unroll
    for (int j = 0; j < CP; ++j)
        if (chan_ok<CP>(j, p.C)) {
            forget_origin(raw[j]);
            forget_origin(graw[j]);
        }
#pragma unroll
    for (int j = 0; j < CP; ++j)
        if (chan_ok<CP>(j, p.C)) {
            float r[V];
#pragma unroll
            for (int k = 0; k < V; ++k) {
                float f, df;
                taylor_pair24<ORD>(Pack<T, V>::get(raw[j], k), f, df);
                const float gj = Pack<T, V>::get(graw[j], k);
                r[k] = LOG ? df * (__builtin_amdgcn_rcpf(f) * gj - mid[k]) : df * (inv[k] * gj - mid[k]);
            }
            raw[j] = Pack<T, V>::put(r);
            forget_origin(raw[j]);      // packed here, channel by channel: nothing of the sweep waits for the stores
        }
    at.store_slice(gx, p.C, p.m_size, raw);
    };
    if (p.order == 2 && p.use_log) run(std::integral_constant<int, 2>(), std::true_type());
    else if (p.order == 2) run(std::integral_constant<int, 2>(), std::false_type());
    else if (p.use_log) run(std::integral_constant<int, 4>(), std::true_type());
    else run(std::integral_constant<int, 4>(), std::false_type());
}

// Cross entropy on the log form: loss per pixel (fp32), and its gradient with the upstream folded in.
template <class T, int CP, int V, int Form>
__global__ __launch_bounds__(kRegsBlock) void taylor_ce_fwd_regs(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                                float *__restrict__ loss, Partials part,
                                                                const TaylorParams p) {
    const bool Reduce = part.sum != nullptr;
    __shared__ float red[4];
    // the order is uniform over the grid: the body is compiled once per order and chosen here, so that no
    // evaluation of the series carries a test of its own
    auto run = [&](auto order_tag) {
    constexpr int ORD = decltype(order_tag)::value;
    const PixelRef<V, Form> at(p.P, p.m_size, p.C, p.xcd_run);
    if (!Reduce && !at.live) return;
    // labels (and the upstream gradient) first: in the rows form the slice arrives through LDS behind a wait
    int64_t lb[V];
    at.labels(lab, p.ignore, lb);
    typename Pack<T, V>::Raw raw[CP];
    at.load_slice(x, p.C, p.m_size, raw);
    float out[V], sums[V];
    float mine = 0.f;
    int cnt = 0;
#pragma unroll
    for (int k = 0; k < V; ++k) {
        bool ign;
        const int tgt = narrow_label(lb[k], p.ignore, p.C, ign);
        float s = 0.f, f_y = 1.f;
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (chan_ok<CP>(j, p.C)) {
                float f, df;
                taylor_pair24<ORD>(Pack<T, V>::get(raw[j], k), f, df);
                s += f;
                f_y = (tgt == j) ? f : f_y;
            }
        const bool valid = at.live && !ign && tgt >= 0;
        out[k] = valid ? logf(s) - logf(f_y) : 0.f;
        sums[k] = s;
        mine += out[k];
        cnt += (at.live && !ign) ? 1 : 0;
    }
    if (at.live && loss) {
        if (loss == p.sums) at.store_f32(loss, sums);      // the slot takes the pixels' S (TaylorParams::sums)
        else at.store_f32(loss, out);
    }
    if (Reduce) {
        const float bs = block_sum_256(mine, red);
        const float bc = block_sum_256((float)cnt, red);
        if (threadIdx.x == 0) {
            part.sum[blockIdx.x] = bs;
            part.cnt[blockIdx.x] = (int)bc;
        }
    }
    };
    if (p.order == 2) run(std::integral_constant<int, 2>());
    else run(std::integral_constant<int, 4>());
}

template <class T, int CP, int V, int Form>
__global__ __launch_bounds__(kRegsBlock) void taylor_ce_bwd_regs(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                                const Upstream up, T *__restrict__ gx,
                                                                const TaylorParams p) {
    // the order is uniform over the grid: the body is compiled once per order and chosen here, so that no
    // evaluation of the series carries a test of its own
    auto run = [&](auto order_tag) {
    constexpr int ORD = decltype(order_tag)::value;
    const PixelRef<V, Form> at(p.P, p.m_size, p.C, p.xcd_run);
    if (!at.live) return;
    // labels and the upstream gradient before the slice, except in the one-pixel-per-lane form on 16-bit elements
    // (see lsr_bwd_regs)
    constexpr bool kLabelsFirst = !(sizeof(T) == 2 && V == 1);
    int64_t lb[V];
    float go[V];
    typename Pack<T, V>::Raw raw[CP];
    if constexpr (kLabelsFirst) {
        at.labels(lab, p.ignore, lb);
        at.upstream(up, go);
    }
    at.load_slice(x, p.C, p.m_size, raw);
    if constexpr (!kLabelsFirst) {
        at.labels(lab, p.ignore, lb);
        at.upstream(up, go);
    }
    // first per pixel (sum of the series, the target's term), then channel by channel so that only one
    // packed result is live at a time
    unsigned keep[V];
    int tgt[V];
    float scale[V], hot[V];
#pragma unroll
    for (int k = 0; k < V; ++k) {
        bool ign;
        tgt[k] = narrow_label(lb[k], p.ignore, p.C, ign);
        keep[k] = (ign || tgt[k] < 0) ? 0u : 0xFFFFFFFFu;
        float s = 0.f, f_y = 1.f;
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (chan_ok<CP>(j, p.C)) {
                float f, df;
                taylor_pair24<ORD>(Pack<T, V>::get(raw[j], k), f, df);
                s += f;
                f_y = (tgt[k] == j) ? f : f_y;
            }
        scale[k] = go[k] * __builtin_amdgcn_rcpf(s);
        hot[k] = scale[k] - go[k] / f_y;                           // per pixel: what the target channel takes
        asm("" : "+v"(hot[k]));
    }
    const typename Pack<T, V>::Raw mask = Pack<T, V>::mask(keep);
#pragma unroll
    for (int j = 0; j < CP; ++j)
        if (chan_ok<CP>(j, p.C)) forget_origin(raw[j]);
#pragma unroll
    for (int j = 0; j < CP; ++j)
        if (chan_ok<CP>(j, p.C)) {
            float r[V];
#pragma unroll
            for (int k = 0; k < V; ++k) {
                float f, df;
                taylor_pair24<ORD>(Pack<T, V>::get(raw[j], k), f, df);
                r[k] = df * ((tgt[k] == j) ? hot[k] : scale[k]);
            }
            raw[j] = Pack<T, V>::put(r) & mask;
            forget_origin(raw[j]);      // packed here, channel by channel: nothing of the sweep waits for the stores
        }
    at.store_slice(gx, p.C, p.m_size, raw);
    };
    if (p.order == 2) run(std::integral_constant<int, 2>());
    else run(std::integral_constant<int, 4>());
}

// --------------------------------------------------------------- split ----
// Cross entropy for 33..256 channels in NCHW (SplitSlice). The series needs no maximum, so the parts of
// a pixel are just each wavefront's sum of the series and the target's term if it is held there.

template <class T, int KW, int V, bool PerImage = false>
__global__ __launch_bounds__(kSplitBlock) void taylor_ce_fwd_split(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                                  float *__restrict__ loss, Partials part,
                                                                  const TaylorParams p) {
    const bool Reduce = part.sum != nullptr;
    __shared__ float parts[2][kSplitWaves][kWave * V];
    // the order is uniform over the grid: the body is compiled once per order and chosen here, so that no
    // evaluation of the series carries a test of its own
    auto run = [&](auto order_tag) {
    constexpr int ORD = decltype(order_tag)::value;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const SplitSlice<T, V, KW, PerImage> at(p.P, p.m_size, p.C, p.xcd_run);
    int64_t lb[V];
    at.labels(lab, p.ignore, lb);
    if (at.here > 0) {                                  // wave-uniform
        typename Pack<T, V>::Raw raw[KW];
        at.load(x, p.C, p.m_size, raw);
#pragma unroll
        for (int k = 0; k < V; ++k) {
            bool ign;
            const int rel = narrow_label(lb[k], p.ignore, p.C, ign) - at.first;
            float s = 0.f, f_y = 0.f;
#pragma unroll
            for (int i = 0; i < KW; ++i) {
                float f, df;
                taylor_pair24<ORD>(Pack<T, V>::get(raw[i], k), f, df);
                s += (i < at.here) ? f : 0.f;
                f_y = (rel == i) ? f : f_y;
            }
            parts[0][wave][lane * V + k] = s;
            parts[1][wave][lane * V + k] = f_y;
        }
    }
    __syncthreads();
    if (wave >= V) return;                              // wavefront k finishes pixel k of every lane 
    const int used = (p.C + KW - 1) / KW;
    bool ign;
    PLH_SPLIT_MY_LABEL(my_lb, lb, wave, V)
    const int tgt = narrow_label(my_lb, p.ignore, p.C, ign);
    float s = 0.f, f_y = 0.f;
    for (int w = 0; w < used; ++w) {
        s += parts[0][w][lane * V + wave];
        f_y += parts[1][w][lane * V + wave];
    }
    const bool here = at.live && wave < at.nv;
    const bool valid = here && !ign && tgt >= 0;
    const float out = valid ? logf(s) - logf(f_y) : 0.f;
    if (here && loss) loss[at.pix + wave] = (loss == p.sums) ? s : out;       // the slot takes the pixels' S (TaylorParams::sums)
    if (Reduce) split_block_partials<V>(out, here && !ign, wave, lane, part);
    };
    if (p.order == 2) run(std::integral_constant<int, 2>());
    else run(std::integral_constant<int, 4>());
}

template <class T, int KW, int V, bool PerImage = false>
__global__ __launch_bounds__(kSplitBlock) void taylor_ce_bwd_split(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                                  const Upstream up, T *__restrict__ gx,
                                                                  const TaylorParams p) {
    __shared__ float parts[2][kSplitWaves][kWave * V];
    // the order is uniform over the grid: the body is compiled once per order and chosen here, so that no
    // evaluation of the series carries a test of its own
    auto run = [&](auto order_tag) {
    constexpr int ORD = decltype(order_tag)::value;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const SplitSlice<T, V, KW, PerImage> at(p.P, p.m_size, p.C, p.xcd_run);
    typename Pack<T, V>::Raw raw[KW];
    int64_t lb[V];
    float go[V];
    int rel[V];
    unsigned keep[V];
    if (at.here > 0) {                                  // wave-uniform
        at.load(x, p.C, p.m_size, raw);
        at.labels(lab, p.ignore, lb);
        at.upstream(up, go);
#pragma unroll
        for (int k = 0; k < V; ++k) {
            bool ign;
            const int tgt = narrow_label(lb[k], p.ignore, p.C, ign);
            rel[k] = tgt - at.first;
            keep[k] = (ign || tgt < 0) ? 0u : 0xFFFFFFFFu;
            float s = 0.f, f_y = 0.f;
#pragma unroll
            for (int i = 0; i < KW; ++i) {
                float f, df;
                taylor_pair24<ORD>(Pack<T, V>::get(raw[i], k), f, df);
                s += (i < at.here) ? f : 0.f;
                f_y = (rel[k] == i) ? f : f_y;
            }
            parts[0][wave][lane * V + k] = s;
            parts[1][wave][lane * V + k] = f_y;
        }
    }
    __syncthreads();
    if (at.here == 0 || !at.live) return;
    const int used = (p.C + KW - 1) / KW;
    float scale[V], hot[V];
#pragma unroll
    for (int k = 0; k < V; ++k) {
        float s = 0.f, f_y = 0.f;
        for (int w = 0; w < used; ++w) {
            s += parts[0][w][lane * V + k];
            f_y += parts[1][w][lane * V + k];
        }
        scale[k] = go[k] * __builtin_amdgcn_rcpf(s);
        hot[k] = scale[k] - go[k] / f_y;                           // per pixel: what the target channel takes
        asm("" : "+v"(hot[k]));
    }
    const typename Pack<T, V>::Raw mask = Pack<T, V>::mask(keep);
#pragma unroll
    for (int i = 0; i < KW; ++i) forget_origin(raw[i]);
#pragma unroll
    for (int i = 0; i < KW; ++i) {
        float r[V];
#pragma unroll
        for (int k = 0; k < V; ++k) {
            float f, df;
            taylor_pair24<ORD>(Pack<T, V>::get(raw[i], k), f, df);
            r[k] = df * ((rel[k] == i) ? hot[k] : scale[k]);
        }
        raw[i] = Pack<T, V>::put(r) & mask;
    }
    at.store(gx, p.m_size, raw);
    };
    if (p.order == 2) run(std::integral_constant<int, 2>());
    else run(std::integral_constant<int, 4>());
}

// The softmax / log-softmax themselves for 33..256 channels in NCHW (SplitSlice): the parts of a pixel are each
// wavefront's sum of the series and, in the backward, of its products with the upstream gradient; every wavefront
// then finishes its own channels. The backward holds two slices (logits and upstream) per wavefront.
template <class T, int KW, int V, bool PerImage = false>
__global__ __launch_bounds__(kSplitBlock) void taylor_sm_fwd_split(const T *__restrict__ x, T *__restrict__ out,
                                                                  const TaylorParams p) {
    __shared__ float parts[kSplitWaves][kWave * V];
    // the order is uniform over the grid: the body is compiled once per order and chosen here, so that no
    // evaluation of the series carries a test of its own
    auto run = [&](auto order_tag, auto log_tag) {
    constexpr int ORD = decltype(order_tag)::value;
    constexpr bool LOG = decltype(log_tag)::value;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const SplitSlice<T, V, KW, PerImage> at(p.P, p.m_size, p.C, p.xcd_run);
    using PK = Pack<T, V>;
    typename PK::Raw raw[KW];
    if (at.here > 0) {                                  // wave-uniform
        at.load(x, p.C, p.m_size, raw);
#pragma unroll
        for (int k = 0; k < V; ++k) {
            float s = 0.f;
#pragma unroll
            for (int i = 0; i < KW; ++i) {
                float f, df;
                taylor_pair24<ORD>(PK::get(raw[i], k), f, df);
                s += (i < at.here) ? f : 0.f;
            }
            parts[wave][lane * V + k] = s;
        }
    }
    __syncthreads();
    if (at.here == 0 || !at.live) return;
    const int used = (p.C + KW - 1) / KW;
    float inv[V], ls[V];
#pragma unroll
    for (int k = 0; k < V; ++k) {
        float s = 0.f;
        for (int w = 0; w < used; ++w) s += parts[w][lane * V + k];
        inv[k] = 1.f / s;
        ls[k] = logf(s);
    }
#pragma unroll
    for (int i = 0; i < KW; ++i) forget_origin(raw[i]);
#pragma unroll
    for (int i = 0; i < KW; ++i) {
        float r[V];
#pragma unroll
        for (int k = 0; k < V; ++k) {
            float f, df;
            taylor_pair24<ORD>(PK::get(raw[i], k), f, df);
            r[k] = LOG ? logf(f) - ls[k] : f * inv[k];
        }
        raw[i] = PK::put(r);
    }
    at.store(out, p.m_size, raw);
    };
    if (p.order == 2 && p.use_log) run(std::integral_constant<int, 2>(), std::true_type());
    else if (p.order == 2) run(std::integral_constant<int, 2>(), std::false_type());
    else if (p.use_log) run(std::integral_constant<int, 4>(), std::true_type());
    else run(std::integral_constant<int, 4>(), std::false_type());
}

template <class T, int KW, int V, bool PerImage = false>
__global__ __launch_bounds__(kSplitBlock) void taylor_sm_bwd_split(const T *__restrict__ g, const T *__restrict__ x,
                                                                  T *__restrict__ gx, const TaylorParams p) {
    __shared__ float parts[2][kSplitWaves][kWave * V];
    // the order is uniform over the grid: the body is compiled once per order and chosen here, so that no
    // evaluation of the series carries a test of its own
    auto run = [&](auto order_tag, auto log_tag) {
    constexpr int ORD = decltype(order_tag)::value;
    constexpr bool LOG = decltype(log_tag)::value;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const SplitSlice<T, V, KW, PerImage> at(p.P, p.m_size, p.C, p.xcd_run);
    using PK = Pack<T, V>;
    typename PK::Raw raw[KW], graw[KW];
    if (at.here > 0) {                                  // wave-uniform
        at.load(x, p.C, p.m_size, raw);
        at.load(g, p.C, p.m_size, graw);
#pragma unroll
        for (int k = 0; k < V; ++k) {
            float s = 0.f, dot = 0.f;
#pragma unroll
            for (int i = 0; i < KW; ++i) {
                float f, df;
                taylor_pair24<ORD>(PK::get(raw[i], k), f, df);
                const float gj = PK::get(graw[i], k);
                s += (i < at.here) ? f : 0.f;
                dot += (i < at.here) ? (LOG ? gj : f * gj) : 0.f;
            }
            parts[0][wave][lane * V + k] = s;
            parts[1][wave][lane * V + k] = dot;
        }
    }
    __syncthreads();
    if (at.here == 0 || !at.live) return;
    const int used = (p.C + KW - 1) / KW;
    float inv[V], mid[V];
#pragma unroll
    for (int k = 0; k < V; ++k) {
        float s = 0.f, dot = 0.f;
        for (int w = 0; w < used; ++w) {
            s += parts[0][w][lane * V + k];
            dot += parts[1][w][lane * V + k];
        }
        inv[k] = 1.f / s;
        mid[k] = LOG ? dot * inv[k] : dot * inv[k] * inv[k];     // csrc/taylor_softmax.cu:163-173
    }
#pragma unroll
    for (int i = 0; i < KW; ++i) {
        forget_origin(raw[i]);
        forget_origin(graw[i]);
    }
#pragma unroll
    for (int i = 0; i < KW; ++i) {
        float r[V];
#pragma unroll
        for (int k = 0; k < V; ++k) {
            float f, df;
            taylor_pair24<ORD>(PK::get(raw[i], k), f, df);
            const float gj = PK::get(graw[i], k);
            r[k] = LOG ? df * (__builtin_amdgcn_rcpf(f) * gj - mid[k]) : df * (inv[k] * gj - mid[k]);
        }
        raw[i] = PK::put(r);
    }
    at.store(gx, p.m_size, raw);
    };
    if (p.order == 2 && p.use_log) run(std::integral_constant<int, 2>(), std::true_type());
    else if (p.order == 2) run(std::integral_constant<int, 2>(), std::false_type());
    else if (p.use_log) run(std::integral_constant<int, 4>(), std::true_type());
    else run(std::integral_constant<int, 4>(), std::false_type());
}

// --------------------------------------------------------------- group ----
// Any dimsize: G lanes share one slice and stride over it (launched with G = 1: a lane per slice, for what
// no other shape takes). The series is re-evaluated in each sweep; re-reads hit cache.

enum TaylorKind { kTaylorFwd = 0, kTaylorBwd = 1, kTaylorCeFwd = 2, kTaylorCeBwd = 3 };

template <class T, int G, int Kind>
__global__ __launch_bounds__(256) void taylor_group(const T *__restrict__ x, const T *__restrict__ g,
                                                    const int64_t *__restrict__ lab, const Upstream up,
                                                    T *__restrict__ out, float *__restrict__ loss, Partials part,
                                                    const TaylorParams p) {
    const bool Reduce = part.sum != nullptr;
    constexpr int kPix = 256 / G;
    __shared__ float red[4];
    const int sub = threadIdx.x % G, grp = threadIdx.x / G;
    float mine = 0.f, cnt = 0.f;
    const int64_t rounds = ceil_div_dev(p.P, (int64_t)gridDim.x * kPix);
    for (int64_t rd = 0; rd < rounds; ++rd) {
        const int64_t pix = (rd * gridDim.x + blockIdx.x) * kPix + grp;
        const bool live = pix < p.P;
        const int64_t pc = live ? pix : 0;
        const int64_t n = pc / p.m_size;
        const int64_t base = pc + n * (int64_t)(p.C - 1) * p.m_size;
        const T *xs = x + base;
        float s = 0.f, dot = 0.f;
#pragma unroll kGroupUnroll<G>
        for (int j = sub; j < p.C; j += G) {
            float f, df;
            taylor_pair(load_one(xs + (int64_t)j * p.m_size), p.order, f, df);
            s += f;
            if constexpr (Kind == kTaylorBwd) {
                const float gj = load_one(g + base + (int64_t)j * p.m_size);
                dot += p.use_log ? gj : f * gj;
            }
        }
        s = group_reduce<G>(s, OpSum());
        if constexpr (Kind == kTaylorBwd) dot = group_reduce<G>(dot, OpSum());
        const float inv = 1.f / s;
        if constexpr (Kind == kTaylorFwd) {
            const float ls = logf(s);
            if (live)
#pragma unroll kGroupUnroll<G>
                for (int j = sub; j < p.C; j += G) {
                    float f, df;
                    taylor_pair(load_one(xs + (int64_t)j * p.m_size), p.order, f, df);
                    store_one(out + base + (int64_t)j * p.m_size, p.use_log ? logf(f) - ls : f * inv);
                }
        } else if constexpr (Kind == kTaylorBwd) {
            const float mid = p.use_log ? dot * inv : dot * inv * inv;
            if (live)
#pragma unroll kGroupUnroll<G>
                for (int j = sub; j < p.C; j += G) {
                    float f, df;
                    taylor_pair(load_one(xs + (int64_t)j * p.m_size), p.order, f, df);
                    const float gj = load_one(g + base + (int64_t)j * p.m_size);
                    store_one(out + base + (int64_t)j * p.m_size,
                              p.use_log ? df / f * gj - mid * df : df * inv * gj - df * mid);
                }
        } else {
            const int64_t lb = lab[pc];
            const bool has_y = lb != p.ignore && lb >= 0 && lb < p.C;
            if constexpr (Kind == kTaylorCeFwd) {
                float f_y = 1.f, df;
                if (has_y) taylor_pair(load_one(xs + lb * p.m_size), p.order, f_y, df);
                const float v = (live && has_y) ? logf(s) - logf(f_y) : 0.f;
                if (live && sub == 0) {
                    if (loss) loss[pix] = v;
                    mine += v;
                    cnt += (lb != p.ignore) ? 1.f : 0.f;
                }
            } else {
                float go[1];
                load_upstream<1>(up, pc, go);
                const float gk = has_y ? go[0] : 0.f;
                // f' times one of two factors per pixel: the division by f(x_y) happens once, not per channel
                float f_y = 1.f, df_y;
                if (has_y) taylor_pair(load_one(xs + lb * p.m_size), p.order, f_y, df_y);
                const float cold = inv * gk, hot = cold - gk / f_y;
                if (live)
#pragma unroll kGroupUnroll<G>
                    for (int j = sub; j < p.C; j += G) {
                        float f, df;
                        taylor_pair(load_one(xs + (int64_t)j * p.m_size), p.order, f, df);
                        store_one(out + base + (int64_t)j * p.m_size, has_y ? df * ((lb == j) ? hot : cold) : 0.f);
                    }
            }
        }
    }
    if (Reduce) {
        const float bs = block_sum_256(mine, red);
        const float bc = block_sum_256(cnt, red);
        if (threadIdx.x == 0) {
            part.sum[blockIdx.x] = bs;
            part.cnt[blockIdx.x] = (int)bc;
        }
    }
}

// ------------------------------------------------- wavefront per row, in registers ----
// (N, C) inputs along dim 1 with 33..2048 channels: the row (and, for the softmax backward, the row of
// upstream gradients) sits in the wavefront's registers, so both sweeps read HBM once. Same arithmetic as
// the group kernel.

template <class T, int NI, int LP, int Kind, int G, bool Cached = false>
__global__ __launch_bounds__(256) void taylor_wrow(const T *__restrict__ x, const T *__restrict__ g,
                                                   const int64_t *__restrict__ lab, const Upstream up,
                                                   T *__restrict__ out, float *__restrict__ loss, Partials part,
                                                   const TaylorParams p) {
    const bool Reduce = part.sum != nullptr;
    __shared__ float red[4];
    // the order is uniform over the grid: the body is compiled once per order and chosen here, so that no
    // evaluation of the series carries a test of its own
    auto run = [&](auto order_tag, auto log_tag) {
    constexpr int ORD = decltype(order_tag)::value;
    constexpr bool LOG = decltype(log_tag)::value;
    constexpr int L = WaveRow<T, NI, LP, G>::L;
    using Span = WaveRowSpan<T, L, G, NI>;
    T *tile = Span::tile();
    const WaveRowAt<G> at;
    const int lane = at.sub;
    float mine = 0.f, cnt = 0.f;
    for (int64_t r0 = at.start; r0 < p.P; r0 += at.stride) {   // wave-uniform
        const bool live = r0 + at.grp < p.P;
        const int64_t row = live ? r0 + at.grp : p.P - 1;
        const T *xs = x + row * p.C;
        WaveRow<T, NI, LP, G> r;
        r.load(xs, p.C, lane);
        WaveRow<T, (Kind == kTaylorBwd) ? NI : 1, LP, G> rg;
        if constexpr (Kind == kTaylorBwd) rg.load(g + row * p.C, p.C, lane);
        float s = 0.f, dot = 0.f;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const bool ok = (lane + G * i) * L < p.C;           // elements beyond the row hold -inf
#pragma unroll
            for (int l = 0; l < L; ++l) {
                float f, df;
                taylor_pair24<ORD>(r.v[i][l], f, df);
                s += ok ? f : 0.f;
                if constexpr (Kind == kTaylorBwd) {
                    const float gj = rg.v[i][l];
                    dot += ok ? (LOG ? gj : f * gj) : 0.f;
                }
            }
        }
        s = group_reduce<G>(s, OpSum());
        if constexpr (Kind == kTaylorBwd) dot = group_reduce<G>(dot, OpSum());
        const float inv = 1.f / s;
        if constexpr (Kind == kTaylorCeFwd) {
            if (lane == 0 && live) {
                const int64_t lb = lab[row];
                const bool has_y = lb != p.ignore && lb >= 0 && lb < p.C;
                float f_y = 1.f, df;
                if (has_y) taylor_pair24<ORD>(load_one(xs + lb), f_y, df);
                const float v = has_y ? logf(s) - logf(f_y) : 0.f;
                if (loss) loss[row] = (loss == p.sums) ? s : v;     // the slot takes the rows' S (TaylorParams::sums)
                mine += v;
                cnt += (lb != p.ignore) ? 1.f : 0.f;
            }
        } else {
            const float ls = logf(s);
            const float mid = LOG ? dot * inv : dot * inv * inv;
            int tgt = -1;
            float cold = 0.f, hot = 0.f;        // cross entropy: f' times one of these, see taylor_group
            if constexpr (Kind == kTaylorCeBwd) {
                const int64_t lb = lab[row];
                float go[1];
                load_upstream<1>(up, row, go);
                if (lb != p.ignore && lb >= 0 && lb < p.C) {
                    tgt = (int)lb;
                    float f_y, df_y;
                    taylor_pair24<ORD>(load_one(xs + lb), f_y, df_y);
                    cold = inv * go[0];
                    hot = cold - go[0] / f_y;
                }
            }
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                const int e0 = (lane + G * i) * L;
                float o[L];
#pragma unroll
                for (int l = 0; l < L; ++l) {
                    float f, df;
                    taylor_pair24<ORD>(r.v[i][l], f, df);
                    if constexpr (Kind == kTaylorFwd) {
                        o[l] = LOG ? logf(f) - ls : f * inv;
                    } else if constexpr (Kind == kTaylorBwd) {
                        const float gj = rg.v[i][l];
                        o[l] = LOG ? df / f * gj - mid * df : df * inv * gj - df * mid;
                    } else {
                        o[l] = (tgt >= 0) ? df * ((e0 + l == tgt) ? hot : cold) : 0.f;
                    }
                }
                if (e0 < p.C && live) {
                    if constexpr (Span::kUse) Span::stage(tile, p.C, at.grp, e0, o);
                    else RowPiece<T, L>::template store<Cached>(out + row * p.C + e0, o);
                }
            }
            if constexpr (Span::kUse) {
                const int64_t left = p.P - r0;
                Span::flush(tile, out + r0 * p.C, left < Span::kRows ? (int)left : Span::kRows, p.C);
            }
        }
    }
    if (Reduce) {
        const float bs = block_sum_256(mine, red);
        const float bc = block_sum_256(cnt, red);
        if (threadIdx.x == 0) {
            part.sum[blockIdx.x] = bs;
            part.cnt[blockIdx.x] = (int)bc;
        }
    }
    };
    // the logarithmic form is a matter of the softmax kinds only
    if constexpr (Kind == kTaylorFwd || Kind == kTaylorBwd) {
        if (p.order == 2 && p.use_log) run(std::integral_constant<int, 2>(), std::true_type());
        else if (p.order == 2) run(std::integral_constant<int, 2>(), std::false_type());
        else if (p.use_log) run(std::integral_constant<int, 4>(), std::true_type());
        else run(std::integral_constant<int, 4>(), std::false_type());
    } else {
        if (p.order == 2) run(std::integral_constant<int, 2>(), std::false_type());
        else run(std::integral_constant<int, 4>(), std::false_type());
    }
}

// ------------------------------------------------------- a block per row ----
// Taylor cross entropy on (N, C) inputs with rows of more than 2048 channels: a 1024-thread block per row
// at a time, 16-byte chunks, four loads in flight; the backward sweeps the row a second time (from cache
// for all but the longest rows) to write the gradient.

// Taylor softmax / log-softmax and their backward on such rows. The backward's first sweep walks the row
// of logits and the row of upstream gradients together, element by element unless both can move in chunks.
template <class T, int Kind>
__global__ __launch_bounds__(kRowBlock) void taylor_sm_row(const T *__restrict__ x, const T *__restrict__ g,
                                                           T *__restrict__ out, const TaylorParams p, int vec) {
    static_assert(Kind == kTaylorFwd || Kind == kTaylorBwd, "softmax forms only");
    __shared__ float red[kRowBlock / 64];
    constexpr int L = RowChunk<T>::kLen;
    for (int64_t row = blockIdx.x; row < p.P; row += gridDim.x) {       // block-uniform
        const T *xs = x + row * p.C;
        float s = 0.f, dot = 0.f;
        if constexpr (Kind == kTaylorFwd) {
            row_visit<T>(xs, p.C, vec != 0, [&](float v, int) {
                float f, df;
                taylor_pair(v, p.order, f, df);
                s += f;
            });
        } else {
            const T *gr = g + row * p.C;
            const RowSplit<T> sp(xs, p.C, vec != 0);       // the row of g sits at the same offset from its boundary
            auto term = [&](float v, float gj) {
                float f, df;
                taylor_pair(v, p.order, f, df);
                s += f;
                dot += p.use_log ? gj : f * gj;
            };
            for (int i = threadIdx.x; i < sp.chunks; i += row_threads()) {
                float v[L], gv[L];
                RowChunk<T>::load(xs + sp.head + (int64_t)i * L, v);
                RowChunk<T>::load(gr + sp.head + (int64_t)i * L, gv);
#pragma unroll
                for (int e = 0; e < L; ++e) term(v[e], gv[e]);
            }
            for (int j = threadIdx.x; j < sp.head; j += row_threads()) term(load_one(xs + j), load_one(gr + j));
            for (int j = sp.tail_from + threadIdx.x; j < p.C; j += row_threads()) term(load_one(xs + j), load_one(gr + j));
            dot = row_block_reduce(dot, red, OpSum());
        }
        s = row_block_reduce(s, red, OpSum());
        const float inv = 1.f / s;
        if constexpr (Kind == kTaylorFwd) {
            const float ls = logf(s);
            row_map<T>(xs, out + row * p.C, p.C, vec != 0, [&](float v, int) {
                float f, df;
                taylor_pair(v, p.order, f, df);
                return p.use_log ? logf(f) - ls : f * inv;
            });
        } else {
            const float mid = p.use_log ? dot * inv : dot * inv * inv;
            const T *gr = g + row * p.C;
            row_map<T>(xs, out + row * p.C, p.C, vec != 0, [&](float v, int j) {
                float f, df;
                taylor_pair(v, p.order, f, df);
                const float gj = load_one(gr + j);
                return p.use_log ? df / f * gj - mid * df : df * inv * gj - df * mid;
            });
        }
    }
}

template <class T, int Kind, int ORD = 0>
__global__ __launch_bounds__(kRowBlock) void taylor_ce_row(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                           const Upstream up, T *__restrict__ out,
                                                           float *__restrict__ loss, Partials part,
                                                           const TaylorParams p, int vec) {
    const bool Reduce = part.sum != nullptr;
    static_assert(Kind == kTaylorCeFwd || Kind == kTaylorCeBwd, "cross entropy only");
    __shared__ float red[kRowBlock / 64];
    float mine = 0.f;
    int cnt = 0;
    for (int64_t row = blockIdx.x; row < p.P; row += gridDim.x) {       // block-uniform
        const T *xs = x + row * p.C;
        const int64_t lb = lab[row];
        const bool has_y = lb != p.ignore && lb >= 0 && lb < p.C;
        float s = 0.f;
        row_visit<T>(xs, p.C, (vec & 1) != 0, [&](float v, int) {
            float f, df;
            taylor_pair_as<ORD>(v, p.order, f, df);
            s += f;
        });
        s = row_block_reduce(s, red, OpSum());
        if constexpr (Kind == kTaylorCeFwd) {
            if (threadIdx.x == 0) {
                float f_y = 1.f, df;
                if (has_y) taylor_pair(load_one(xs + lb), p.order, f_y, df);
                const float v = has_y ? logf(s) - logf(f_y) : 0.f;
                if (loss) loss[row] = (vec & 2) ? s : v;       // bit 1: the slot takes the rows' S (TaylorParams::sums)
                mine += v;
                cnt += (lb != p.ignore) ? 1 : 0;
            }
        } else {
            float go[1];
            load_upstream<1>(up, row, go);
            const float gk = has_y ? go[0] : 0.f;
            const float inv = 1.f / s;
            const int tgt = has_y ? (int)lb : -1;
            float f_y = 1.f, df_y;
            if (has_y) taylor_pair(load_one(xs + lb), p.order, f_y, df_y);
            const float cold = inv * gk, hot = cold - gk / f_y;          // see taylor_group
            row_map<T>(xs, out + row * p.C, p.C, (vec & 1) != 0, [&](float v, int j) {
                float f, df;
                taylor_pair_as<ORD>(v, p.order, f, df);
                return has_y ? df * ((j == tgt) ? hot : cold) : 0.f;
            });
        }
    }
    if (Reduce) {
        if (threadIdx.x == 0) {
            part.sum[blockIdx.x] = mine;
            part.cnt[blockIdx.x] = cnt;
        }
    }
}

// Cross-entropy backward of long rows from the sums the forward left (TaylorParams::sums), elementwise over the
// flattened (rows x classes) tensor: a block takes 256 * kFlatChunks consecutive 16-byte chunks wherever rows begin and
// end, so the accesses are those of a copy; a chunk finds its row by one 32-bit division (the block's first element by
// a 64-bit one, block-uniform), and a chunk that straddles two rows goes element by element. The target's own term
// needs f(x_y), which the target element computes from itself. Logits and gradient on 16-byte boundaries, one scalar
// upstream gradient, rows longer than a chunk.
// ORD: the order when it is 2 or 4 (the series inlined without tests), 0 for any other.
template <class T, int ORD>
__global__ __launch_bounds__(256) void taylor_ce_bwd_flat_sums(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                               const Upstream up, T *__restrict__ grad,
                                                               const TaylorParams p, int64_t chunks) {
    constexpr int L = RowChunk<T>::kLen, U = kFlatChunks;
    float gk0 = up.gout ? *up.gout * up.scale : up.scale;
    if (up.divide_by) gk0 = gk0 / (float)(*up.divide_by);
    const int64_t first = (int64_t)blockIdx.x * (256 * U);
    const int64_t row0 = first * L / p.C;                               // block-uniform
    const unsigned col0 = (unsigned)(first * L - row0 * p.C);
    const unsigned C = (unsigned)p.C;
    struct RowTerms { float gk, cold; int tgt; };
    auto row_terms = [&](int64_t r) {
        RowTerms t;
        const int64_t lb = lab[r];
        const bool has_y = lb != p.ignore && lb >= 0 && lb < p.C;
        t.gk = has_y ? gk0 : 0.f;
        t.cold = t.gk / p.sums[r];
        t.tgt = has_y ? (int)lb : -1;
        return t;
    };
    // rows without a target: exact zeros whatever the logits are (taylor_ce_row)
    auto one = [&](float xv, int j, const RowTerms &t) {
        float f, df;
        if constexpr (ORD == 0) taylor_pair(xv, p.order, f, df);
        else taylor_pair24<ORD>(xv, f, df);
        const float k = (j == t.tgt) ? t.cold - t.gk / f : t.cold;
        return t.tgt >= 0 ? df * k : 0.f;
    };
    auto cold_only = [&](float xv, const RowTerms &t) {
        float f, df;
        if constexpr (ORD == 0) taylor_pair(xv, p.order, f, df);
        else taylor_pair24<ORD>(xv, f, df);
        return t.tgt >= 0 ? df * t.cold : 0.f;
    };
    float v[U][L];
    bool live[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int64_t ch = first + threadIdx.x + 256 * u;
        live[u] = ch < chunks;
        RowChunk<T>::load(x + (live[u] ? ch : first) * L, v[u]);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        if (!live[u]) continue;
        const unsigned off = col0 + (threadIdx.x + 256u * u) * L;       // from the start of row0: below 2^32 (C < 2^31)
        const unsigned dr = off / C;
        unsigned col = off - dr * C;
        int64_t row = row0 + dr;
        RowTerms t = row_terms(row);
        if (col + L <= C) {
            if (t.tgt >= (int)col && t.tgt < (int)(col + L)) {          // the one chunk of its row that holds the target
#pragma unroll
                for (int e = 0; e < L; ++e) v[u][e] = one(v[u][e], (int)(col + e), t);
            } else {
#pragma unroll
                for (int e = 0; e < L; ++e) v[u][e] = cold_only(v[u][e], t);
            }
        } else {                                        // the chunk crosses into the next row: both rows' terms, chosen per element
            RowTerms t2 = row_terms(row + 1);
            t2.tgt = t2.tgt < 0 ? -1 : t2.tgt + (int)C;     // in the first row's column numbers
#pragma unroll
            for (int e = 0; e < L; ++e) {
                const bool next = col + e >= C;
                RowTerms te;
                te.gk = next ? t2.gk : t.gk;
                te.cold = next ? t2.cold : t.cold;
                te.tgt = next ? t2.tgt : t.tgt;
                v[u][e] = one(v[u][e], (int)(col + e), te);
            }
        }
        RowChunk<T>::store(grad + (first + threadIdx.x + 256 * u) * L, v[u]);
    }
    // what is left after the last whole chunk: at most L - 1 elements of the last row
    if (blockIdx.x == gridDim.x - 1) {
        const int64_t at = chunks * L + threadIdx.x;
        if (at < p.P * p.C) {
            const RowTerms t = row_terms(p.P - 1);
            store_one(grad + at, one(load_one(x + at), (int)(at - (p.P - 1) * p.C), t));
        }
    }
}

// Cross-entropy backward from the forward's per-pixel S, for channel planes that start on element boundaries only (odd
// crops): the walk of lsr_bwd_planes - a block takes 1024 pixels of an image and in plane c its 256 threads move the
// 32 whole lines that begin at the tile's first pixel shifted back by the plane's offset into its line, so loads and
// stores are aligned 16-byte accesses in every plane; the pixels' (gout / S, label) pairs, the tile's and one line's
// worth before it, are staged in LDS once, transposed by pixel index mod 4. With k = gout / S the gradient is
// f'(x) k, and f'(x) (k - gout / f(x)) in the target's plane. One scalar upstream gradient, fp32, orders 2 and 4.
template <class T, int ORD>
__global__ __launch_bounds__(256) void taylor_ce_bwd_planes(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                            const Upstream up, T *__restrict__ grad, const TaylorParams p,
                                                            int tiles, int planes_per_block) {
    static_assert(sizeof(T) == 4, "fp32 logits (see taylor_sums_apply)");
    using G = PlaneGeom<T>;
    constexpr int kPer = G::kPer, kTile = G::kTile, kHalo = G::kHalo;
    __shared__ PlanePixel pairs[kPer][(kTile + kHalo) / kPer];          // entry i at [i % kPer][i / kPer]
    const int64_t M = p.m_size;
    const int64_t n = blockIdx.x / tiles;
    const int t = (int)(blockIdx.x - n * tiles);
    const int l = threadIdx.x;
    float gk = up.gout ? *up.gout * up.scale : up.scale;
    if (up.divide_by) gk = gk / (float)(*up.divide_by);
    const int64_t p_first = (int64_t)t * kTile - kHalo;                 // image-local pixel of staged entry 0
    for (int i = l; i < kTile + kHalo; i += 256) {
        const int64_t q = p_first + i;
        PlanePixel px{0.f, -1};
        if (q >= 0 && q < M) {
            const int64_t at = n * M + q;
            const int64_t lb = lab[at];
            const bool has_y = lb != p.ignore && lb >= 0 && lb < p.C;
            px.lse = gk / p.sums[at];
            px.lab = has_y ? (int)lb : -1;              // pixels without a target: exact zeros (taylor_ce_bwd_regs)
        }
        pairs[i % kPer][i / kPer] = px;
    }
    __syncthreads();
    auto one = [&](float xv, PlanePixel px, int c) {
        float f, df;
        taylor_pair24<ORD>(xv, f, df);
        const float k = (px.lab == c) ? px.lse - gk / f : px.lse;
        return px.lab < 0 ? 0.f : df * k;
    };
    constexpr int U = 4;                            // planes in flight per thread
    // blockIdx.y: which planes of the tile (many channels are shared out over several blocks, so that the grid fills the chip)
    const int c_begin = blockIdx.y * planes_per_block;
    const int c_end = c_begin + planes_per_block < p.C ? c_begin + planes_per_block : p.C;
    for (int c0 = c_begin; c0 < c_end; c0 += U) {
        plh_u4 xv[U];
        int64_t q[U], plane[U];
        bool full[U];
        int first[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int c = c0 + u < c_end ? c0 + u : c_end - 1;
            plane[u] = (n * p.C + c) * M;
            // the plane's offset into its line, in elements
            const int shift = (int)((reinterpret_cast<uintptr_t>(x + plane[u]) / sizeof(T)) & (unsigned)(G::kLine - 1));
            first[u] = kHalo + kPer * l - shift;                     // staged index of this lane's first pixel
            q[u] = (int64_t)t * kTile - shift + kPer * l;
            full[u] = q[u] >= 0 && q[u] + (kPer - 1) < M;
            xv[u] = __builtin_nontemporal_load(reinterpret_cast<const plh_u4 *>(x + plane[u] + (full[u] ? q[u] : 0)));
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int c = c0 + u;
            if (c >= c_end) break;
            const int i0 = first[u];
            if (full[u]) {
                const unsigned in[4] = {xv[u].x, xv[u].y, xv[u].z, xv[u].w};
                unsigned out[4];
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    const int i = i0 + d;
                    out[d] = f32_bits(one(bits_f32(in[d]), pairs[i % kPer][i / kPer], c));
                }
                __builtin_nontemporal_store(plh_u4{out[0], out[1], out[2], out[3]},
                                            reinterpret_cast<plh_u4 *>(grad + plane[u] + q[u]));
            } else {                    // the two ends of a plane, element by element
                for (int k = 0; k < kPer; ++k)
                    if (q[u] + k >= 0 && q[u] + k < M)
                        store_one(grad + plane[u] + q[u] + k,
                                  one(load_one(x + plane[u] + q[u] + k), pairs[(i0 + k) % kPer][(i0 + k) / kPer], c));
            }
        }
    }
}

// ------------------------------------------------------------ dispatch ----

template <class T, int Kind>
unsigned taylor_launch(const T *x, const T *g, const int64_t *lab, const Upstream &up, T *out, float *loss, Partials part,
                       const TaylorParams &p, hipStream_t st) {
    constexpr int VT = ElemTraits<T>::kVec;
    const float *go_vec = (Kind == kTaylorCeBwd && up.gout && up.stride == 1) ? up.gout : nullptr;
    constexpr bool kIsCe = (Kind == kTaylorCeFwd || Kind == kTaylorCeBwd);       // the deep split form is theirs only
    const bool walk = p.order > 4;          // the register-resident forms are compiled for orders 2 and 4 (taylor_pair24)
    const Shape shape = walk ? Shape::Lane : pick_shape(p.C, p.m_size, VT, sizeof(T), x, (Kind == kTaylorCeFwd) ? nullptr : (const void *)out,
                                   lab, (Kind == kTaylorCeFwd) ? (const void *)loss : nullptr, go_vec, true, kIsCe, true,
                                   kImageFormMaxChannels<T, (Kind == kTaylorBwd) ? 2 : 1>);
    const bool g_ok = (Kind != kTaylorBwd) || !misaligned(g, VT * sizeof(T));
    if constexpr (Kind == kTaylorCeBwd && sizeof(T) == 4) {
        // odd crops, from the forward's per-pixel S, plane by plane: one scalar upstream gradient, logits and gradient at
        // the same offset into a 128-byte line (whole lines of the one are whole lines of the other)
        const int64_t tiles = ceil_div(p.m_size + PlaneGeom<T>::kHalo - 1, (int64_t)PlaneGeom<T>::kTile);
        if (p.sums && !go_vec && p.m_size > 1 && !walk && taylor_sums_apply(sizeof(T), p.C, p.m_size) &&
            ((reinterpret_cast<uintptr_t>(x) ^ reinterpret_cast<uintptr_t>(out)) & 127) == 0 && !misaligned(x, sizeof(T)) &&
            p.P / p.m_size * tiles < ((int64_t)1 << 31)) {
            // planes per block as for lsr_bwd_planes: all of them up to 32 channels; beyond, 16 on planes of 1 MiB and
            // more, else 4 (8 when the tiles alone outnumber the blocks the chip holds at once)
            const int64_t tiles_all = p.P / p.m_size * tiles;
            const int per = p.C <= kMaxRegsChannels                      ? p.C
                            : p.m_size * (int64_t)sizeof(T) >= (1 << 20) ? 16
                            : tiles_all <= 2048                          ? 4
                                                                         : 8;
            const dim3 grid((unsigned)tiles_all, (unsigned)ceil_div(p.C, per));
            if (p.order == 2)
                hipLaunchKernelGGL((taylor_ce_bwd_planes<T, 2>), grid, dim3(256), 0, st, x, lab, up, out, p, (int)tiles, per);
            else
                hipLaunchKernelGGL((taylor_ce_bwd_planes<T, 4>), grid, dim3(256), 0, st, x, lab, up, out, p, (int)tiles, per);
            return (unsigned)tiles_all;
        }
    }
    if constexpr (Kind == kTaylorCeBwd) {
        // long rows, from the sums the forward left: elementwise over the flattened tensor
        constexpr int L = RowChunk<T>::kLen;
        const int64_t chunks = p.P * p.C / L, flat_blocks = ceil_div(chunks, (int64_t)(256 * kFlatChunks));
        if (p.sums && !go_vec && p.m_size == 1 && taylor_sums_apply(sizeof(T), p.C, p.m_size) && !misaligned(x, 16) && !misaligned(out, 16) &&
            flat_blocks >= 1 && flat_blocks < ((int64_t)1 << 31)) {
            // (the order as a compile-time constant pays on 16-bit logits, bf16 (4194304,64) 0.238 -> 0.215 ms, and costs fp32
            // ones 3 %, (4194304,64) 0.357 -> 0.372: those keep the test per evaluation)
            constexpr int kOrd2 = sizeof(T) == 2 ? 2 : 0, kOrd4 = sizeof(T) == 2 ? 4 : 0;
            if (p.order == 2)
                hipLaunchKernelGGL((taylor_ce_bwd_flat_sums<T, kOrd2>), dim3((unsigned)flat_blocks), dim3(256), 0, st, x, lab, up,
                                   out, p, chunks);
            else if (p.order == 4)
                hipLaunchKernelGGL((taylor_ce_bwd_flat_sums<T, kOrd4>), dim3((unsigned)flat_blocks), dim3(256), 0, st, x, lab, up,
                                   out, p, chunks);
            else
                hipLaunchKernelGGL((taylor_ce_bwd_flat_sums<T, 0>), dim3((unsigned)flat_blocks), dim3(256), 0, st, x, lab, up,
                                   out, p, chunks);
            return (unsigned)flat_blocks;
        }
    }
    if constexpr (kIsCe) {
        if (shape == Shape::SplitDeep) {            // 257..512 channels: up to 64 slots per wavefront, half the pixels per lane
            constexpr int VD = VT / 2;
            const unsigned grid = split_grid<VD>(p.P);
            // (the forward that leaves the pixels' S has no per-pixel losses to write, so their slot serves)
            float *const loss_dp = (Kind == kTaylorCeFwd && p.sums != nullptr && loss == nullptr &&
                                    taylor_sums_apply(sizeof(T), p.C, p.m_size)) ? p.sums : loss;
            switch (split_slots_deep(p.C)) {
#define PLH_CASE(KW)                                                                                                  \
    case KW:                                                                                                          \
        if constexpr (Kind == kTaylorCeFwd)                                                                           \
            hipLaunchKernelGGL((taylor_ce_fwd_split<T, KW, VD>), dim3(grid), dim3(kSplitBlock), 0, st, x, lab, \
                               loss_dp, part, p);                                                                     \
        else                                                                                                          \
            hipLaunchKernelGGL((taylor_ce_bwd_split<T, KW, VD>), dim3(grid), dim3(kSplitBlock), 0, st, x, lab, up, out, \
                               p);                                                                                    \
        break;
                PLH_SPLIT_DEEP_CASES
#undef PLH_CASE
            }
            return grid;
        }
    }
    // 33..256 channels in NCHW; in tiles per image where the planes start on element boundaries only (or the
    // upstream tensor of the softmax backward does)
    const bool image = shape == Shape::SplitImage || (shape == Shape::Split && !g_ok && p.m_size >= 4096);
    if (image || (shape == Shape::Split && g_ok)) {
        const unsigned grid = image ? split_image_grid<VT>(p.P / p.m_size, p.m_size) : split_grid<VT>(p.P);
        // (the tiles-per-image forward that leaves the pixels' S has no per-pixel losses to write, so their slot serves)
        float *const loss_sp = (Kind == kTaylorCeFwd && shape == Shape::SplitImage && p.sums != nullptr && loss == nullptr &&
                                taylor_sums_apply(sizeof(T), p.C, p.m_size)) ? p.sums : loss;
#define PLH_GO(KW, IMG)                                                                                               \
    do {                                                                                                              \
        if constexpr (Kind == kTaylorFwd)                                                                             \
            hipLaunchKernelGGL((taylor_sm_fwd_split<T, KW, VT, IMG>), dim3(grid), dim3(kSplitBlock), 0, st, x, out, p); \
        else if constexpr (Kind == kTaylorBwd)                                                                        \
            hipLaunchKernelGGL((taylor_sm_bwd_split<T, KW, VT, IMG>), dim3(grid), dim3(kSplitBlock), 0, st, g, x, out, p); \
        else if constexpr (Kind == kTaylorCeFwd)                                                                      \
            hipLaunchKernelGGL((taylor_ce_fwd_split<T, KW, VT, IMG>), dim3(grid), dim3(kSplitBlock), 0, st, x, \
                               lab, loss_sp, part, p);                                                                \
        else                                                                                                          \
            hipLaunchKernelGGL((taylor_ce_bwd_split<T, KW, VT, IMG>), dim3(grid), dim3(kSplitBlock), 0, st, x, lab, up, \
                               out, p);                                                                               \
    } while (0)
        switch (split_slots(p.C)) {
#define PLH_CASE(KW)                   \
    case KW:                           \
        if (image) PLH_GO(KW, true);   \
        else PLH_GO(KW, false);        \
        break;
            PLH_SPLIT_SLOT_CASES
#undef PLH_CASE
#undef PLH_GO
        }
        return grid;
    }
    if (shape == Shape::RegsVec || shape == Shape::RegsOne) {
        const bool vec = (shape == Shape::RegsVec) && g_ok;
        const bool uni = vec && tiles_are_uniform(p.m_size, VT, sizeof(T));
        // planes that start on element boundaries only: tiles per image, four pixels per lane (the softmax
        // backward holds two slices, so half the channels)
        constexpr int kSlices = (Kind == kTaylorBwd) ? 2 : 1;
        const bool image = !vec && image_form_pays<T, kSlices>(p.C, p.m_size);
        const unsigned grid = vec ? regs_grid<VT>(p.P) : (image ? image_grid<4>(p.P / p.m_size, p.m_size) : regs_grid<1>(p.P));
        // (the per-image forward that leaves the pixels' S has no per-pixel losses to write, so their slot serves)
        float *const loss_px = (Kind == kTaylorCeFwd && image && p.sums != nullptr && loss == nullptr && p.m_size > 1 &&
                                taylor_sums_apply(sizeof(T), p.C, p.m_size)) ? p.sums : loss;
#define PLH_GO(CPV, VV, UU)                                                                                          \
    do {                                                                                                             \
        if constexpr (Kind == kTaylorFwd)                                                                            \
            hipLaunchKernelGGL((taylor_fwd_regs<T, CPV, VV, UU>), dim3(grid), dim3(kRegsBlock), 0, st, x, out, p);   \
        else if constexpr (Kind == kTaylorBwd)                                                                       \
            hipLaunchKernelGGL((taylor_bwd_regs<T, CPV, VV, UU>), dim3(grid), dim3(kRegsBlock), 0, st, g, x, out, p); \
        else if constexpr (Kind == kTaylorCeFwd)                                                                     \
            hipLaunchKernelGGL((taylor_ce_fwd_regs<T, CPV, VV, UU>), dim3(grid), dim3(kRegsBlock), 0, st, x, \
                               lab, loss_px, part, p);                                                               \
        else                                                                                                         \
            hipLaunchKernelGGL((taylor_ce_bwd_regs<T, CPV, VV, UU>), dim3(grid), dim3(kRegsBlock), 0, st, x, lab,    \
                               up, out, p);                                                                          \
    } while (0)
        switch ((p.C + 3) / 4) {
#define PLH_CASE(K)                                                    \
    case K:                                                            \
        if (uni) PLH_GO(4 * K, VT, kUniform);                          \
        else if (vec) PLH_GO(4 * K, VT, kGeneral);                     \
        else if (image) {                                              \
            if constexpr (4 * K <= kImageFormMaxChannels<T, kSlices>)  \
                PLH_GO(4 * K, 4, kPerImage);                           \
        } else PLH_GO(4 * K, 1, kGeneral);                             \
        break;
            PLH_CASE(1) PLH_CASE(2) PLH_CASE(3) PLH_CASE(4) PLH_CASE(5) PLH_CASE(6) PLH_CASE(7) PLH_CASE(8)
#undef PLH_CASE
#undef PLH_GO
        }
        return grid;
    }
    if (p.m_size == 1) {
        const int piece = wrow_piece<T>(x, (Kind == kTaylorCeFwd) ? (const T *)nullptr : (const T *)out, p.C,
                                        (Kind == kTaylorBwd) ? g : (const T *)nullptr);
        // the backwards keep the 2048-element limit: the softmax backward holds two rows in registers, and the
        // cross-entropy backward with 64 registers of row ran at a third of its two-sweep form (bf16 (65536, 4096):
        // 0.782 against 0.304 ms)
        constexpr bool kForward = (Kind == kTaylorFwd || Kind == kTaylorCeFwd);
        // (the forward that leaves the rows' sums has no per-row losses to write, so their slot serves)
        const bool keep = Kind == kTaylorCeFwd && p.sums != nullptr && loss == nullptr &&
                          taylor_sums_apply(sizeof(T), p.C, p.m_size);
        float *const loss_slot = keep ? p.sums : loss;
        if (!walk && p.C <= (kForward ? wrow_cap<T>(piece) : kWaveRowCap)) {
            unsigned grid = 0;
#define PLH_GO(NI, W, G)                                                                                          \
    do {                                                                                                          \
        grid = group_grid(p.P, WaveRowAt<G>::kRowsPerBlock);                                                      \
        if constexpr (Kind != kTaylorCeFwd && wrow_cached_form<T>(W, G)) {                                        \
            if (wrow_rows_end_inside_lines<T>(p.C)) {                                                             \
                hipLaunchKernelGGL((taylor_wrow<T, NI, W, Kind, G, true>), dim3(grid), dim3(256), 0, st, x, g, \
                                   lab, up, out, loss_slot, part, p);                                             \
                break;                                                                                            \
            }                                                                                                     \
        }                                                                                                         \
        hipLaunchKernelGGL((taylor_wrow<T, NI, W, Kind, G>), dim3(grid), dim3(256), 0, st, x, g, lab, up, out, \
                           loss_slot, part, p);                                                                   \
    } while (0)
            PLH_WROW_DISPATCH_IF(piece, p.C, PLH_GO, (kForward ? 2 : 0));
#undef PLH_GO
            return grid;
        }
        const unsigned grid = (unsigned)(p.P < kMinPartialSlots ? p.P : kMinPartialSlots);
        if constexpr (Kind == kTaylorCeFwd || Kind == kTaylorCeBwd) {
            // short rows get small blocks in the forward (more rows in flight per CU, no idle lanes behind the barrier):
            // fp32 (65536,3000) 0.173 -> 0.152 ms with 64 threads, (65536,2049) 0.146 -> 0.110, bf16 (65536,3001) 0.164 ->
            // 0.104; rows of 16 KiB lose with them (fp32 (32768,4096) 0.096 -> 0.105)
            const int threads = (Kind == kTaylorCeFwd && (int64_t)p.C * (int64_t)sizeof(T) <= 12 * 1024) ? 64 : row_threads_for_sweep<T>(p.C);
            const int row_flags = (row_chunks_ok<T>(x, (Kind == kTaylorCeBwd) ? (const T *)out : (const T *)nullptr, p.C) ? 1 : 0) |
                                  (keep ? 2 : 0);
            // (16-bit forwards: the order a compile-time constant of the sweep, as in the elementwise backward)
            if (Kind == kTaylorCeFwd && sizeof(T) == 2 && p.order == 2)
                hipLaunchKernelGGL((taylor_ce_row<T, Kind, (Kind == kTaylorCeFwd && sizeof(T) == 2) ? 2 : 0>), dim3(grid),
                                   dim3(threads), 0, st, x, lab, up, out, loss_slot, part, p, row_flags);
            else if (Kind == kTaylorCeFwd && sizeof(T) == 2 && p.order == 4)
                hipLaunchKernelGGL((taylor_ce_row<T, Kind, (Kind == kTaylorCeFwd && sizeof(T) == 2) ? 4 : 0>), dim3(grid),
                                   dim3(threads), 0, st, x, lab, up, out, loss_slot, part, p, row_flags);
            else
                hipLaunchKernelGGL((taylor_ce_row<T, Kind>), dim3(grid), dim3(threads), 0, st, x, lab, up, out, loss_slot,
                                   part, p, row_flags);
        } else {
            const int vec = row_chunks_ok<T>(x, out, p.C) && !(Kind == kTaylorBwd && misaligned(g, 16));
            hipLaunchKernelGGL((taylor_sm_row<T, Kind>), dim3(grid), dim3(row_threads_for_sweep<T>(p.C)), 0, st, x, g, out, p, vec);
        }
        return grid;
    }
    const unsigned grid = group_grid(p.P, 256);
    hipLaunchKernelGGL((taylor_group<T, 1, Kind>), dim3(grid), dim3(256), 0, st, x, g, lab, up, out, loss, part, p);
    return grid;
}

// One translation unit per element type and kind (taylor_f32_fwd.hip, taylor_f32_bwd.hip, taylor_f32_cefwd.hip,
// taylor_f32_cebwd.hip, ...) so that the twelve parts compile in parallel.
#define PLH_TAYLOR_SIGNATURE(T, K)                                                                                    \
    unsigned taylor_launch<T, K>(const T *, const T *, const int64_t *, const Upstream &, T *, float *, Partials,     \
                                 const TaylorParams &, hipStream_t);
#define PLH_TAYLOR_EXTERN(T)                              \
    extern template PLH_TAYLOR_SIGNATURE(T, kTaylorFwd)   \
    extern template PLH_TAYLOR_SIGNATURE(T, kTaylorBwd)   \
    extern template PLH_TAYLOR_SIGNATURE(T, kTaylorCeFwd) \
    extern template PLH_TAYLOR_SIGNATURE(T, kTaylorCeBwd)
#define PLH_TAYLOR_INSTANTIATE(T, K) template PLH_TAYLOR_SIGNATURE(T, K)

}  // namespace plh
