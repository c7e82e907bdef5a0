// Label-smoothed softmax cross entropy, forward and backward, for gfx950.
//
// Math (per pixel, target y, smoothing s, C channels):
//   w_y = 1 - s, w_j = s / C otherwise            (csrc/lsr_kernel.cu:83-84)
//   loss = -sum_j w_j * log_softmax(x)_j          (csrc/lsr_kernel.cu:174-182)
//   grad_j = (sumw * softmax(x)_j - w_j) * upstream, sumw = (C-1) s/C + (1-s)
//                                                 (csrc/lsr_kernel.cu:123-143)
//   ignored pixel: loss 0, every grad 0.
// Unlike the reference (ATen log_softmax/softmax into a full-size temporary, a
// second kernel, then a Python-side multiply) each direction is ONE kernel that
// reads the logits once: forward 4E + 12P bytes, backward 8E + 12P bytes.
// The "reduced" forward additionally leaves per-block partial sums and valid-pixel
// counts behind, which a one-block finishing kernel turns into sum or mean, so the
// module-level reduction costs no further pass over the pixels.
#include "plh_common.hpp"

namespace plh {

struct LsrParams {
    int64_t P;        // pixels = n_size * m_size
    int64_t m_size;
    int C;
    int64_t ignore;
    float w_pos, w_neg, sumw;
};

// ---------------------------------------------------------------- regs ----

// loss = -sum_j w_j logp_j with logp_j = t_j - lse, t_j = x_j - max:
//      = -( w_neg * (sum_j t_j - C*lse) + (w_pos - w_neg) * (t_y - lse) )
// so one pass over the slice gathers max-shifted sum, exp-sum and the target's t.
template <int CP, int V, bool Uniform, bool Reduce>
__global__ __launch_bounds__(kRegsBlock) void lsr_fwd_regs(const float *__restrict__ x,
                                                          const int64_t *__restrict__ lab,
                                                          float *__restrict__ loss, Partials part,
                                                          const LsrParams p) {
    __shared__ float red[4];
    const PixelRef<V, Uniform> at(p.P, p.m_size, p.C);
    if (!Reduce && !at.live) return;

    float v[CP][V];
#pragma unroll
    for (int j = 0; j < CP; ++j)
        if (j < p.C) load_vec<V>(at.chan(x, j, p.m_size), v[j]);
    int64_t lb[V];
    load_labels<V>(lab + at.pix, lb);

    float out[V];
    float mine = 0.f;
    int cnt = 0;
#pragma unroll
    for (int k = 0; k < V; ++k) {
        bool ign;
        const int tgt = narrow_label(lb[k], p.ignore, p.C, ign);
        float mx = v[0][k];
#pragma unroll
        for (int j = 1; j < CP; ++j)
            if (j < p.C) mx = fmaxf(mx, v[j][k]);
        float s = 0.f, sum_t = 0.f, t_y = 0.f;
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (j < p.C) {
                const float t = v[j][k] - mx;
                s += fast_exp(t);
                sum_t += t;
                t_y = (tgt == j) ? t : t_y;
            }
        const float lse = fast_log(s);
        const float all = sum_t - (float)p.C * lse;
        // no target channel (label outside [0, C)): every weight is w_neg
        const float hot = (tgt >= 0) ? (p.w_pos - p.w_neg) * (t_y - lse) : 0.f;
        const float acc = -(p.w_neg * all + hot);
        const bool valid = at.live && !ign;
        out[k] = valid ? acc : 0.f;
        mine += out[k];
        cnt += valid ? 1 : 0;
    }
    if (at.live && loss) store_vec<V>(loss + at.pix, out);
    if constexpr (Reduce) {
        const float bs = block_sum_256(mine, red);
        const float bc = block_sum_256((float)cnt, red);   // at most 512 per block: exact in fp32
        if (threadIdx.x == 0) {
            part.sum[blockIdx.x] = bs;
            part.cnt[blockIdx.x] = (int)bc;
        }
    }
}

template <int CP, int V, bool Uniform>
__global__ __launch_bounds__(kRegsBlock) void lsr_bwd_regs(const float *__restrict__ x,
                                                          const int64_t *__restrict__ lab,
                                                          const Upstream up, float *__restrict__ grad,
                                                          const LsrParams p) {
    const PixelRef<V, Uniform> at(p.P, p.m_size, p.C);
    if (!at.live) return;

    float v[CP][V];
#pragma unroll
    for (int j = 0; j < CP; ++j)
        if (j < p.C) load_vec<V>(at.chan(x, j, p.m_size), v[j]);
    int64_t lb[V];
    load_labels<V>(lab + at.pix, lb);
    float go[V];
    load_upstream<V>(up, at.pix, go);

#pragma unroll
    for (int k = 0; k < V; ++k) {
        float mx = v[0][k];
#pragma unroll
        for (int j = 1; j < CP; ++j)
            if (j < p.C) mx = fmaxf(mx, v[j][k]);
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (j < p.C) {
                v[j][k] = fast_exp(v[j][k] - mx);
                s += v[j][k];
            }
        bool ign;
        const int tgt = narrow_label(lb[k], p.ignore, p.C, ign);
        const float gk = go[k];
        const float scale = p.sumw * gk / s;          // one division per pixel
        const float g_pos = p.w_pos * gk, g_neg = p.w_neg * gk;
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (j < p.C) {
                const float g = v[j][k] * scale - ((tgt == j) ? g_pos : g_neg);
                v[j][k] = ign ? 0.f : g;              // exact zero even for non-finite logits
            }
    }
#pragma unroll
    for (int j = 0; j < CP; ++j)
        if (j < p.C) store_vec<V>(at.chan(grad, j, p.m_size), v[j]);
}

// --------------------------------------------------------------- group ----
// G lanes per pixel. G = 64 stages the wave's slice in LDS (each lane re-reads
// only what it wrote, so no barrier is needed); G = 1 re-reads global memory,
// which the preceding pass has just pulled into cache.

constexpr int kStageCap = 2048;   // floats per wave -> 32 KiB of LDS per 256-thread block

template <int G, bool Reduce>
__global__ __launch_bounds__(256) void lsr_fwd_group(const float *__restrict__ x,
                                                     const int64_t *__restrict__ lab,
                                                     float *__restrict__ loss, Partials part,
                                                     const LsrParams p) {
    constexpr int kPix = 256 / G;
    __shared__ float stage_mem[(G == 64) ? 4 * kStageCap : 1];
    __shared__ float red[4];
    const int sub = threadIdx.x % G;
    const int grp = threadIdx.x / G;
    float *stage = stage_mem + ((G == 64) ? grp * kStageCap : 0);
    const bool staged = (G == 64) && (p.C <= kStageCap);

    float mine = 0.f, cnt = 0.f;
    // every lane of a group walks the same pixels, so the loop is group-uniform
    const int64_t rounds = ceil_div_dev(p.P, (int64_t)gridDim.x * kPix);
    for (int64_t r = 0; r < rounds; ++r) {
        const int64_t pix = (r * gridDim.x + blockIdx.x) * kPix + grp;
        const bool live = pix < p.P;
        const int64_t pc = live ? pix : 0;
        const int64_t n = pc / p.m_size;
        const float *xs = x + (pc + n * (int64_t)(p.C - 1) * p.m_size);
        const int64_t lb = lab[pc];

        float mx = -INFINITY;
        for (int j = sub; j < p.C; j += G) {
            const float t = xs[(int64_t)j * p.m_size];
            if (staged) stage[j] = t;
            mx = fmaxf(mx, t);
        }
        mx = group_reduce<G>(mx, OpMax());
        float s = 0.f;
        for (int j = sub; j < p.C; j += G) {
            const float t = staged ? stage[j] : xs[(int64_t)j * p.m_size];
            s += fast_exp(t - mx);
        }
        s = group_reduce<G>(s, OpSum());
        const float lse = logf(s);
        float acc = 0.f;
        for (int j = sub; j < p.C; j += G) {
            const float t = staged ? stage[j] : xs[(int64_t)j * p.m_size];
            acc -= ((t - mx) - lse) * ((lb == j) ? p.w_pos : p.w_neg);
        }
        acc = group_reduce<G>(acc, OpSum());
        const bool valid = live && (lb != p.ignore);
        if (live && sub == 0) {
            if (loss) loss[pix] = valid ? acc : 0.f;
            mine += valid ? acc : 0.f;
            cnt += valid ? 1.f : 0.f;
        }
    }
    if constexpr (Reduce) {
        const float bs = block_sum_256(mine, red);
        const float bc = block_sum_256(cnt, red);     // exact while a block sees < 2^24 pixels
        if (threadIdx.x == 0) {
            part.sum[blockIdx.x] = bs;
            part.cnt[blockIdx.x] = (int)bc;
        }
    }
}

template <int G>
__global__ __launch_bounds__(256) void lsr_bwd_group(const float *__restrict__ x,
                                                     const int64_t *__restrict__ lab,
                                                     const Upstream up, float *__restrict__ grad,
                                                     const LsrParams p) {
    constexpr int kPix = 256 / G;
    __shared__ float stage_mem[(G == 64) ? 4 * kStageCap : 1];
    const int sub = threadIdx.x % G;
    const int grp = threadIdx.x / G;
    float *stage = stage_mem + ((G == 64) ? grp * kStageCap : 0);
    const bool staged = (G == 64) && (p.C <= kStageCap);

    const int64_t rounds = ceil_div_dev(p.P, (int64_t)gridDim.x * kPix);
    for (int64_t r = 0; r < rounds; ++r) {
        const int64_t pix = (r * gridDim.x + blockIdx.x) * kPix + grp;
        const bool live = pix < p.P;
        const int64_t pc = live ? pix : 0;
        const int64_t n = pc / p.m_size;
        const int64_t base = pc + n * (int64_t)(p.C - 1) * p.m_size;
        const float *xs = x + base;
        float *gs = grad + base;
        const int64_t lb = lab[pc];
        float go[1];
        load_upstream<1>(up, pc, go);

        float mx = -INFINITY;
        for (int j = sub; j < p.C; j += G) {
            const float t = xs[(int64_t)j * p.m_size];
            if (staged) stage[j] = t;
            mx = fmaxf(mx, t);
        }
        mx = group_reduce<G>(mx, OpMax());
        float s = 0.f;
        for (int j = sub; j < p.C; j += G) {
            const float t = staged ? stage[j] : xs[(int64_t)j * p.m_size];
            const float e = fast_exp(t - mx);
            if (staged) stage[j] = e;
            s += e;
        }
        s = group_reduce<G>(s, OpSum());
        if (live) {
            const float gk = (lb == p.ignore) ? 0.f : go[0];
            const float scale = p.sumw * gk / s;
            for (int j = sub; j < p.C; j += G) {
                const float e = staged ? stage[j] : fast_exp(xs[(int64_t)j * p.m_size] - mx);
                gs[(int64_t)j * p.m_size] = e * scale - ((lb == j) ? p.w_pos : p.w_neg) * gk;
            }
        }
    }
}

// ------------------------------------------------------------ dispatch ----

static LsrParams make_params(int64_t n_size, int64_t dimsize, int64_t m_size, int64_t ignore, float smooth) {
    LsrParams p;
    p.P = n_size * m_size;
    p.m_size = m_size;
    p.C = (int)dimsize;
    p.ignore = ignore;
    p.w_pos = 1.f - smooth;                        // csrc/lsr_kernel.cu:83
    p.w_neg = smooth / (float)dimsize;             // csrc/lsr_kernel.cu:84
    p.sumw = p.w_neg * (float)(dimsize - 1) + p.w_pos;   // csrc/lsr_kernel.cu:125
    return p;
}

template <int V, bool Reduce>
static unsigned launch_fwd_regs(const float *x, const int64_t *lab, float *loss, Partials part, const LsrParams &p,
                                hipStream_t st) {
    const unsigned grid = regs_grid<V>(p.P);
    const bool uni = tiles_are_uniform(p.m_size, V);
    switch ((p.C + 3) / 4) {
#define PLH_CASE(K)                                                                                              \
    case K:                                                                                                      \
        if (uni) hipLaunchKernelGGL((lsr_fwd_regs<4 * K, V, true, Reduce>), dim3(grid), dim3(kRegsBlock), 0, st, \
                                    x, lab, loss, part, p);                                                      \
        else hipLaunchKernelGGL((lsr_fwd_regs<4 * K, V, false, Reduce>), dim3(grid), dim3(kRegsBlock), 0, st, x, \
                                lab, loss, part, p);                                                             \
        break;
        PLH_CASE(1) PLH_CASE(2) PLH_CASE(3) PLH_CASE(4) PLH_CASE(5) PLH_CASE(6) PLH_CASE(7) PLH_CASE(8)
#undef PLH_CASE
    }
    return grid;
}

template <int V>
static void launch_bwd_regs(const float *x, const int64_t *lab, const Upstream &up, float *grad,
                            const LsrParams &p, hipStream_t st) {
    const unsigned grid = regs_grid<V>(p.P);
    const bool uni = tiles_are_uniform(p.m_size, V);
    switch ((p.C + 3) / 4) {
#define PLH_CASE(K)                                                                                               \
    case K:                                                                                                       \
        if (uni) hipLaunchKernelGGL((lsr_bwd_regs<4 * K, V, true>), dim3(grid), dim3(kRegsBlock), 0, st, x, lab,  \
                                    up, grad, p);                                                                 \
        else hipLaunchKernelGGL((lsr_bwd_regs<4 * K, V, false>), dim3(grid), dim3(kRegsBlock), 0, st, x, lab, up, \
                                grad, p);                                                                         \
        break;
        PLH_CASE(1) PLH_CASE(2) PLH_CASE(3) PLH_CASE(4) PLH_CASE(5) PLH_CASE(6) PLH_CASE(7) PLH_CASE(8)
#undef PLH_CASE
    }
}

// Launches the forward; returns the number of blocks that wrote partials.
template <bool Reduce>
static unsigned forward(const float *logits, const int64_t *labels, float *losses, Partials part,
                        const LsrParams &p, hipStream_t st) {
    switch (pick_shape(p.C, p.m_size, logits, nullptr, labels, losses, nullptr)) {
        case Shape::Regs2: return launch_fwd_regs<2, Reduce>(logits, labels, losses, part, p, st);
        case Shape::Regs1: return launch_fwd_regs<1, Reduce>(logits, labels, losses, part, p, st);
        case Shape::Wave: {
            const unsigned grid = group_grid(p.P, 4);
            hipLaunchKernelGGL((lsr_fwd_group<64, Reduce>), dim3(grid), dim3(256), 0, st, logits, labels, losses, part, p);
            return grid;
        }
        case Shape::Lane: {
            const unsigned grid = group_grid(p.P, 256);
            hipLaunchKernelGGL((lsr_fwd_group<1, Reduce>), dim3(grid), dim3(256), 0, st, logits, labels, losses, part, p);
            return grid;
        }
    }
    return 0;
}

static int backward(const float *logits, const int64_t *labels, const Upstream &up, float *grad_logits,
                    int64_t n_size, int64_t dimsize, int64_t m_size, int64_t ignore_index, float smooth,
                    void *stream) {
    const int rc = check_slice_args(logits, labels, grad_logits, n_size, dimsize, m_size);
    if (rc != PLH_OK) return rc;
    if (n_size * dimsize * m_size == 0) return PLH_OK;
    const LsrParams p = make_params(n_size, dimsize, m_size, ignore_index, smooth);
    hipStream_t st = (hipStream_t)stream;
    const float *go_vec = (up.gout && up.stride == 1) ? up.gout : nullptr;
    switch (pick_shape(dimsize, m_size, logits, grad_logits, labels, go_vec, nullptr)) {
        case Shape::Regs2: launch_bwd_regs<2>(logits, labels, up, grad_logits, p, st); break;
        case Shape::Regs1: launch_bwd_regs<1>(logits, labels, up, grad_logits, p, st); break;
        case Shape::Wave:
            hipLaunchKernelGGL((lsr_bwd_group<64>), dim3(group_grid(p.P, 4)), dim3(256), 0, st, logits, labels, up,
                               grad_logits, p);
            break;
        case Shape::Lane:
            hipLaunchKernelGGL((lsr_bwd_group<1>), dim3(group_grid(p.P, 256)), dim3(256), 0, st, logits, labels, up,
                               grad_logits, p);
            break;
    }
    return check_launch();
}

}  // namespace plh

using namespace plh;

extern "C" int plh_lsr_forward(const float *logits, const int64_t *labels, float *losses,
                               int64_t n_size, int64_t dimsize, int64_t m_size,
                               int64_t ignore_index, float smooth, void *stream) {
    const int rc = check_slice_args(logits, labels, losses, n_size, dimsize, m_size);
    if (rc != PLH_OK) return rc;
    if (n_size * dimsize * m_size == 0) return PLH_OK;
    const LsrParams p = make_params(n_size, dimsize, m_size, ignore_index, smooth);
    forward<false>(logits, labels, losses, Partials{nullptr, nullptr}, p, (hipStream_t)stream);
    return check_launch();
}

extern "C" int plh_lsr_forward_reduced(const float *logits, const int64_t *labels, float *losses,
                                       float *loss_out, int64_t *n_valid_out, int32_t mean,
                                       void *workspace, int64_t workspace_bytes,
                                       int64_t n_size, int64_t dimsize, int64_t m_size,
                                       int64_t ignore_index, float smooth, void *stream) {
    int rc = check_slice_args(logits, labels, loss_out, n_size, dimsize, m_size);
    if (rc != PLH_OK) return rc;
    Partials part;
    rc = carve_partials(workspace, workspace_bytes, n_size * m_size, loss_out, n_valid_out, part);
    if (rc != PLH_OK) return rc;
    if (losses && misaligned(losses, 4)) return PLH_ERR_MISALIGNED;
    hipStream_t st = (hipStream_t)stream;
    unsigned blocks = 0;
    if (n_size * dimsize * m_size != 0) {
        const LsrParams p = make_params(n_size, dimsize, m_size, ignore_index, smooth);
        blocks = forward<true>(logits, labels, losses, part, p, st);
    }
    finish_partials(part, blocks, loss_out, n_valid_out, mean ? kFinishMeanOverCount : kFinishSum, 0, st);
    return check_launch();
}

extern "C" int plh_lsr_backward(const float *logits, const int64_t *labels,
                                const float *grad_output, int64_t grad_output_stride,
                                float *grad_logits,
                                int64_t n_size, int64_t dimsize, int64_t m_size,
                                int64_t ignore_index, float smooth, void *stream) {
    const int rc = check_gout(grad_output, grad_output_stride);
    if (rc != PLH_OK) return rc;
    const Upstream up{grad_output, grad_output_stride, nullptr, 1.f};
    return backward(logits, labels, up, grad_logits, n_size, dimsize, m_size, ignore_index, smooth, stream);
}

extern "C" int plh_lsr_backward_scaled(const float *logits, const int64_t *labels,
                                       const float *grad_scalar, float scale, const int64_t *divide_by,
                                       float *grad_logits,
                                       int64_t n_size, int64_t dimsize, int64_t m_size,
                                       int64_t ignore_index, float smooth, void *stream) {
    if (n_size * dimsize * m_size != 0 && !grad_scalar) return PLH_ERR_NULL_POINTER;
    if (misaligned(grad_scalar, 4) || misaligned(divide_by, 8)) return PLH_ERR_MISALIGNED;
    const Upstream up{grad_scalar, 0, divide_by, scale};
    return backward(logits, labels, up, grad_logits, n_size, dimsize, m_size, ignore_index, smooth, stream);
}
