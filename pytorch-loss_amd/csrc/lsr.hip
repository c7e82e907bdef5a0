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

template <int CP, int V>
__global__ __launch_bounds__(256) void lsr_fwd_regs(const float *__restrict__ x,
                                                    const int64_t *__restrict__ lab,
                                                    float *__restrict__ loss, const LsrParams p) {
    const int64_t pix = ((int64_t)blockIdx.x * 256 + threadIdx.x) * V;
    if (pix >= p.P) return;
    const int64_t n = pix / p.m_size;
    const float *xs = x + (pix + n * (int64_t)(p.C - 1) * p.m_size);

    float v[CP][V];
#pragma unroll
    for (int j = 0; j < CP; ++j)
        if (j < p.C) load_vec<V>(xs + (int64_t)j * p.m_size, v[j]);
    int64_t lb[V];
    load_labels<V>(lab + pix, lb);

    float out[V];
#pragma unroll
    for (int k = 0; k < V; ++k) {
        float mx = v[0][k];
#pragma unroll
        for (int j = 1; j < CP; ++j)
            if (j < p.C) mx = fmaxf(mx, v[j][k]);
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (j < p.C) s += expf(v[j][k] - mx);
        const float lse = logf(s);
        float acc = 0.f;
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (j < p.C) {
                const float logp = (v[j][k] - mx) - lse;
                acc -= logp * ((lb[k] == j) ? p.w_pos : p.w_neg);
            }
        out[k] = (lb[k] == p.ignore) ? 0.f : acc;
    }
    store_vec<V>(loss + pix, out);
}

template <int CP, int V>
__global__ __launch_bounds__(256) void lsr_bwd_regs(const float *__restrict__ x,
                                                    const int64_t *__restrict__ lab,
                                                    const float *__restrict__ gout, int64_t gstride,
                                                    float *__restrict__ grad, const LsrParams p) {
    const int64_t pix = ((int64_t)blockIdx.x * 256 + threadIdx.x) * V;
    if (pix >= p.P) return;
    const int64_t n = pix / p.m_size;
    const int64_t base = pix + n * (int64_t)(p.C - 1) * p.m_size;
    const float *xs = x + base;
    float *gs = grad + base;

    float v[CP][V];
#pragma unroll
    for (int j = 0; j < CP; ++j)
        if (j < p.C) load_vec<V>(xs + (int64_t)j * p.m_size, v[j]);
    int64_t lb[V];
    load_labels<V>(lab + pix, lb);
    float go[V];
    load_gout<V>(gout, gstride, pix, go);

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
                v[j][k] = expf(v[j][k] - mx);
                s += v[j][k];
            }
        const bool ign = (lb[k] == p.ignore);
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (j < p.C) {
                const float prob = v[j][k] / s;
                const float g = (p.sumw * prob - ((lb[k] == j) ? p.w_pos : p.w_neg)) * go[k];
                v[j][k] = ign ? 0.f : g;
            }
    }
#pragma unroll
    for (int j = 0; j < CP; ++j)
        if (j < p.C) store_vec<V>(gs + (int64_t)j * p.m_size, v[j]);
}

// --------------------------------------------------------------- group ----
// G lanes per pixel. G = 64 stages the wave's slice in LDS (each lane re-reads
// only what it wrote, so no barrier is needed); G = 1 re-reads global memory,
// which the preceding pass has just pulled into cache.

constexpr int kStageCap = 2048;   // floats per wave -> 32 KiB of LDS per 256-thread block

template <int G>
__global__ __launch_bounds__(256) void lsr_fwd_group(const float *__restrict__ x,
                                                     const int64_t *__restrict__ lab,
                                                     float *__restrict__ loss, const LsrParams p) {
    constexpr int kPix = 256 / G;
    __shared__ float stage_mem[(G == 64) ? 4 * kStageCap : 1];
    const int sub = threadIdx.x % G;
    const int grp = threadIdx.x / G;
    float *stage = stage_mem + ((G == 64) ? grp * kStageCap : 0);
    const bool staged = (G == 64) && (p.C <= kStageCap);

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
            s += expf(t - mx);
        }
        s = group_reduce<G>(s, OpSum());
        const float lse = logf(s);
        float acc = 0.f;
        for (int j = sub; j < p.C; j += G) {
            const float t = staged ? stage[j] : xs[(int64_t)j * p.m_size];
            acc -= ((t - mx) - lse) * ((lb == j) ? p.w_pos : p.w_neg);
        }
        acc = group_reduce<G>(acc, OpSum());
        if (live && sub == 0) loss[pix] = (lb == p.ignore) ? 0.f : acc;
    }
}

template <int G>
__global__ __launch_bounds__(256) void lsr_bwd_group(const float *__restrict__ x,
                                                     const int64_t *__restrict__ lab,
                                                     const float *__restrict__ gout, int64_t gstride,
                                                     float *__restrict__ grad, const LsrParams p) {
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
        load_gout<1>(gout, gstride, pc, go);

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
            const float e = expf(t - mx);
            if (staged) stage[j] = e;
            s += e;
        }
        s = group_reduce<G>(s, OpSum());
        if (live) {
            const bool ign = (lb == p.ignore);
            for (int j = sub; j < p.C; j += G) {
                const float e = staged ? stage[j] : expf(xs[(int64_t)j * p.m_size] - mx);
                const float g = (p.sumw * (e / s) - ((lb == j) ? p.w_pos : p.w_neg)) * go[0];
                gs[(int64_t)j * p.m_size] = ign ? 0.f : g;
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

template <int V>
static void launch_fwd_regs(const float *x, const int64_t *lab, float *loss, const LsrParams &p, hipStream_t st) {
    const unsigned grid = (unsigned)ceil_div(ceil_div(p.P, V), 256);
    switch ((p.C + 3) / 4) {
#define PLH_CASE(K) case K: hipLaunchKernelGGL((lsr_fwd_regs<4 * K, V>), dim3(grid), dim3(256), 0, st, x, lab, loss, p); break;
        PLH_CASE(1) PLH_CASE(2) PLH_CASE(3) PLH_CASE(4) PLH_CASE(5) PLH_CASE(6) PLH_CASE(7) PLH_CASE(8)
#undef PLH_CASE
    }
}

template <int V>
static void launch_bwd_regs(const float *x, const int64_t *lab, const float *gout, int64_t gstride, float *grad,
                            const LsrParams &p, hipStream_t st) {
    const unsigned grid = (unsigned)ceil_div(ceil_div(p.P, V), 256);
    switch ((p.C + 3) / 4) {
#define PLH_CASE(K) case K: hipLaunchKernelGGL((lsr_bwd_regs<4 * K, V>), dim3(grid), dim3(256), 0, st, x, lab, gout, gstride, grad, p); break;
        PLH_CASE(1) PLH_CASE(2) PLH_CASE(3) PLH_CASE(4) PLH_CASE(5) PLH_CASE(6) PLH_CASE(7) PLH_CASE(8)
#undef PLH_CASE
    }
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
    hipStream_t st = (hipStream_t)stream;
    switch (pick_shape(dimsize, m_size, logits, nullptr, labels, losses, nullptr)) {
        case Shape::Regs4: launch_fwd_regs<4>(logits, labels, losses, p, st); break;
        case Shape::Regs1: launch_fwd_regs<1>(logits, labels, losses, p, st); break;
        case Shape::Wave:
            hipLaunchKernelGGL((lsr_fwd_group<64>), dim3(group_grid(p.P, 4)), dim3(256), 0, st, logits, labels, losses, p);
            break;
        case Shape::Lane:
            hipLaunchKernelGGL((lsr_fwd_group<1>), dim3(group_grid(p.P, 256)), dim3(256), 0, st, logits, labels, losses, p);
            break;
    }
    return check_launch();
}

extern "C" int plh_lsr_backward(const float *logits, const int64_t *labels,
                                const float *grad_output, int64_t grad_output_stride,
                                float *grad_logits,
                                int64_t n_size, int64_t dimsize, int64_t m_size,
                                int64_t ignore_index, float smooth, void *stream) {
    int rc = check_slice_args(logits, labels, grad_logits, n_size, dimsize, m_size);
    if (rc != PLH_OK) return rc;
    rc = check_gout(grad_output, grad_output_stride);
    if (rc != PLH_OK) return rc;
    if (n_size * dimsize * m_size == 0) return PLH_OK;
    const LsrParams p = make_params(n_size, dimsize, m_size, ignore_index, smooth);
    hipStream_t st = (hipStream_t)stream;
    const float *go_vec = (grad_output && grad_output_stride == 1) ? grad_output : nullptr;
    switch (pick_shape(dimsize, m_size, logits, grad_logits, labels, go_vec, nullptr)) {
        case Shape::Regs4: launch_bwd_regs<4>(logits, labels, grad_output, grad_output_stride, grad_logits, p, st); break;
        case Shape::Regs1: launch_bwd_regs<1>(logits, labels, grad_output, grad_output_stride, grad_logits, p, st); break;
        case Shape::Wave:
            hipLaunchKernelGGL((lsr_bwd_group<64>), dim3(group_grid(p.P, 4)), dim3(256), 0, st, logits, labels,
                               grad_output, grad_output_stride, grad_logits, p);
            break;
        case Shape::Lane:
            hipLaunchKernelGGL((lsr_bwd_group<1>), dim3(group_grid(p.P, 256)), dim3(256), 0, st, logits, labels,
                               grad_output, grad_output_stride, grad_logits, p);
            break;
    }
    return check_launch();
}
