// Large-margin softmax cross entropy (Kobayashi, BMVC 2019), forward / backward /
// fused forward+backward, for gfx950.
//
// Per valid pixel with target y (csrc/large_margin_kernel.cu:450-475, comment :450-460):
//   p = softmax(x) over all C channels, q = softmax(x) over the channels j != y,
//   coeff = 1/(C-1), h = lam/2
//   loss = -log p_y + h * sum_{j!=y} (q_j - coeff) * log q_j
//   g_y  = p_y - 1
//   g_j  = p_j + h * ((x_j + 1 - sum_k q_k x_k) * q_j - coeff)          (j != y)
//   ignored pixel: loss 0, every grad 0                      (large_margin_kernel.cu:414-421)
// The two softmaxes keep separate maxima (m_no over j != y, m_all = max(m_no, x_y)),
// so a dominant target logit cannot underflow the non-target sum; the full sum is
// rebuilt from the non-target one:  s_all = s_no * exp(m_no - m_all) + exp(x_y - m_all).
// Each direction is one kernel that reads the logits once.
#include "plh_common.hpp"

namespace plh {

struct LmParams {
    int64_t P;
    int64_t m_size;
    int C;
    int64_t ignore;
    float half_lam, coeff;
};

// ---------------------------------------------------------------- regs ----

template <int CP, int V, bool WantLoss, bool WantGrad, bool WantCount>
__global__ __launch_bounds__(256) void lm_regs(const float *__restrict__ x, const int64_t *__restrict__ lab,
                                               const float *__restrict__ gout, int64_t gstride,
                                               float *__restrict__ loss, float *__restrict__ grad,
                                               unsigned long long *__restrict__ valid_cnt, const LmParams p) {
    const int64_t pix = ((int64_t)blockIdx.x * 256 + threadIdx.x) * V;
    if (pix >= p.P) return;
    const int64_t n = pix / p.m_size;
    const int64_t base = pix + n * (int64_t)(p.C - 1) * p.m_size;
    const float *xs = x + base;

    float v[CP][V];
#pragma unroll
    for (int j = 0; j < CP; ++j)
        if (j < p.C) load_vec<V>(xs + (int64_t)j * p.m_size, v[j]);
    int64_t lb[V];
    load_labels<V>(lab + pix, lb);
    float go[V];
    if constexpr (WantGrad) load_gout<V>(gout, gstride, pix, go);

    float out[V];
    unsigned n_valid = 0;
#pragma unroll
    for (int k = 0; k < V; ++k) {
        const bool ign = (lb[k] == p.ignore);
        float m_no = -INFINITY, x_y = -INFINITY;
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (j < p.C) {
                const bool hot = (lb[k] == j);
                m_no = hot ? m_no : fmaxf(m_no, v[j][k]);
                x_y = hot ? v[j][k] : x_y;
            }
        const float m_all = fmaxf(m_no, x_y);
        float s_no = 0.f, sum_ex = 0.f;
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (j < p.C) {
                const float e = (lb[k] == j) ? 0.f : expf(v[j][k] - m_no);
                s_no += e;
                if constexpr (WantGrad) sum_ex += e * v[j][k];
            }
        const float t = expf(m_no - m_all);
        const float e_y = expf(x_y - m_all);
        const float s_all = s_no * t + e_y;
        const float inv_no = 1.f / s_no;
        const float inv_all = 1.f / s_all;
        const float sum_qx = sum_ex * inv_no;
        const float lse_no = logf(s_no);
        float acc = 0.f;
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (j < p.C) {
                const bool hot = (lb[k] == j);
                const float xv = v[j][k];
                const float e = expf(xv - m_no);
                const float q = e * inv_no;
                if constexpr (WantLoss) {
                    const float term = p.half_lam * (q - p.coeff) * ((xv - m_no) - lse_no);
                    acc += hot ? 0.f : term;
                }
                if constexpr (WantGrad) {
                    const float g_hot = e_y * inv_all - 1.f;
                    const float g_cold = e * t * inv_all + p.half_lam * ((xv + 1.f - sum_qx) * q - p.coeff);
                    const float g = (hot ? g_hot : g_cold) * go[k];
                    v[j][k] = ign ? 0.f : g;
                }
            }
        if constexpr (WantLoss) {
            acc += -(x_y - m_all) + logf(s_all);
            out[k] = ign ? 0.f : acc;
        }
        if constexpr (WantCount) n_valid += __builtin_popcountll(__builtin_amdgcn_ballot_w64(!ign));
    }
    if constexpr (WantLoss) store_vec<V>(loss + pix, out);
    if constexpr (WantGrad) {
        float *gs = grad + base;
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (j < p.C) store_vec<V>(gs + (int64_t)j * p.m_size, v[j]);
    }
    if constexpr (WantCount) {
        // lanes leave only at the tail of the grid, so lane 0 of a wave with work is alive
        if ((threadIdx.x & 63) == 0) atomicAdd(valid_cnt, (unsigned long long)n_valid);
    }
}

// --------------------------------------------------------------- group ----

constexpr int kLmStageCap = 2048;

template <int G, bool WantLoss, bool WantGrad, bool WantCount>
__global__ __launch_bounds__(256) void lm_group(const float *__restrict__ x, const int64_t *__restrict__ lab,
                                                const float *__restrict__ gout, int64_t gstride,
                                                float *__restrict__ loss, float *__restrict__ grad,
                                                unsigned long long *__restrict__ valid_cnt, const LmParams p) {
    constexpr int kPix = 256 / G;
    __shared__ float stage_mem[(G == 64) ? 4 * kLmStageCap : 1];
    const int sub = threadIdx.x % G;
    const int grp = threadIdx.x / G;
    float *stage = stage_mem + ((G == 64) ? grp * kLmStageCap : 0);
    const bool staged = (G == 64) && (p.C <= kLmStageCap);

    unsigned long long n_valid = 0;
    const int64_t rounds = ceil_div_dev(p.P, (int64_t)gridDim.x * kPix);
    for (int64_t r = 0; r < rounds; ++r) {
        const int64_t pix = (r * gridDim.x + blockIdx.x) * kPix + grp;
        const bool live = pix < p.P;
        const int64_t pc = live ? pix : 0;
        const int64_t n = pc / p.m_size;
        const int64_t base = pc + n * (int64_t)(p.C - 1) * p.m_size;
        const float *xs = x + base;
        const int64_t lb = lab[pc];
        const bool ign = (lb == p.ignore);
        float go[1] = {1.f};
        if constexpr (WantGrad) load_gout<1>(gout, gstride, pc, go);

        float m_no = -INFINITY, x_y = -INFINITY;
        for (int j = sub; j < p.C; j += G) {
            const float t = xs[(int64_t)j * p.m_size];
            if (staged) stage[j] = t;
            if (lb == j) x_y = t; else m_no = fmaxf(m_no, t);
        }
        m_no = group_reduce<G>(m_no, OpMax());
        x_y = group_reduce<G>(x_y, OpMax());
        const float m_all = fmaxf(m_no, x_y);
        float s_no = 0.f, sum_ex = 0.f;
        for (int j = sub; j < p.C; j += G) {
            const float t = staged ? stage[j] : xs[(int64_t)j * p.m_size];
            const float e = (lb == j) ? 0.f : expf(t - m_no);
            s_no += e;
            sum_ex += e * t;
        }
        s_no = group_reduce<G>(s_no, OpSum());
        sum_ex = group_reduce<G>(sum_ex, OpSum());
        const float t_all = expf(m_no - m_all);
        const float e_y = expf(x_y - m_all);
        const float s_all = s_no * t_all + e_y;
        const float inv_no = 1.f / s_no, inv_all = 1.f / s_all;
        const float sum_qx = sum_ex * inv_no;
        const float lse_no = logf(s_no);
        float acc = 0.f;
        for (int j = sub; j < p.C; j += G) {
            const float xv = staged ? stage[j] : xs[(int64_t)j * p.m_size];
            const bool hot = (lb == j);
            const float e = expf(xv - m_no);
            const float q = e * inv_no;
            if constexpr (WantLoss) acc += hot ? 0.f : p.half_lam * (q - p.coeff) * ((xv - m_no) - lse_no);
            if constexpr (WantGrad) {
                const float g_hot = e_y * inv_all - 1.f;
                const float g_cold = e * t_all * inv_all + p.half_lam * ((xv + 1.f - sum_qx) * q - p.coeff);
                if (live) grad[base + (int64_t)j * p.m_size] = ign ? 0.f : (hot ? g_hot : g_cold) * go[0];
            }
        }
        if constexpr (WantLoss) {
            acc = group_reduce<G>(acc, OpSum());
            acc += -(x_y - m_all) + logf(s_all);
            if (live && sub == 0) loss[pix] = ign ? 0.f : acc;
        }
        // every lane of the wave is inside the loop, so the ballot sees the whole wave
        if constexpr (WantCount)
            n_valid += __builtin_popcountll(__builtin_amdgcn_ballot_w64(live && sub == 0 && !ign));
    }
    if constexpr (WantCount) {
        if ((threadIdx.x & 63) == 0 && n_valid) atomicAdd(valid_cnt, n_valid);
    }
}

__global__ void lm_zero_count(unsigned long long *cnt) { *cnt = 0; }

// ------------------------------------------------------------ dispatch ----

template <int V, bool WantLoss, bool WantGrad, bool WantCount>
static void launch_regs(const float *x, const int64_t *lab, const float *gout, int64_t gstride, float *loss,
                        float *grad, unsigned long long *cnt, const LmParams &p, hipStream_t st) {
    const unsigned grid = (unsigned)ceil_div(ceil_div(p.P, V), 256);
    switch ((p.C + 3) / 4) {
#define PLH_CASE(K)                                                                                          \
    case K:                                                                                                  \
        hipLaunchKernelGGL((lm_regs<4 * K, V, WantLoss, WantGrad, WantCount>), dim3(grid), dim3(256), 0, st, \
                           x, lab, gout, gstride, loss, grad, cnt, p);                                       \
        break;
        PLH_CASE(1) PLH_CASE(2) PLH_CASE(3) PLH_CASE(4) PLH_CASE(5) PLH_CASE(6) PLH_CASE(7) PLH_CASE(8)
#undef PLH_CASE
    }
}

template <bool WantLoss, bool WantGrad, bool WantCount>
static int launch(const float *x, const int64_t *lab, const float *gout, int64_t gstride, float *loss, float *grad,
                  int64_t *valid_cnt, int64_t n_size, int64_t dimsize, int64_t m_size, int64_t ignore, float lam,
                  void *stream) {
    int rc = check_slice_args(x, lab, WantLoss ? (const void *)loss : (const void *)grad, n_size, dimsize, m_size);
    if (rc != PLH_OK) return rc;
    rc = check_gout(gout, gstride);
    if (rc != PLH_OK) return rc;
    if (WantCount && (!valid_cnt || misaligned(valid_cnt, 8))) return valid_cnt ? PLH_ERR_MISALIGNED : PLH_ERR_NULL_POINTER;
    hipStream_t st = (hipStream_t)stream;
    unsigned long long *cnt = reinterpret_cast<unsigned long long *>(valid_cnt);
    if (WantCount) hipLaunchKernelGGL(lm_zero_count, dim3(1), dim3(1), 0, st, cnt);
    if (n_size * dimsize * m_size == 0) return check_launch();
    if (WantLoss && WantGrad && (!grad || misaligned(grad, 4))) return grad ? PLH_ERR_MISALIGNED : PLH_ERR_NULL_POINTER;

    LmParams p;
    p.P = n_size * m_size;
    p.m_size = m_size;
    p.C = (int)dimsize;
    p.ignore = ignore;
    p.half_lam = lam / 2.f;                          // csrc/large_margin_kernel.cu:188
    p.coeff = 1.f / (float)(dimsize - 1);            // csrc/large_margin_kernel.cu:404
    const float *go_vec = (gout && gstride == 1) ? gout : nullptr;
    switch (pick_shape(dimsize, m_size, x, WantGrad ? grad : nullptr, lab, WantLoss ? loss : nullptr, go_vec)) {
        case Shape::Regs4: launch_regs<4, WantLoss, WantGrad, WantCount>(x, lab, gout, gstride, loss, grad, cnt, p, st); break;
        case Shape::Regs1: launch_regs<1, WantLoss, WantGrad, WantCount>(x, lab, gout, gstride, loss, grad, cnt, p, st); break;
        case Shape::Wave:
            hipLaunchKernelGGL((lm_group<64, WantLoss, WantGrad, WantCount>), dim3(group_grid(p.P, 4)), dim3(256), 0, st,
                               x, lab, gout, gstride, loss, grad, cnt, p);
            break;
        case Shape::Lane:
            hipLaunchKernelGGL((lm_group<1, WantLoss, WantGrad, WantCount>), dim3(group_grid(p.P, 256)), dim3(256), 0, st,
                               x, lab, gout, gstride, loss, grad, cnt, p);
            break;
    }
    return check_launch();
}

}  // namespace plh

extern "C" int plh_lmargin_forward(const float *logits, const int64_t *labels, float *losses,
                                   int64_t n_size, int64_t dimsize, int64_t m_size,
                                   int64_t ignore_index, float lam, void *stream) {
    return plh::launch<true, false, false>(logits, labels, nullptr, 0, losses, nullptr, nullptr, n_size, dimsize,
                                           m_size, ignore_index, lam, stream);
}

extern "C" int plh_lmargin_backward(const float *logits, const int64_t *labels,
                                    const float *grad_output, int64_t grad_output_stride, float *grad_logits,
                                    int64_t n_size, int64_t dimsize, int64_t m_size,
                                    int64_t ignore_index, float lam, void *stream) {
    return plh::launch<false, true, false>(logits, labels, grad_output, grad_output_stride, nullptr, grad_logits,
                                           nullptr, n_size, dimsize, m_size, ignore_index, lam, stream);
}

extern "C" int plh_lmargin_forward_backward(const float *logits, const int64_t *labels, float *losses,
                                            float *grad_logits, int64_t *valid_cnt,
                                            int64_t n_size, int64_t dimsize, int64_t m_size,
                                            int64_t ignore_index, float lam, void *stream) {
    return plh::launch<true, true, true>(logits, labels, nullptr, 0, losses, grad_logits, valid_cnt, n_size,
                                         dimsize, m_size, ignore_index, lam, stream);
}
