// Large-margin softmax cross entropy (Kobayashi, BMVC 2019), forward / backward /
// fused forward+backward, for gfx950: kernels and launchers.
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
#pragma once
#include "plh_common.hpp"

namespace plh {

struct LmParams {
    int64_t P;
    int64_t m_size;
    int C;
    int64_t ignore;
    float half_lam, coeff;
    unsigned xcd_run;   // tile permutation run length (xcd_run_for)
    float *scores;      // forward kernels: if set, also the softmax probability at the label per pixel
    float no_target_score;   // what `scores` gets where a pixel has no target (ignored, label out of range): 1, as the
                             // reference's score pass writes it, or a mark above 1 that the selection tells apart
                        // (1 for a pixel without a target), what the OHEM relabelling ranks
    // lm_regs as the score pass of the OHEM loss (OhemEarly in plh_common.hpp): with `early_kept` the partial sums of a
    // reduced forward run over the pixels that score within `early_thresh` and have a target, their byte mask goes
    // to early_kept and per block the number of pixels whose score, capped at 1, lies within the threshold to early_below
    uint8_t *early_kept = nullptr;
    int *early_below = nullptr;
    float early_thresh = 0.f;
    // (N, C) rows of more than 32 classes: kLmSavedFloats floats per row that the forward leaves (lm_wrow, lm_row)
    // and the backward reads instead of sweeping the row for them (lm_bwd_flat_saved); see lm_saved_applies
    float *saved = nullptr;
};

// What the forward of (N, C) rows leaves per row for the elementwise backward: the maximum m over the classes other than
// the target, 1 / sum exp(x - m) over them, t_all / s_all (which turns exp(x - m) into the full softmax), sum q x, and
// the target's p_y - 1; padded to 32 bytes.
constexpr int kLmSavedFloats = 8;
inline bool lm_saved_applies(size_t elem_bytes, int64_t dimsize, int64_t m_size) {
    if (m_size != 1 || dimsize <= kMaxRegsChannels) return false;
    if (dimsize > kWaveRowCap) return true;     // the block-per-row forward's rows: every element type
    // Rows that a wavefront holds in registers: the elementwise backward runs at 67-82 % of the HBM peak whatever the row
    // length; the backward that recomputes reaches 74-87 % on fp32 rows of a multiple of 32 classes between 96 and 1536
    // and 17-70 % elsewhere (fp32 (262144,300) 0.125 against 0.105 ms), on 16-bit rows 73-75 % at 256, 512 and 1024
    // classes (against 68-70 %) and 17-69 % elsewhere (bf16 (65536,1100) 0.128 against 0.052 ms)
    return elem_bytes != 4 || dimsize % 32 != 0 || dimsize < 96 || dimsize > 1536;
}

// ---------------------------------------------------------------- regs ----

// The target channel is taken out of the non-target statistics by overwriting its widened logit
// with a large negative sentinel: its exponential is an exact 0 and 0 * sentinel stays 0, so the
// inner loops carry no per-channel selects. exp(x - m_no) is evaluated as exp2(u), u = fma(x,
// log2e, -c), c = fl(m_no * log2e); r = m_no*log2e - c (exact, one fma) is what the rounding of c
// left out: it scales every e_j by 2^r, cancels in q_j = e_j / s_no and is taken back out of
// log2(s_no), sum q_j u_j and the rebuilt full sum.
constexpr float kLmMasked = -1e30f;
constexpr unsigned kLmTookEarly = 0x80000000u;      // in launch_typed's block count: the kernel took LmParams::early_*

// Early: the forward as the score pass of the OHEM loss (LmParams::early_*), instances of their own - tested at run time
// inside the pixel loop, the by-products cost the plain forward 5 % ((8,19,1024,1024) fp32: 0.1132 -> 0.1185 ms).
template <class T, int CP, int V, int Form, bool WantLoss, bool WantGrad, bool Early = false>
__global__ __launch_bounds__(kRegsBlock) void lm_regs(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                     const Upstream up,
                                                     float *__restrict__ loss, T *__restrict__ grad,
                                                     unsigned long long *__restrict__ valid_cnt, Partials part,
                                                     const LmParams p) {
    // whether a launch wants the partial sums shows in their pointer: they come from the forward and from the fused
    // pair (the module's 'mean' / 'sum' in one pass), so the backward carries no code for them. (valid_cnt: the fused
    // pair's count of valid pixels comes from a pass over the labels, count_valid_total; the kernels do not touch it.)
    constexpr bool kMayReduce = WantLoss;
    const bool Reduce = kMayReduce && part.sum != nullptr;
    __shared__ float red[4];
    const PixelRef<V, Form> at(p.P, p.m_size, p.C, p.xcd_run);
    const bool live = at.live;
    if (!Reduce && !live) return;

    // labels (and the upstream gradient) before the slice, except in the one-pixel-per-lane backwards on 16-bit
    // elements (see lsr_bwd_regs)
    constexpr bool kLabelsFirst = !(sizeof(T) == 2 && V == 1 && WantGrad);
    int64_t lb[V];
    float go[V];
    typename Pack<T, V>::Raw raw[CP];
    if constexpr (kLabelsFirst) {
        at.labels(lab, p.ignore, lb);
        if constexpr (WantGrad) at.upstream(up, go);
    }
    at.load_slice(x, p.C, p.m_size, raw);
    if constexpr (!kLabelsFirst) {
        at.labels(lab, p.ignore, lb);
        if constexpr (WantGrad) at.upstream(up, go);
    }

    // Four fp32 pixels per lane: a pixel's gradient takes the place of its logits in the slice as soon as it
    // is formed, and the pixels are worked through one after the other (no second array, no four
    // pixels' intermediates alive at once). 16-bit pixels share dwords in pairs and keep the second array.
    constexpr bool kInPlace = (Form == kPerImage) && sizeof(T) == 4;
    float out[V], score[V];
    float g[(WantGrad && !kInPlace) ? CP : 1][V];
    unsigned keep[V];      // all ones for a pixel that counts, 0 for an ignored one
    float mine = 0.f;
    int cnt = 0, below = 0;
    static_assert(!Early || kMayReduce, "the OHEM by-products belong to the forward");
    constexpr bool early = Early;
    bool kp[V];
#pragma unroll
    for (int k = 0; k < V; ++k) {
        bool ign;
        const int tgt = narrow_label(lb[k], p.ignore, p.C, ign);
        keep[k] = ign ? 0u : 0xFFFFFFFFu;
        float xv[CP];
        float sx = 0.f, x_y = -INFINITY;
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (chan_ok<CP>(j, p.C)) {
                const float xj = Pack<T, V>::get(raw[j], k);
                const bool hot = (tgt == j);
                sx += xj;
                x_y = hot ? xj : x_y;
                xv[j] = hot ? kLmMasked : xj;
            }
        float m_no = xv[0];
#pragma unroll
        for (int j = 1; j + 1 < CP - 3; j += 2) m_no = max3(m_no, xv[j], xv[j + 1]);
#pragma unroll
        for (int j = CP - 3; j < CP; ++j)
            if (j > 0 && j < p.C) m_no = max3(m_no, xv[j], xv[j]);
        const float m_all = fmaxf(m_no, x_y);

        //   sum_j (q_j - coeff) log q_j = sum q_j t_j - lse_no - coeff * (sum t_j - others * lse_no),
        //   t_j = x_j - m_no over the non-target channels
        const float c = m_no * kLog2e;
        const float r = __builtin_fmaf(m_no, kLog2e, -c);
        float s_no = 0.f, sum_eu = 0.f;
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (chan_ok<CP>(j, p.C)) {
                const float u = __builtin_fmaf(xv[j], kLog2e, -c);
                const float e = __builtin_amdgcn_exp2f(u);
                s_no += e;
                sum_eu = __builtin_fmaf(e, u, sum_eu);
                if constexpr (WantGrad) xv[j] = e;
            }
        const float inv_no = __builtin_amdgcn_rcpf(s_no);
        const float sum_qt = (sum_eu * inv_no - r) * kLn2;                       // sum q_j t_j
        // full-softmax pieces: s_all = s_no_true * exp(m_no - m_all) + exp(x_y - m_all), s_no_true = s_no * 2^-r
        const float t_all = __builtin_amdgcn_exp2f(__builtin_fmaf(m_no - m_all, kLog2e, -r));
        const float e_y = fast_exp(x_y - m_all);
        const float s_all = __builtin_fmaf(s_no, t_all, e_y);
        if constexpr (WantLoss) {
            const float lse_no = (__builtin_amdgcn_logf(s_no) - r) * kLn2;
            const float others = (float)(p.C - 1 - ((tgt < 0) ? -1 : 0));        // channels that are not the target
            const float sum_t = (sx - ((tgt < 0) ? 0.f : x_y)) - others * m_no;
            const float margin = sum_qt - lse_no - p.coeff * (sum_t - others * lse_no);
            const float acc = p.half_lam * margin - (x_y - m_all) + fast_log(s_all);
            out[k] = (ign || !live) ? 0.f : acc;
            score[k] = (tgt < 0) ? p.no_target_score : fminf(e_y * __builtin_amdgcn_rcpf(s_all), 1.f);
            // formed here: left to itself the compiler moves a pixel's whole reduction down to the guarded
            // stores at the end and keeps every pixel's exponentials alive until then
            asm volatile("" : "+v"(out[k]), "+v"(score[k]));
            if constexpr (kMayReduce) {
                if (early) {
                    kp[k] = live && tgt >= 0 && !(score[k] > p.early_thresh);
                    mine += kp[k] ? out[k] : 0.f;
                    cnt += kp[k] ? 1 : 0;
                    below += (live && fminf(score[k], 1.f) <= p.early_thresh) ? 1 : 0;   // fminf: a NaN score counts as 1
                } else {
                    mine += out[k];
                    cnt += (ign || !live) ? 0 : 1;
                }
            }
        }
        if constexpr (WantGrad) {
            // g_j = gk * (p_j + h * ((x_j + 1 - sum_qx) * q_j - coeff))
            //     = e_j * (x_j * B + A) - K  with  B = h gk / s_no,  A = gk * t_all / s_all + B * (1 - sum_qx),
            //       K = h gk coeff; the target channel takes g_y = gk * (p_y - 1) instead.
            const float inv_all = __builtin_amdgcn_rcpf(s_all);
            const float sum_qx = sum_qt + m_no;
            const float gk = go[k];
            float B = p.half_lam * gk * inv_no;
            float A = __builtin_fmaf(B, 1.f - sum_qx, gk * t_all * inv_all);
            float nK = -p.half_lam * gk * p.coeff;
            float g_hot = (e_y * inv_all - 1.f) * gk;
            asm("" : "+v"(A), "+v"(B), "+v"(nK), "+v"(g_hot));                  // formed per pixel, not per channel
#pragma unroll
            for (int j = 0; j < CP; ++j)
                if (chan_ok<CP>(j, p.C)) {
                    const float w = __builtin_fmaf(Pack<T, V>::get(raw[j], k), B, A);
                    const float gj = __builtin_fmaf(xv[j], w, nK);
                    float gv = (tgt == j) ? g_hot : gj;
                    asm volatile("" : "+v"(gv));        // formed here, not down at the guarded stores
                    if constexpr (kInPlace) {
                        const float one[1] = {gv};
                        Pack<T, V>::set(raw[j], k, one);
                    } else {
                        g[j][k] = gv;
                    }
                }
        }
        if constexpr (kInPlace) __builtin_amdgcn_sched_barrier(0);
    }
    if (live) {
        if (WantLoss && loss) {
            if (early) at.store_f32_cached(loss, out);      // the relabelling pass may read them again
            else at.store_f32(loss, out);
        }
        if (WantLoss && p.scores) at.store_f32_cached(p.scores, score);
        if constexpr (kMayReduce) {
            if (early) store_kept<V>(p.early_kept, at.pix, at.nv, kp);
        }
        if constexpr (WantGrad) {
            // ignored pixels get exact zeros whatever their logits were (the bitwise AND also clears NaN)
            const typename Pack<T, V>::Raw mask = Pack<T, V>::mask(keep);
#pragma unroll
            for (int j = 0; j < CP; ++j)
                if (chan_ok<CP>(j, p.C)) {
                    if constexpr (kInPlace) raw[j] = raw[j] & mask;
                    else raw[j] = Pack<T, V>::put(g[j]) & mask;
                }
            at.store_slice(grad, p.C, p.m_size, raw);
        }
    }
    if (Reduce) {
        const float bs = block_sum_256(mine, red);
        const float bc = block_sum_256((float)cnt, red);
        const float bb = early ? block_sum_256((float)below, red) : 0.f;
        if (threadIdx.x == 0) {
            part.sum[blockIdx.x] = bs;
            part.cnt[blockIdx.x] = (int)bc;
            if (early) p.early_below[blockIdx.x] = (int)bb;
        }
    }
}

// --------------------------------------------------------------- split ----
// 33..256 channels in NCHW (SplitSlice): every wavefront reduces its channels other than the target,
//   m_w = max x_j,  s_w = sum e^(x_j - m_w),  a_w = sum e^(x_j - m_w) (x_j - m_w),  d_w = sum (x_j - m_w),
//   n_w = their number, y_w = the target logit if it is held here,
// and with M = max_w m_w, h_w = m_w - M the parts combine to
//   S_no = sum_w s_w e^h_w,  sum_j e^(x_j - M)(x_j - M) = sum_w e^h_w (a_w + h_w s_w),  sum_j (x_j - M) = sum_w d_w + n_w h_w.
// From there on the formulas are those of lm_regs. Forward: wavefront 0 finishes the pixel; backward:
// every wavefront finishes it and writes the gradient of its own channels.

template <int V>
struct LmSplitStats {
    float m_no, s_no, sum_qt, sum_t, x_y;
};

template <class T, int KW, int V, bool WantSumT, class Slice>
__device__ __forceinline__ void lm_split_parts(const Slice &at, const typename Pack<T, V>::Raw (&raw)[KW],
                                               int k, int rel, float (*parts)[kSplitWaves][kWave * V], int q, int wave) {
    float xv[KW];
    float mx = -INFINITY, x_y = -INFINITY;
    int others = 0;
#pragma unroll
    for (int i = 0; i < KW; ++i) {
        const float xi = Pack<T, V>::get(raw[i], k);
        const bool hot = (rel == i);
        x_y = hot ? xi : x_y;
        xv[i] = (i < at.here && !hot) ? xi : -INFINITY;
        mx = fmaxf(mx, xv[i]);
        others += (i < at.here && !hot) ? 1 : 0;
    }
    // a wavefront that holds nothing but the target has no maximum: its parts must stay neutral
    const float ref = (others > 0) ? mx : 0.f;
    float s = 0.f, a = 0.f, d = 0.f;
#pragma unroll
    for (int i = 0; i < KW; ++i) {
        const float t = xv[i] - ref;                    // -inf for a slot that takes no part
        const float e = fast_exp(t);
        s += e;
        a += (xv[i] > -INFINITY) ? e * t : 0.f;
        if constexpr (WantSumT) d += (xv[i] > -INFINITY) ? t : 0.f;
    }
    parts[0][wave][q] = (others > 0) ? mx : -INFINITY;
    parts[1][wave][q] = s;
    parts[2][wave][q] = a;
    parts[3][wave][q] = x_y;
    if constexpr (WantSumT) {
        parts[4][wave][q] = d;
        parts[5][wave][q] = (float)others;
    }
}

template <int V, bool WantSumT>
__device__ __forceinline__ LmSplitStats<V> lm_split_combine(float (*parts)[kSplitWaves][kWave * V], int q, int used) {
    LmSplitStats<V> r;
    float M = parts[0][0][q];
    for (int w = 1; w < used; ++w) M = fmaxf(M, parts[0][w][q]);
    float S = 0.f, A = 0.f, D = 0.f, x_y = -INFINITY;
    for (int w = 0; w < used; ++w) {
        const float m_w = parts[0][w][q];
        x_y = fmaxf(x_y, parts[3][w][q]);
        if (m_w == -INFINITY) continue;                 // nothing but the target there
        const float h = m_w - M;
        const float eh = fast_exp(h);
        const float s_w = parts[1][w][q];
        S = __builtin_fmaf(s_w, eh, S);
        A = __builtin_fmaf(eh, __builtin_fmaf(h, s_w, parts[2][w][q]), A);
        if constexpr (WantSumT) D += __builtin_fmaf(parts[5][w][q], h, parts[4][w][q]);
    }
    r.m_no = M;
    r.s_no = S;
    r.sum_qt = A * __builtin_amdgcn_rcpf(S);
    r.sum_t = D;
    r.x_y = x_y;
    return r;
}

template <class T, int KW, int V, bool PerImage = false>
__global__ __launch_bounds__(kSplitBlock) void lm_fwd_split(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                           float *__restrict__ loss, Partials part, const LmParams p) {
    const bool Reduce = part.sum != nullptr;
    __shared__ float parts[6][kSplitWaves][kWave * V];
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
            lm_split_parts<T, KW, V, true>(at, raw, k, rel, parts, lane * V + k, wave);
        }
    }
    __syncthreads();
    if (wave >= V) return;                              // wavefront k finishes pixel k of every lane 
    const int used = (p.C + KW - 1) / KW;
    bool ign;
    PLH_SPLIT_MY_LABEL(my_lb, lb, wave, V)
    const int tgt = narrow_label(my_lb, p.ignore, p.C, ign);
    const LmSplitStats<V> st = lm_split_combine<V, true>(parts, lane * V + wave, used);
    const float m_all = fmaxf(st.m_no, st.x_y);
    const float t_all = fast_exp(st.m_no - m_all);
    const float e_y = fast_exp(st.x_y - m_all);
    const float s_all = __builtin_fmaf(st.s_no, t_all, e_y);
    const float lse_no = fast_log(st.s_no);
    const float others = (float)(p.C - 1 - ((tgt < 0) ? -1 : 0));
    const float margin = st.sum_qt - lse_no - p.coeff * (st.sum_t - others * lse_no);
    const float acc = p.half_lam * margin - (st.x_y - m_all) + fast_log(s_all);
    const bool here = at.live && wave < at.nv;
    const bool valid = here && !ign;
    const float out = valid ? acc : 0.f;
    if (here && loss) loss[at.pix + wave] = out;
    if (here && p.scores) p.scores[at.pix + wave] = (tgt < 0) ? p.no_target_score : fminf(e_y * __builtin_amdgcn_rcpf(s_all), 1.f);
    if (Reduce) split_block_partials<V>(out, valid, wave, lane, part);
}

template <class T, int KW, int V, bool PerImage = false>
__global__ __launch_bounds__(kSplitBlock) void lm_bwd_split(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                           const Upstream up, T *__restrict__ grad, const LmParams p) {
    __shared__ float parts[4][kSplitWaves][kWave * V];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const SplitSlice<T, V, KW, PerImage> at(p.P, p.m_size, p.C, p.xcd_run);
    using PK = Pack<T, V>;
    typename PK::Raw raw[KW];
    int64_t lb[V];
    float go[V];
    if (at.here > 0) {                                  // wave-uniform
        at.load(x, p.C, p.m_size, raw);
        at.labels(lab, p.ignore, lb);
        at.upstream(up, go);
#pragma unroll
        for (int k = 0; k < V; ++k) {
            bool ign;
            const int rel = narrow_label(lb[k], p.ignore, p.C, ign) - at.first;
            lm_split_parts<T, KW, V, false>(at, raw, k, rel, parts, lane * V + k, wave);
        }
    }
    __syncthreads();
    if (at.here == 0 || !at.live) return;
    const int used = (p.C + KW - 1) / KW;
    unsigned keep[V];
#pragma unroll
    for (int k0 = 0; k0 < V; k0 += PK::kStep) {
        float g[KW][PK::kStep];
#pragma unroll
        for (int kk = 0; kk < PK::kStep; ++kk) {
            const int k = k0 + kk;
            bool ign;
            const int rel = narrow_label(lb[k], p.ignore, p.C, ign) - at.first;
            keep[k] = ign ? 0u : 0xFFFFFFFFu;
            const LmSplitStats<V> st = lm_split_combine<V, false>(parts, lane * V + k, used);
            const float m_all = fmaxf(st.m_no, st.x_y);
            const float t_all = fast_exp(st.m_no - m_all);
            const float e_y = fast_exp(st.x_y - m_all);
            const float s_all = __builtin_fmaf(st.s_no, t_all, e_y);
            const float inv_all = __builtin_amdgcn_rcpf(s_all);
            const float sum_qx = st.sum_qt + st.m_no;
            const float gk = go[k];
            // g_j = e_j (x_j B + A) - K, e_j = e^(x_j - m_no); the target takes g_y = gk (p_y - 1): see lm_regs
            float B = p.half_lam * gk * __builtin_amdgcn_rcpf(st.s_no);
            float A = __builtin_fmaf(B, 1.f - sum_qx, gk * t_all * inv_all);
            float nK = -p.half_lam * gk * p.coeff;
            float g_hot = (e_y * inv_all - 1.f) * gk;
            asm("" : "+v"(A), "+v"(B), "+v"(nK), "+v"(g_hot));                  // formed per pixel, not per channel
#pragma unroll
            for (int i = 0; i < KW; ++i) {
                const float xi = PK::get(raw[i], k);
                const float e = fast_exp(xi - st.m_no);
                const float gj = __builtin_fmaf(e, __builtin_fmaf(xi, B, A), nK);
                g[i][kk] = (rel == i) ? g_hot : gj;
            }
        }
#pragma unroll
        for (int i = 0; i < KW; ++i) PK::set(raw[i], k0 / PK::kStep, g[i]);
    }
    const typename PK::Raw mask = PK::mask(keep);
#pragma unroll
    for (int i = 0; i < KW; ++i) raw[i] = raw[i] & mask;
    at.store(grad, p.m_size, raw);
}

// --------------------------------------------------------------- group ----
// G lanes per pixel, striding over its channels; three sweeps, the later ones re-reading what the first
// pulled into cache. Launched with G = 1: a lane per pixel, for channel counts no other shape takes.

template <class T, int G, bool WantLoss, bool WantGrad>
__global__ __launch_bounds__(256) void lm_group(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                const Upstream up,
                                                float *__restrict__ loss, T *__restrict__ grad,
                                                unsigned long long *__restrict__ valid_cnt, Partials part,
                                                const LmParams p) {
    // whether a launch wants the partial sums shows in their pointer: they come from the forward and from the fused
    // pair (the module's 'mean' / 'sum' in one pass), so the backward carries no code for them. (valid_cnt: the fused
    // pair's count of valid pixels comes from a pass over the labels, count_valid_total; the kernels do not touch it.)
    constexpr bool kMayReduce = WantLoss;
    const bool Reduce = kMayReduce && part.sum != nullptr;
    constexpr int kPix = 256 / G;
    __shared__ float red[4];
    float mine = 0.f, cnt = 0.f;
    const int sub = threadIdx.x % G;
    const int grp = threadIdx.x / G;

    const int64_t rounds = ceil_div_dev(p.P, (int64_t)gridDim.x * kPix);
    for (int64_t r = 0; r < rounds; ++r) {
        const int64_t pix = (r * gridDim.x + blockIdx.x) * kPix + grp;
        const bool live = pix < p.P;
        const int64_t pc = live ? pix : 0;
        const int64_t n = pc / p.m_size;
        const int64_t base = pc + n * (int64_t)(p.C - 1) * p.m_size;
        const T *xs = x + base;
        const int64_t lb = lab[pc];
        const bool ign = (lb == p.ignore);
        float go[1] = {1.f};
        if constexpr (WantGrad) load_upstream<1>(up, pc, go);

        float m_no = -INFINITY, x_y = -INFINITY;
#pragma unroll kGroupUnroll<G>
        for (int j = sub; j < p.C; j += G) {
            const float t = load_one(xs + (int64_t)j * p.m_size);
            if (lb == j) x_y = t; else m_no = fmaxf(m_no, t);
        }
        m_no = group_reduce<G>(m_no, OpMax());
        x_y = group_reduce<G>(x_y, OpMax());
        const float m_all = fmaxf(m_no, x_y);
        float s_no = 0.f, sum_ex = 0.f;
#pragma unroll kGroupUnroll<G>
        for (int j = sub; j < p.C; j += G) {
            const float t = load_one(xs + (int64_t)j * p.m_size);
            const float e = (lb == j) ? 0.f : fast_exp(t - m_no);
            s_no += e;
            sum_ex += e * t;
        }
        s_no = group_reduce<G>(s_no, OpSum());
        sum_ex = group_reduce<G>(sum_ex, OpSum());
        const float t_all = fast_exp(m_no - m_all);
        const float e_y = fast_exp(x_y - m_all);
        const float s_all = s_no * t_all + e_y;
        const float inv_no = 1.f / s_no, inv_all = 1.f / s_all;
        const float sum_qx = sum_ex * inv_no;
        const float lse_no = logf(s_no);
        float acc = 0.f;
#pragma unroll kGroupUnroll<G>
        for (int j = sub; j < p.C; j += G) {
            const float xv = load_one(xs + (int64_t)j * p.m_size);
            const bool hot = (lb == j);
            const float e = fast_exp(xv - m_no);
            const float q = e * inv_no;
            if constexpr (WantLoss) acc += hot ? 0.f : p.half_lam * (q - p.coeff) * ((xv - m_no) - lse_no);
            if constexpr (WantGrad) {
                const float g_hot = e_y * inv_all - 1.f;
                const float g_cold = e * t_all * inv_all + p.half_lam * ((xv + 1.f - sum_qx) * q - p.coeff);
                if (live) store_one(grad + (base + (int64_t)j * p.m_size), ign ? 0.f : (hot ? g_hot : g_cold) * go[0]);
            }
        }
        if constexpr (WantLoss) {
            acc = group_reduce<G>(acc, OpSum());
            acc += -(x_y - m_all) + logf(s_all);
            if (live && sub == 0) {
                if (loss) loss[pix] = ign ? 0.f : acc;
                if (p.scores) p.scores[pix] = (ign || lb < 0 || lb >= p.C) ? p.no_target_score : fminf(e_y * inv_all, 1.f);
                mine += ign ? 0.f : acc;
                cnt += ign ? 0.f : 1.f;
            }
        }
        // every lane of the wave is inside the loop, so the ballot sees the whole wave
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
// (N, C) inputs with 33..2048 channels: the row sits in the wavefront's registers (WaveRow), so the three
// sweeps of the group kernel (maxima, sums, terms) read HBM once. Same arithmetic as lm_group.

template <class T, int NI, int LP, bool WantLoss, bool WantGrad, int G, bool Cached = false>
__global__ __launch_bounds__(256) void lm_wrow(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                               const Upstream up, float *__restrict__ loss, T *__restrict__ grad,
                                               unsigned long long *__restrict__ valid_cnt, Partials part,
                                               const LmParams p) {
    // whether a launch wants the partial sums shows in their pointer: they come from the forward and from the fused
    // pair (the module's 'mean' / 'sum' in one pass), so the backward carries no code for them. (valid_cnt: the fused
    // pair's count of valid pixels comes from a pass over the labels, count_valid_total; the kernels do not touch it.)
    constexpr bool kMayReduce = WantLoss;
    const bool Reduce = kMayReduce && part.sum != nullptr;
    __shared__ float red[4];
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
        const int64_t lb = lab[row];
        const bool ign = (lb == p.ignore);
        const int tgt = (lb >= 0 && lb < p.C) ? (int)lb : -1;
        float go[1] = {1.f};
        if constexpr (WantGrad) load_upstream<1>(up, row, go);

        // The target leaves the row: with -inf in its slot, as in the slots beyond the row, the sweeps over
        // "the other channels" need no mask of their own (exp gives 0, the linear terms test for -inf).
        const float x_y = (tgt >= 0) ? load_one(xs + tgt) : -INFINITY;
        float m_no = -INFINITY;
#pragma unroll
        for (int i = 0; i < NI; ++i)
#pragma unroll
            for (int l = 0; l < L; ++l) {
                const bool hot = ((lane + G * i) * L + l == tgt);
                r.v[i][l] = hot ? -INFINITY : r.v[i][l];
                m_no = fmaxf(m_no, r.v[i][l]);
            }
        m_no = group_reduce<G>(m_no, OpMax());
        const float m_all = fmaxf(m_no, x_y);
        // Without gradients the margin term needs no third sweep: with d = x - m_no over the channels other
        // than the target, sum (q - coeff) (d - lse_no) = (sum e d) / s_no - lse_no - coeff (sum d - n lse_no).
        constexpr bool kClosed = WantLoss && !WantGrad;
        float s_no = 0.f, sum_ex = 0.f, sum_d = 0.f;
        int finite_slots = 0;                   // wave-uniform: slots of the wavefront's rows that hold a finite logit
#pragma unroll
        for (int i = 0; i < NI; ++i)
#pragma unroll
            for (int l = 0; l < L; ++l) {
                const float t = r.v[i][l];
                const float d = t - m_no;
                const float e = fast_exp(d);
                const bool in = d > -INFINITY;
                s_no += e;
                if constexpr (kClosed) {
                    const float dz = in ? d : 0.f;
                    sum_ex = __builtin_fmaf(e, dz, sum_ex);
                    sum_d += dz;
                    finite_slots += __builtin_popcountll(__builtin_amdgcn_ballot_w64(in));   // scalar unit: the vote exists already
                } else {
                    sum_ex = __builtin_fmaf(e, in ? t : 0.f, sum_ex);
                }
            }
        s_no = group_reduce<G>(s_no, OpSum());
        sum_ex = group_reduce<G>(sum_ex, OpSum());
        if constexpr (kClosed) sum_d = group_reduce<G>(sum_d, OpSum());
        const float t_all = fast_exp(m_no - m_all);
        const float e_y = fast_exp(x_y - m_all);
        const float s_all = s_no * t_all + e_y;
        const float inv_no = 1.f / s_no, inv_all = 1.f / s_all;
        const float sum_qx = sum_ex * inv_no;
        const float lse_no = logf(s_no);
        const float g_hot = (e_y * inv_all - 1.f) * go[0];
        float acc = 0.f;
        // The closed form counts every channel other than the target as a finite term. A row with a logit of -inf
        // among them (a masked class) has a term (0 - coeff) * log 0 instead, which the sweep below evaluates as
        // the kernels with gradients do; whether any row of this wavefront has one shows in the number of finite
        // slots, which the votes above counted on the scalar unit.
        bool closed = kClosed;
        if constexpr (kClosed) {
            const int with_target = __builtin_popcountll(__builtin_amdgcn_ballot_w64(tgt >= 0)) / G;
            closed = finite_slots == (kWave / G) * p.C - with_target;      // wave-uniform
            const float n_no = (float)(p.C - (tgt >= 0 ? 1 : 0));
            acc = p.half_lam * (sum_ex * inv_no - lse_no - p.coeff * (sum_d - n_no * lse_no));
            if (!closed) acc = 0.f;
        }
        if constexpr (kClosed) {
            // (read again from memory, one element per lane and step: with the registers' values the compiler keeps the
            // exponentials of the sweep above alive for this path, and the registers that costs the common path up to half
            // its speed - fp32 (65536,1100) forward 0.086 -> 0.055 ms without it)
            if (!closed) {
#pragma nounroll
                for (int j = lane; j < p.C; j += G) {
                    const float xv = load_one(xs + j);
                    const float q = fast_exp(xv - m_no) * inv_no;
                    acc += (j == tgt) ? 0.f : p.half_lam * (q - p.coeff) * ((xv - m_no) - lse_no);
                }
            }
        } else {
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int e0 = (lane + G * i) * L;
            const bool ok = e0 < p.C;
            float g[L];
#pragma unroll
            for (int l = 0; l < L; ++l) {
                const float xv = r.v[i][l];
                const bool hot = (e0 + l == tgt);
                const float e = fast_exp(xv - m_no);
                const float q = e * inv_no;
                if constexpr (WantLoss)
                    acc += (hot || !ok) ? 0.f : p.half_lam * (q - p.coeff) * ((xv - m_no) - lse_no);
                if constexpr (WantGrad) {
                    const float g_cold = (e * t_all * inv_all + p.half_lam * ((xv + 1.f - sum_qx) * q - p.coeff)) * go[0];
                    g[l] = ign ? 0.f : (hot ? g_hot : g_cold);
                }
            }
            if constexpr (WantGrad) {
                if (ok && live) {
                    if constexpr (Span::kUse) Span::stage(tile, p.C, at.grp, e0, g);
                    else RowPiece<T, L>::template store<Cached>(grad + row * p.C + e0, g);
                }
            }
        }
        }
        if constexpr (WantGrad && Span::kUse) {
            const int64_t left = p.P - r0;
            Span::flush(tile, grad + r0 * p.C, left < Span::kRows ? (int)left : Span::kRows, p.C);
        }
        if constexpr (WantLoss) {
            if (!closed) acc = group_reduce<G>(acc, OpSum());
            acc += -(x_y - m_all) + logf(s_all);
            if (lane == 0 && live) {
                if (loss) {
                    if (kClosed && loss == p.saved) {       // the slot takes the row's statistics (LmParams::saved)
                        plh_f4 *to = reinterpret_cast<plh_f4 *>(loss + row * kLmSavedFloats);
                        to[0] = plh_f4{m_no, inv_no, t_all * inv_all, sum_qx + m_no};     // here sum_qx is sum q (x - m_no)
                        to[1] = plh_f4{e_y * inv_all - 1.f, 0.f, 0.f, 0.f};
                    } else {
                        loss[row] = ign ? 0.f : acc;
                    }
                }
                if (p.scores) p.scores[row] = (ign || tgt < 0) ? p.no_target_score : fminf(e_y * inv_all, 1.f);
                mine += ign ? 0.f : acc;
                cnt += ign ? 0.f : 1.f;
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

// ------------------------------------------------------- a block per row ----
// (N, C) inputs with rows of more than 2048 channels: a 1024-thread block per row at a time. One sweep
// with running statistics over the channels other than the target -- maximum, sum e, sum e*x (rescaled
// when the maximum moves) and sum x -- gives the loss in closed form:
//   sum_{j != y} (q_j - c) log q_j = (sum q_j x_j - m - lse) - c * (sum x_j - n * (m + lse)),  log q_j = x_j - m - lse;
// the backward sweeps the row a second time (from cache for all but the longest rows) to write the gradient.

struct LmRowStats { float m, s, ex, sx; };

// Four block-wide reductions per row: the small block pays at every length measured ((8192, 32000) fp32
// fwd+bwd 0.66 ms with 256 threads, 0.79 ms with 1024; (8192, 16384) 0.34 against 0.51 ms).
constexpr int kLmRowShortMax = 1 << 30;

// MayHot: whether the target can be among these L elements. A chunk that cannot hold it (all but one chunk of a row, and
// the caller knows which) carries no per-element test for it: the 16-bit rows are bound by instruction issue, and the
// tests were a third of the loop (bf16 (8192,32000) forward 0.131 -> 0.110 ms).
template <int L, bool MayHot>
__device__ __forceinline__ void lm_row_absorb_as(const float (&v)[L], int idx0, int tgt, LmRowStats &st) {
    float cm = -INFINITY;
#pragma unroll
    for (int i = 0; i < L; ++i) cm = (MayHot && idx0 + i == tgt) ? cm : fmaxf(cm, v[i]);
    if (cm > st.m) {
        const float f = fast_exp(st.m - cm);           // 0 on the first chunk
        st.s *= f;
        st.ex *= f;
        st.m = cm;
    }
#pragma unroll
    for (int i = 0; i < L; ++i) {
        const bool hot = MayHot && (idx0 + i == tgt);
        const float e = hot ? 0.f : fast_exp(v[i] - st.m);
        st.s += e;
        // e is 0 for the target and for a masked (-inf) logit: clamping the logit keeps 0 * -inf out of the sum,
        // while the plain sum below still turns -inf, so that a masked class gives the (0 - coeff) * log 0 = +inf
        // of the per-element form
        st.ex = __builtin_fmaf(e, fmaxf(v[i], -3.0e38f), st.ex);
        st.sx += hot ? 0.f : v[i];
    }
}

template <int L>
__device__ __forceinline__ void lm_row_absorb(const float (&v)[L], int idx0, int tgt, LmRowStats &st) {
    if (tgt >= idx0 && tgt < idx0 + L) lm_row_absorb_as<L, true>(v, idx0, tgt, st);
    else lm_row_absorb_as<L, false>(v, idx0, tgt, st);
}

template <class T>
__device__ __forceinline__ LmRowStats lm_row_sweep(const T *xs, int C, int tgt, bool aligned, float *lds) {
    constexpr int L = RowChunk<T>::kLen;
    const RowSplit<T> sp(xs, C, aligned);
    LmRowStats st{-INFINITY, 0.f, 0.f, 0.f};
    const T *body = xs + sp.head;
    int i = threadIdx.x;
    for (; i + 3 * row_threads() < sp.chunks; i += 4 * row_threads()) {
        float v[4][L];
#pragma unroll
        for (int u = 0; u < 4; ++u) RowChunk<T>::load(body + (int64_t)(i + u * row_threads()) * L, v[u]);
#pragma unroll
        for (int u = 0; u < 4; ++u) lm_row_absorb<L>(v[u], sp.head + (i + u * row_threads()) * L, tgt, st);
    }
    for (; i < sp.chunks; i += row_threads()) {
        float v[L];
        RowChunk<T>::load(body + (int64_t)i * L, v);
        lm_row_absorb<L>(v, sp.head + i * L, tgt, st);
    }
    for (int j = threadIdx.x; j < sp.head; j += row_threads()) {
        const float v[1] = {load_one(xs + j)};
        lm_row_absorb<1>(v, j, tgt, st);
    }
    for (int j = sp.tail_from + threadIdx.x; j < C; j += row_threads()) {
        const float v[1] = {load_one(xs + j)};
        lm_row_absorb<1>(v, j, tgt, st);
    }
    // One exchange through LDS per row instead of four block-wide reductions (eight barriers): every wavefront brings
    // its lanes to the wavefront's maximum and adds them up across lanes, leaves its four numbers in LDS, and every
    // thread combines the wavefronts' sets itself, in a fixed order ((65536,3000) fp32 forward 0.267 -> 0.251 ms,
    // (8192,32000) bf16 0.145 -> 0.132).
    // lds: 4 floats per wavefront of the block.
    const float mw = group_reduce<64>(st.m, OpMax());
    const float f = (st.m == -INFINITY) ? 0.f : fast_exp(st.m - mw);
    const float sw = group_reduce<64>(st.s * f, OpSum());
    const float exw = group_reduce<64>(st.ex * f, OpSum());
    const float sxw = group_reduce<64>(st.sx, OpSum());
    if ((threadIdx.x & 63) == 0) {
        float *mine = lds + 4 * (threadIdx.x >> 6);
        mine[0] = mw; mine[1] = sw; mine[2] = exw; mine[3] = sxw;
    }
    __syncthreads();
    const int waves = row_threads() / 64;
    LmRowStats r{lds[0], 0.f, 0.f, 0.f};
    for (int w = 1; w < waves; ++w) r.m = fmaxf(r.m, lds[4 * w]);
    for (int w = 0; w < waves; ++w) {
        const float fw = (lds[4 * w] == -INFINITY) ? 0.f : fast_exp(lds[4 * w] - r.m);
        r.s = __builtin_fmaf(lds[4 * w + 1], fw, r.s);
        r.ex = __builtin_fmaf(lds[4 * w + 2], fw, r.ex);
        r.sx += lds[4 * w + 3];
    }
    __syncthreads();                    // before the next row's wavefronts write their numbers
    return r;
}

template <class T, bool WantLoss, bool WantGrad>
__global__ __launch_bounds__(kRowBlock) void lm_row(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                    const Upstream up, float *__restrict__ loss, T *__restrict__ grad,
                                                    unsigned long long *__restrict__ valid_cnt, Partials part,
                                                    const LmParams p, int vec_flags) {
    // whether a launch wants the partial sums shows in their pointer: they come from the forward and from the fused
    // pair (the module's 'mean' / 'sum' in one pass), so the backward carries no code for them. (valid_cnt: the fused
    // pair's count of valid pixels comes from a pass over the labels, count_valid_total; the kernels do not touch it.)
    // vec_flags: bit 0 - rows can be walked in 16-byte chunks; bit 1 - `loss` takes kLmSavedFloats statistics per row
    // instead of the row's loss (LmParams::saved: the reduced forward writes no per-row losses, so the slot serves)
    constexpr bool kMayReduce = WantLoss;
    const bool Reduce = kMayReduce && part.sum != nullptr;
    const int vec = vec_flags & 1;
    __shared__ float red[4 * (kRowBlock / 64)];
    constexpr int L = RowChunk<T>::kLen;
    float mine = 0.f;
    int cnt = 0;
    for (int64_t row = blockIdx.x; row < p.P; row += gridDim.x) {       // block-uniform
        const T *xs = x + row * p.C;
        const int64_t lb = lab[row];
        const bool ign = (lb == p.ignore);
        const int tgt = (lb >= 0 && lb < p.C) ? (int)lb : -1;
        const LmRowStats st = lm_row_sweep<T>(xs, p.C, tgt, vec != 0, red);
        const float x_y = (tgt >= 0) ? load_one(xs + tgt) : -INFINITY;
        const float m_all = fmaxf(st.m, x_y);
        const float t_all = fast_exp(st.m - m_all);
        const float e_y = fast_exp(x_y - m_all);
        const float s_all = st.s * t_all + e_y;
        const float inv_no = 1.f / st.s, inv_all = 1.f / s_all;
        const float sum_qx = st.ex * inv_no;
        const float lse_no = logf(st.s);
        if constexpr (WantLoss) {
            if (threadIdx.x == 0) {
                const float n_no = (float)(p.C - (tgt >= 0 ? 1 : 0));
                const float off = st.m + lse_no;
                const float margin = p.half_lam * ((sum_qx - off) - p.coeff * (st.sx - n_no * off));
                const float acc = margin - (x_y - m_all) + logf(s_all);
                if (loss) {
                    if (vec_flags & 2) {
                        plh_f4 *to = reinterpret_cast<plh_f4 *>(loss + row * kLmSavedFloats);
                        to[0] = plh_f4{st.m, inv_no, t_all * inv_all, sum_qx};
                        to[1] = plh_f4{e_y * inv_all - 1.f, 0.f, 0.f, 0.f};
                    } else {
                        loss[row] = ign ? 0.f : acc;
                    }
                }
                if (p.scores) p.scores[row] = (ign || tgt < 0) ? p.no_target_score : fminf(e_y * inv_all, 1.f);
                mine += ign ? 0.f : acc;
                cnt += ign ? 0 : 1;
            }
        }
        if constexpr (WantGrad) {
            float go[1];
            load_upstream<1>(up, row, go);
            const float gk = ign ? 0.f : go[0];
            const float g_hot = (e_y * inv_all - 1.f) * gk;
            const float k_all = t_all * inv_all;
            T *gs = grad + row * p.C;
            auto one = [&](float xv, int j) {
                const float e = fast_exp(xv - st.m);
                const float q = e * inv_no;
                const float g_cold = (e * k_all + p.half_lam * ((xv + 1.f - sum_qx) * q - p.coeff)) * gk;
                return ign ? 0.f : ((j == tgt) ? g_hot : g_cold);
            };
            const RowSplit<T> sp(xs, p.C, vec != 0);     // the gradient row sits at the same offset from its own boundary
            for (int i = threadIdx.x; i < sp.chunks; i += row_threads()) {
                float v[L];
                RowChunk<T>::load(xs + sp.head + (int64_t)i * L, v);
#pragma unroll
                for (int e = 0; e < L; ++e) v[e] = one(v[e], sp.head + i * L + e);
                RowChunk<T>::store(gs + sp.head + (int64_t)i * L, v);
            }
            for (int j = threadIdx.x; j < sp.head; j += row_threads()) store_one(gs + j, one(load_one(xs + j), j));
            for (int j = sp.tail_from + threadIdx.x; j < p.C; j += row_threads()) store_one(gs + j, one(load_one(xs + j), j));
        }
    }
    if (Reduce) {
        if (threadIdx.x == 0) {
            part.sum[blockIdx.x] = mine;
            part.cnt[blockIdx.x] = cnt;
        }
    }
}

// Backward of long rows from the statistics the forward left (LmParams::saved), elementwise over the flattened
// (rows x classes) tensor like lsr_bwd_flat_lse: a block takes 512 consecutive 16-byte chunks wherever rows begin and
// end; the arithmetic per element is lm_row's. Logits and gradient on 16-byte boundaries, one scalar upstream
// gradient, optionally the byte mask of an OHEM selection.
template <class T>
__global__ __launch_bounds__(256) void lm_bwd_flat_saved(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                         const Upstream up, T *__restrict__ grad, const LmParams p,
                                                         int64_t chunks) {
    constexpr int L = RowChunk<T>::kLen, U = kFlatChunks;
    float gk0 = up.gout ? *up.gout * up.scale : up.scale;
    if (up.divide_by) gk0 = gk0 / (float)(*up.divide_by);
    const int64_t first = (int64_t)blockIdx.x * (256 * U);
    const int64_t row0 = first * L / p.C;                               // block-uniform
    const unsigned col0 = (unsigned)(first * L - row0 * p.C);
    const unsigned C = (unsigned)p.C;
    struct RowTerms { float m, inv_no, k_all, sum_qx, g_hot, gk; int tgt; bool dropped; };
    auto row_terms = [&](int64_t r) {
        RowTerms t;
        const int64_t lb = lab[r];
        t.dropped = lb == p.ignore || (up.keep && up.keep[r] == 0);
        t.gk = t.dropped ? 0.f : gk0;
        const plh_f4 *from = reinterpret_cast<const plh_f4 *>(p.saved + r * kLmSavedFloats);
        const plh_f4 a = from[0];
        t.m = a.x; t.inv_no = a.y; t.k_all = a.z; t.sum_qx = a.w;
        t.g_hot = p.saved[r * kLmSavedFloats + 4] * t.gk;
        t.tgt = (lb >= 0 && lb < p.C) ? (int)lb : -1;
        return t;
    };
    auto one = [&](float xv, int j, const RowTerms &t) {
        const float e = fast_exp(xv - t.m);
        const float q = e * t.inv_no;
        const float g_cold = (e * t.k_all + p.half_lam * ((xv + 1.f - t.sum_qx) * q - p.coeff)) * t.gk;
        return t.dropped ? 0.f : ((j == t.tgt) ? t.g_hot : g_cold);
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
#pragma unroll
            for (int e = 0; e < L; ++e) v[u][e] = one(v[u][e], (int)(col + e), t);
        } else {                                        // the chunk crosses into the next row
#pragma unroll
            for (int e = 0; e < L; ++e) {
                if (col + e == C) {
                    row += 1;
                    col -= C;                           // wraps: col + e becomes 0 for this element
                    t = row_terms(row);
                }
                v[u][e] = one(v[u][e], (int)(col + e), t);
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

static __global__ void lm_zero_count(unsigned long long *cnt) { *cnt = 0; }

// ------------------------------------------------------------ dispatch ----

template <class T, int V, bool WantLoss, bool WantGrad>
static unsigned launch_regs(const T *x, const int64_t *lab, const Upstream &up, float *loss, T *grad,
                            unsigned long long *cnt, Partials part, const LmParams &p, hipStream_t st) {
    const unsigned grid = regs_grid<V>(p.P);
    const bool uni = tiles_are_uniform(p.m_size, V, sizeof(T));
    const bool early = WantLoss && !WantGrad && p.early_kept && part.sum;
    switch ((p.C + 3) / 4) {
#define PLH_CASE(K)                                                                                                  \
    case K:                                                                                                          \
        if constexpr (WantLoss && !WantGrad) {                                                                       \
            if (early) {                                                                                             \
                if (V * sizeof(T) == 8 && uni)                                                                       \
                    hipLaunchKernelGGL((lm_regs<T, 4 * K, V, (V * sizeof(T) == 8 ? kUniform : kGeneral), true, false, true>), \
                                       dim3(grid), dim3(kRegsBlock), 0, st, x, lab, up, loss, grad, cnt, part, p);    \
                else                                                                                                 \
                    hipLaunchKernelGGL((lm_regs<T, 4 * K, V, kGeneral, true, false, true>), dim3(grid),              \
                                       dim3(kRegsBlock), 0, st, x, lab, up, loss, grad, cnt, part, p);               \
                break;                                                                                               \
            }                                                                                                        \
        }                                                                                                            \
        if constexpr (V * sizeof(T) == 8) {                                                                          \
            if (uni) {                                                                                               \
                hipLaunchKernelGGL((lm_regs<T, 4 * K, V, kUniform, WantLoss, WantGrad>), dim3(grid),  \
                                   dim3(kRegsBlock), 0, st, x, lab, up, loss, grad, cnt, part, p);                   \
                break;                                                                                               \
            }                                                                                                        \
        }                                                                                                            \
        hipLaunchKernelGGL((lm_regs<T, 4 * K, V, kGeneral, WantLoss, WantGrad>), dim3(grid),         \
                           dim3(kRegsBlock), 0, st, x, lab, up, loss, grad, cnt, part, p);                           \
        break;
        PLH_CASE(1) PLH_CASE(2) PLH_CASE(3) PLH_CASE(4) PLH_CASE(5) PLH_CASE(6) PLH_CASE(7) PLH_CASE(8)
#undef PLH_CASE
    }
    return grid;
}

// NCHW whose channel planes start on element boundaries only (odd lengths): the per-image form, four
// pixels per lane.
template <class T, bool WantLoss, bool WantGrad>
static unsigned launch_image(const T *x, const int64_t *lab, const Upstream &up, float *loss, T *grad,
                             unsigned long long *cnt, Partials part, const LmParams &p, hipStream_t st) {
    const unsigned grid = image_grid<4>(p.P / p.m_size, p.m_size);
    const bool early = WantLoss && !WantGrad && p.early_kept && part.sum;
    switch ((p.C + 3) / 4) {
#define PLH_CASE(K)                                                                                                  \
    case K:                                                                                                          \
        if constexpr (4 * K <= kImageFormMaxChannels<T>) {                                                           \
            if constexpr (WantLoss && !WantGrad) {                                                                   \
                if (early) {                                                                                         \
                    hipLaunchKernelGGL((lm_regs<T, 4 * K, 4, kPerImage, true, false, true>), dim3(grid),             \
                                       dim3(kRegsBlock), 0, st, x, lab, up, loss, grad, cnt, part, p);               \
                    break;                                                                                           \
                }                                                                                                    \
            }                                                                                                        \
            hipLaunchKernelGGL((lm_regs<T, 4 * K, 4, kPerImage, WantLoss, WantGrad>), dim3(grid),                    \
                               dim3(kRegsBlock), 0, st, x, lab, up, loss, grad, cnt, part, p);                       \
        }                                                                                                            \
        break;
        PLH_CASE(1) PLH_CASE(2) PLH_CASE(3) PLH_CASE(4) PLH_CASE(5) PLH_CASE(6) PLH_CASE(7) PLH_CASE(8)
#undef PLH_CASE
    }
    return grid;
}

template <class T, bool WantLoss, bool WantGrad>
unsigned launch_typed(const T *x, const int64_t *lab, const Upstream &up, float *loss, T *grad,
                             unsigned long long *cnt, Partials part, const LmParams &p, hipStream_t st) {
    constexpr int V = ElemTraits<T>::kVec;
    const float *go_vec = (up.gout && up.stride == 1) ? up.gout : nullptr;
    const float *second_f32 = go_vec ? go_vec : p.scores;      // the score output belongs to forwards without upstream
    unsigned blocks = 0;
    if constexpr (WantGrad && !WantLoss) {
        // long rows, from the statistics the forward left: elementwise over the flattened tensor
        constexpr int L = RowChunk<T>::kLen;
        const int64_t chunks = p.P * p.C / L, flat_blocks = ceil_div(chunks, (int64_t)(256 * kFlatChunks));
        if (p.saved && !go_vec && lm_saved_applies(sizeof(T), p.C, p.m_size) && !misaligned(x, 16) && !misaligned(grad, 16) &&
            flat_blocks >= 1 && flat_blocks < ((int64_t)1 << 31)) {
            hipLaunchKernelGGL((lm_bwd_flat_saved<T>), dim3((unsigned)flat_blocks), dim3(256), 0, st, x, lab, up, grad, p,
                               chunks);
            return (unsigned)flat_blocks;
        }
    }
    const unsigned early_bit = (WantLoss && !WantGrad && p.early_kept && part.sum) ? kLmTookEarly : 0u;
    // the split shape exists for the one-direction kernels (forward, reduced forward, backward)
    constexpr bool kHasSplit = !(WantLoss && WantGrad);
    switch (pick_shape(p.C, p.m_size, V, sizeof(T), x, WantGrad ? grad : nullptr, lab, WantLoss ? loss : nullptr,
                       second_f32, kHasSplit, kHasSplit, kHasSplit, kImageFormMaxChannels<T>)) {
        case Shape::SplitDeep:
            if constexpr (kHasSplit) {
                constexpr int VD = V / 2;
                blocks = split_grid<VD>(p.P);
                switch (split_slots_deep(p.C)) {
#define PLH_CASE(KW)                                                                                                  \
    case KW:                                                                                                          \
        if constexpr (WantLoss)                                                                                       \
            hipLaunchKernelGGL((lm_fwd_split<T, KW, VD>), dim3(blocks), dim3(kSplitBlock), 0, st, x, lab, loss, \
                               part, p);                                                                              \
        else                                                                                                          \
            hipLaunchKernelGGL((lm_bwd_split<T, KW, VD>), dim3(blocks), dim3(kSplitBlock), 0, st, x, lab, up, grad, p); \
        break;
                    PLH_SPLIT_DEEP_CASES
#undef PLH_CASE
                }
            }
            break;
        case Shape::Split:
            if constexpr (kHasSplit) {
                blocks = split_grid<V>(p.P);
                switch (split_slots(p.C)) {
#define PLH_CASE(KW)                                                                                                  \
    case KW:                                                                                                          \
        if constexpr (WantLoss)                                                                                       \
            hipLaunchKernelGGL((lm_fwd_split<T, KW, V>), dim3(blocks), dim3(kSplitBlock), 0, st, x, lab, loss, \
                               part, p);                                                                              \
        else                                                                                                          \
            hipLaunchKernelGGL((lm_bwd_split<T, KW, V>), dim3(blocks), dim3(kSplitBlock), 0, st, x, lab, up, grad, p); \
        break;
                    PLH_SPLIT_SLOT_CASES
#undef PLH_CASE
                }
            }
            break;
        case Shape::SplitImage:                // tiles per image: channel planes that start on element boundaries only
            if constexpr (kHasSplit) {
                blocks = split_image_grid<V>(p.P / p.m_size, p.m_size);
                switch (split_slots(p.C)) {
#define PLH_CASE(KW)                                                                                                  \
    case KW:                                                                                                          \
        if constexpr (WantLoss)                                                                                       \
            hipLaunchKernelGGL((lm_fwd_split<T, KW, V, true>), dim3(blocks), dim3(kSplitBlock), 0, st, x, lab, \
                               loss, part, p);                                                                        \
        else                                                                                                          \
            hipLaunchKernelGGL((lm_bwd_split<T, KW, V, true>), dim3(blocks), dim3(kSplitBlock), 0, st, x, lab, up,    \
                               grad, p);                                                                              \
        break;
                    PLH_SPLIT_SLOT_CASES
#undef PLH_CASE
                }
            }
            break;
        // (the register-resident kernels are the ones that take LmParams::early_*: bit 31 of the result says so)
        case Shape::RegsVec:
            blocks = launch_regs<T, V, WantLoss, WantGrad>(x, lab, up, loss, grad, cnt, part, p, st) | early_bit;
            break;
        case Shape::RegsOne:
            if (image_form_pays<T>(p.C, p.m_size)) {
                blocks = launch_image<T, WantLoss, WantGrad>(x, lab, up, loss, grad, cnt, part, p, st) | early_bit;
                break;
            }
            blocks = launch_regs<T, 1, WantLoss, WantGrad>(x, lab, up, loss, grad, cnt, part, p, st) | early_bit;
            break;
        case Shape::Wave:
            // (16-bit rows of 2049 .. 4096 classes: the forward goes to the block-per-row kernel even where a wavefront
            // could hold the row in pieces of 8 - bf16 (65536,3000) forward 0.169 -> 0.145 ms - and leaves the row
            // statistics for the elementwise backward, 0.211 -> 0.144 ms)
            float *loss_w;
            loss_w = (WantLoss && !WantGrad && p.saved != nullptr && loss == nullptr &&
                      lm_saved_applies(sizeof(T), p.C, p.m_size)) ? p.saved : loss;
            if (p.C <= wrow_cap<T>(wrow_piece<T>(x, WantGrad ? grad : nullptr, p.C)) &&
                !(WantLoss && !WantGrad && sizeof(T) == 2 && p.C > kWaveRowCap)) {
#define PLH_GO(NI, W, G)                                                                                           \
    do {                                                                                                           \
        blocks = group_grid(p.P, WaveRowAt<G>::kRowsPerBlock);                                                     \
        if constexpr (WantGrad && wrow_cached_form<T>(W, G)) {                                                     \
            if (wrow_rows_end_inside_lines<T>(p.C)) {                                                              \
                hipLaunchKernelGGL((lm_wrow<T, NI, W, WantLoss, WantGrad, G, true>), dim3(blocks), \
                                   dim3(256), 0, st, x, lab, up, loss_w, grad, cnt, part, p);                        \
                break;                                                                                             \
            }                                                                                                      \
        }                                                                                                          \
        hipLaunchKernelGGL((lm_wrow<T, NI, W, WantLoss, WantGrad, G>), dim3(blocks), dim3(256), 0, \
                           st, x, lab, up, loss_w, grad, cnt, part, p);                                              \
    } while (0)
                PLH_WROW_DISPATCH_IF(wrow_piece<T>(x, WantGrad ? grad : nullptr, p.C), p.C, PLH_GO, (WantGrad ? 1 : 2));
#undef PLH_GO
                break;
            }
            blocks = (unsigned)(p.P < kMinPartialSlots ? p.P : kMinPartialSlots);
            {
                // (the forward that leaves the rows' statistics has no per-row losses to write: lmargin.hip)
                const bool keep = WantLoss && !WantGrad && p.saved != nullptr && loss == nullptr &&
                                  lm_saved_applies(sizeof(T), p.C, p.m_size);
                // short rows get small blocks (more rows in flight per CU, no idle lanes behind the barriers): forward
                // fp32 (65536,3000) 0.249 -> 0.181 ms with 64 threads, (65536,2049) 0.214 -> 0.127, bf16 (65536,3001) 0.251 ->
                // 0.145; the backward sweeps (65536,3000) 0.398 -> 0.349 with 128. Rows of 32000 fp32 classes and more keep 256.
                const int64_t row_bytes = (int64_t)p.C * (int64_t)sizeof(T);
                const int threads = WantGrad ? (row_bytes <= 12 * 1024 ? 128 : kRowBlockShort)
                                             : (row_bytes <= 32 * 1024 ? 64 : kRowBlockShort);
                hipLaunchKernelGGL((lm_row<T, WantLoss, WantGrad>), dim3(blocks), dim3(threads), 0,
                                   st, x, lab, up, keep ? p.saved : loss, grad, cnt, part, p,
                                   (row_chunks_ok<T>(x, WantGrad ? grad : nullptr, p.C) ? 1 : 0) | (keep ? 2 : 0));
            }
            break;
        case Shape::Lane:
            blocks = group_grid(p.P, 256);
            hipLaunchKernelGGL((lm_group<T, 1, WantLoss, WantGrad>), dim3(blocks), dim3(256), 0, st,
                               x, lab, up, loss, grad, cnt, part, p);
            break;
    }
    return blocks;
}

// Per-dtype entries into the kernels of this header. The entry points use three combinations of (loss, gradient):
// forward (plain or with partial sums), backward, and the fused pair (with the count of valid pixels); each is
// explicitly instantiated per element type in a translation unit of its own (lmargin_f32_fwd.hip, lmargin_f32_bwd.hip,
// lmargin_f32_both.hip, ...) so that the nine parts compile in parallel.
enum LmVariant { kLmForward = 0, kLmForwardReduced = 1, kLmBackward = 2, kLmForwardBackwardCount = 3, kLmForwardBackwardReduced = 4 };

#define PLH_LM_SIGNATURE(T, L, G)                                                                                    \
    unsigned launch_typed<T, L, G>(const T *, const int64_t *, const Upstream &, float *, T *, unsigned long long *, \
                                   Partials, const LmParams &, hipStream_t);
#define PLH_LM_EXTERN(T)                              \
    extern template PLH_LM_SIGNATURE(T, true, false)  \
    extern template PLH_LM_SIGNATURE(T, false, true)  \
    extern template PLH_LM_SIGNATURE(T, true, true)
#define PLH_LM_INSTANTIATE(T, L, G) template PLH_LM_SIGNATURE(T, L, G)

}  // namespace plh
