// Label-smoothed softmax cross entropy, forward and backward, for gfx950: kernels and launchers.
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
#pragma once
#include "plh_common.hpp"

namespace plh {

struct LsrParams {
    int64_t P;        // pixels = n_size * m_size
    int64_t m_size;
    int C;
    int64_t ignore;
    float w_pos, w_neg, sumw;
    unsigned xcd_run;   // tile permutation run length (xcd_run_for)
    // Per-pixel log-sum-exp of the logits, fp32 [P]. Forward, fp32 logits in NCHW: written when set, by the per-image
    // form of the register-resident kernel, the split kernels and the lane-per-pixel kernel (the shapes that
    // lsr_lse_applies sends here).
    // Backward: when set, lsr_bwd_planes forms the gradient from it plane by plane (see there).
    float *lse = nullptr;
};

// ---------------------------------------------------------------- regs ----

// loss = -sum_j w_j logp_j with logp_j = (x_j - mx) - lse:
//      = -( w_neg * (sum_j x_j - C*mx - C*lse) + (w_pos - w_neg) * (x_y - mx - lse) )
// so one pass over the slice gathers the plain sum, the exp-sum and the target's logit.
// exp(x - mx) is evaluated as exp2(fma(x, log2e, -c)) with c = fl(mx * log2e); what the rounding
// of c left out, r = mx*log2e - c (exact, one fma), scales every term by 2^r and is taken back
// out of log2(sum).
template <class T, int CP, int V, int Form>
__global__ __launch_bounds__(kRegsBlock) void lsr_fwd_regs(const T *__restrict__ x,
                                                          const int64_t *__restrict__ lab,
                                                          float *__restrict__ loss, Partials part,
                                                          const LsrParams p) {
    const bool Reduce = part.sum != nullptr;
    __shared__ float red[4];
    const PixelRef<V, Form> at(p.P, p.m_size, p.C, p.xcd_run);
    if (!Reduce && !at.live) return;

    // labels (and the upstream gradient) first: in the rows form the slice arrives through LDS behind a wait
    int64_t lb[V];
    at.labels(lab, p.ignore, lb);
    typename Pack<T, V>::Raw raw[CP];
    at.load_slice(x, p.C, p.m_size, raw);

    float out[V];
    float mine = 0.f;
    int cnt = 0;
    const float fc = (float)p.C;
    // the per-image form on fp32 logits also leaves each pixel's log-sum-exp where it is given a place (LsrParams::lse)
    constexpr bool kMayLse = Form == kPerImage && sizeof(T) == 4;
    float lse_abs[kMayLse ? V : 1];
#pragma unroll
    for (int k = 0; k < V; ++k) {
        bool ign;
        const int tgt = narrow_label(lb[k], p.ignore, p.C, ign);
        float xv[CP];
        const float mx = widen_and_max<T, V, CP>(raw, k, p.C, xv);
        const float c = mx * kLog2e;
        const float r = __builtin_fmaf(mx, kLog2e, -c);
        float s = 0.f, sx = 0.f, x_y = 0.f;
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (chan_ok<CP>(j, p.C)) {
                s += __builtin_amdgcn_exp2f(__builtin_fmaf(xv[j], kLog2e, -c));
                sx += xv[j];
                x_y = (tgt == j) ? xv[j] : x_y;
            }
        const float lse = (__builtin_amdgcn_logf(s) - r) * kLn2;
        if constexpr (kMayLse) lse_abs[k] = mx + lse;
        const float all = (sx - fc * mx) - fc * lse;
        // no target channel (label outside [0, C)): every weight is w_neg
        const float hot = (tgt >= 0) ? (p.w_pos - p.w_neg) * ((x_y - mx) - lse) : 0.f;
        const float acc = -(p.w_neg * all + hot);
        const bool valid = at.live && !ign;
        out[k] = valid ? acc : 0.f;
        mine += out[k];
        cnt += valid ? 1 : 0;
    }
    if (at.live && loss) at.store_f32(loss, out);
    if constexpr (kMayLse) {
        if (p.lse && at.live) at.store_f32(p.lse, lse_abs);     // past the caches: 0.1466 -> 0.1428 ms at (16,19,769,769)
    }
    if (Reduce) {
        const float bs = block_sum_256(mine, red);
        const float bc = block_sum_256((float)cnt, red);   // at most 1024 per block: exact in fp32
        if (threadIdx.x == 0) {
            part.sum[blockIdx.x] = bs;
            part.cnt[blockIdx.x] = (int)bc;
        }
    }
}

// WithLoss: the same kernel also leaves the block's sum of losses and its count of valid pixels in `part`, with the
// forward kernel's arithmetic (the module's 'mean' / 'sum' and its gradient from one pass over the logits).
template <class T, int CP, int V, int Form, bool WithLoss = false>
__global__ __launch_bounds__(kRegsBlock) void lsr_bwd_regs(const T *__restrict__ x,
                                                          const int64_t *__restrict__ lab,
                                                          const Upstream up, T *__restrict__ grad,
                                                          const LsrParams p, Partials part) {
    __shared__ float red[WithLoss ? 4 : 1];
    const PixelRef<V, Form> at(p.P, p.m_size, p.C, p.xcd_run);
    if (!WithLoss && !at.live) return;
    float mine = 0.f;
    int cnt = 0;

    // Labels and the upstream gradient are asked for before the slice: in the rows form the slice arrives through
    // LDS behind a wait, and the block-uniform forms gain as well (fp32 (8,19,1024,1024) backward 0.2305 -> 0.227 ms,
    // bf16 forward 0.0726 -> 0.0655 ms). The one-pixel-per-lane backwards on 16-bit elements keep the old order:
    // their rows form lost 4-9 % with the new one ((4 M, 32) bf16 0.111 -> 0.121 ms).
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

    // The gradient of a pixel replaces its logits in the slice as soon as they are no longer needed
    // (one pixel at a time for fp32, two for 16-bit elements, which share a dword): no second array.
    using PK = Pack<T, V>;
    unsigned keep[V];      // all ones for a pixel that counts, 0 for an ignored one
#pragma unroll
    for (int k0 = 0; k0 < V; k0 += PK::kStep) {
        float g[CP][PK::kStep];
#pragma unroll
        for (int kk = 0; kk < PK::kStep; ++kk) {
            const int k = k0 + kk;
            bool ign;
            const int tgt = narrow_label(lb[k], p.ignore, p.C, ign);
            keep[k] = ign ? 0u : 0xFFFFFFFFu;
            float xv[CP];
            const float mx = widen_and_max<T, V, CP>(raw, k, p.C, xv);
            const float c = mx * kLog2e;
            float s = 0.f, sx = 0.f, x_y = 0.f;
#pragma unroll
            for (int j = 0; j < CP; ++j)
                if (chan_ok<CP>(j, p.C)) {
                    if constexpr (WithLoss) {
                        sx += xv[j];
                        x_y = (tgt == j) ? xv[j] : x_y;
                    }
                    xv[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(xv[j], kLog2e, -c));
                    s += xv[j];
                }
            if constexpr (WithLoss) {           // as lsr_fwd_regs
                const float fc = (float)p.C;
                const float r = __builtin_fmaf(mx, kLog2e, -c);
                const float lse = (__builtin_amdgcn_logf(s) - r) * kLn2;
                const float all = (sx - fc * mx) - fc * lse;
                const float hot = (tgt >= 0) ? (p.w_pos - p.w_neg) * ((x_y - mx) - lse) : 0.f;
                const bool valid = at.live && !ign;
                mine += valid ? -(p.w_neg * all + hot) : 0.f;
                cnt += valid ? 1 : 0;
            }
            const float gk = go[k];
            const float scale = p.sumw * gk * __builtin_amdgcn_rcpf(s);     // one reciprocal per pixel
            float n_pos = -p.w_pos * gk, n_neg = -p.w_neg * gk;
            asm("" : "+v"(n_pos), "+v"(n_neg));                             // formed per pixel, not per channel
#pragma unroll
            for (int j = 0; j < CP; ++j)
                if (chan_ok<CP>(j, p.C)) g[j][kk] = __builtin_fmaf(xv[j], scale, (tgt == j) ? n_pos : n_neg);
        }
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (chan_ok<CP>(j, p.C)) PK::set(raw[j], k0 / PK::kStep, g[j]);
    }
    // ignored pixels get exact zeros whatever their logits were (the bitwise AND also clears NaN)
    const typename PK::Raw mask = PK::mask(keep);
#pragma unroll
    for (int j = 0; j < CP; ++j)
        if (chan_ok<CP>(j, p.C)) raw[j] = raw[j] & mask;
    if (!WithLoss || at.live) at.store_slice(grad, p.C, p.m_size, raw);
    if constexpr (WithLoss) {
        const float bs = block_sum_256(mine, red);
        const float bc = block_sum_256((float)cnt, red);   // at most 1024 per block: exact in fp32
        if (threadIdx.x == 0) {
            part.sum[blockIdx.x] = bs;
            part.cnt[blockIdx.x] = (int)bc;
        }
    }
}

// -------------------------------------------------------------- planes ----
// Backward from the forward's per-pixel log-sum-exp, for channel planes that start on element boundaries only (odd
// lengths: 513 x 513, 769 x 769 crops; any plane that does not start on a 128-byte line). With lse[p] at hand the
// gradient is elementwise,
//   g[c][p] = gk (sumw exp(x[c][p] - lse[p]) - w(label[p] == c)),
// so nothing ties the thread that writes an element to the other channels of its pixel, and every plane can be
// walked in its OWN cache lines: a block takes 1024 pixels of an image (2048 of 16-bit elements), and in plane c its
// 256 threads move the 32 whole lines that begin at the tile's first pixel shifted back by the plane's offset into
// its line - 16 aligned bytes per lane, loads and stores alike; lines are shared only where two planes meet. (The
// register-resident kernel has one pixel set for all channels, and with it runs that begin and end inside lines in
// every plane but one: 57 % of peak at (16,19,769,769) against 75 % here.) The pixels' (lse, label) pairs - the
// tile's and one line's worth before it - are staged in LDS once, transposed by pixel index mod the pixels of a
// lane, so that the reads of a lane's shifted window are conflict-free for every shift. One scalar upstream gradient
// (the module's 'mean' / 'sum'), optionally the byte mask of an OHEM selection; logits whose gradient tensor sits at
// the same offset into a 128-byte line.
// Per element type: a lane moves 16 bytes (4 fp32 or 8 16-bit elements), a line holds kLine elements, a block's tile
// is 256 lanes' worth of pixels and the stage holds one line's worth of pixels before it.
// (PlaneGeom and PlanePixel: plh_common.hpp, shared with the Taylor cross entropy's backward of the same form.)

__device__ __forceinline__ float plane_grad(float x, PlanePixel px, int c, float scale, float n_pos, float n_neg) {
    const float e = __builtin_amdgcn_exp2f((x - px.lse) * kLog2e);
    const float g = __builtin_fmaf(e, scale, (px.lab == c) ? n_pos : n_neg);
    return px.lab < 0 ? 0.f : g;
}

template <class T>
__global__ __launch_bounds__(256) void lsr_bwd_planes(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                      const Upstream up, T *__restrict__ grad, const LsrParams p,
                                                      int tiles, int planes_per_block) {
    static_assert(sizeof(T) == 4, "fp32 logits (see lsr_lse_applies)");
    using G = PlaneGeom<T>;
    constexpr int kPer = G::kPer, kTile = G::kTile, kHalo = G::kHalo;
    __shared__ PlanePixel pairs[kPer][(kTile + kHalo) / kPer];          // entry i at [i % kPer][i / kPer]
    const int64_t M = p.m_size;
    const int64_t n = blockIdx.x / tiles;
    const int t = (int)(blockIdx.x - n * tiles);
    const int l = threadIdx.x;
    const int64_t p_first = (int64_t)t * kTile - kHalo;                 // image-local pixel of staged entry 0
    for (int i = l; i < kTile + kHalo; i += 256) {
        const int64_t q = p_first + i;
        PlanePixel px{0.f, -1};
        if (q >= 0 && q < M) {
            const int64_t at = n * M + q;
            const int64_t lb = lab[at];
            const bool dropped = lb == p.ignore || (up.keep && up.keep[at] == 0);
            px.lse = p.lse[at];
            px.lab = dropped ? -1 : ((lb < 0 || lb >= p.C) ? p.C : (int)lb);
        }
        pairs[i % kPer][i / kPer] = px;
    }
    float gk = up.gout ? *up.gout * up.scale : up.scale;
    if (up.divide_by) gk = gk / (float)(*up.divide_by);
    const float scale = p.sumw * gk, n_pos = -p.w_pos * gk, n_neg = -p.w_neg * gk;
    __syncthreads();
    constexpr int U = 4;                            // planes in flight per thread
    // blockIdx.y: which planes of the tile (many channels are shared out over several blocks, so that the grid fills
    // the chip: (8,300,256,256) has 512 tiles)
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
                    out[d] = f32_bits(plane_grad(bits_f32(in[d]), pairs[i % kPer][i / kPer], c, scale, n_pos, n_neg));
                }
                __builtin_nontemporal_store(plh_u4{out[0], out[1], out[2], out[3]},
                                            reinterpret_cast<plh_u4 *>(grad + plane[u] + q[u]));
            } else {                    // the two ends of a plane, element by element
                for (int k = 0; k < kPer; ++k)
                    if (q[u] + k >= 0 && q[u] + k < M)
                        store_one(grad + plane[u] + q[u] + k,
                                  plane_grad(load_one(x + plane[u] + q[u] + k), pairs[(i0 + k) % kPer][(i0 + k) / kPer], c,
                                             scale, n_pos, n_neg));
            }
        }
    }
}

// Whether the forward leaves the log-sum-exp for these sizes and the backward runs plane by plane: fp32 logits on
// planes of 4096 pixels or more that do not start on 128-byte lines - up to 24 channels (the register-resident
// forward's per-image form) or 33 and more (channels shared among wavefronts in tiles per image: fwd+bwd at
// (8,150,513,513) 0.780 -> 0.670 ms) - and, whatever the planes' alignment, more than 256 channels, where the
// recomputing kernels keep a pixel's slice in two halves per wavefront ((8,300,256,256) 0.359 -> 0.334 ms,
// (4,512,256,256) 0.343 -> 0.301 ms) or have a lane walk its pixel's channels ((4,600,256,256) 0.761 -> 0.523 ms).
// On aligned planes with up to 256 channels the recomputing backward is as fast or faster (40 channels: 0.179 against
// 0.196 ms for the pair, 150: 0.629 / 0.634).
// fp32 logits only: with 16-bit logits (8 elements per lane, 64 per line) the pair measured no gain - bf16
// (16,19,769,769): forward 0.0815 -> 0.0963 ms with the extra output, backward 0.180 -> 0.160 ms, bound by its
// conversions.
// (N, C) rows of more than 32 classes, any element type: the forward leaves one value per row (lsr_fwd_wrow, lsr_fwd_row)
// and the backward from it (lsr_bwd_flat_lse) needs no reduction and no row in registers; which rows take it:
// row_backward_is_elementwise.
inline bool lsr_lse_applies(size_t elem_bytes, int64_t dimsize, int64_t m_size) {
    if (m_size == 1) {
        // (fp32 rows of 2049 .. 4096 classes stay with the backward that keeps the row in the block's registers:
        // (32768,4096) forward + backward 0.255 ms against 0.272)
        if (elem_bytes == 4 && dimsize > kWaveRowCap && dimsize <= 2 * kWaveRowCap) return false;
        return row_backward_is_elementwise(elem_bytes, dimsize, 1024);
    }
    if (elem_bytes != 4 || dimsize < 1 || m_size < 4096) return false;
    const bool off_lines = (m_size * (int64_t)elem_bytes) % 128 != 0;
    if (dimsize <= kMaxRegsChannels) return off_lines && image_form_pays<float>((int)dimsize, m_size);
    return off_lines || dimsize > kMaxSplitChannels;
}

// --------------------------------------------------------------- split ----
// 33..256 channels in NCHW: the 8 wavefronts of a block hold KW channels each (SplitSlice). Every
// wavefront reduces its part of a pixel's slice, the parts meet in LDS:
//   forward   (m_w, s_w, d_w, y_w) = max, sum_j exp(x_j - m_w), sum_j (x_j - m_w), target logit if it is here;
//             with M = max_w m_w:  S = sum_w s_w exp(m_w - M),  sum_j (x_j - M) = sum_w d_w + n_w (m_w - M),
//             and wavefront k forms the loss of pixel k of every lane as the regs kernel does;
//   backward  (c_w, s_w) in the base-2 domain, c_w = fl(m_w log2e), s_w = sum_j 2^(x_j log2e - c_w); every
//             wavefront then evaluates 2^(x_j log2e - max_w c_w) / sum_w s_w 2^(c_w - max c) for its channels.

template <class T, int KW, int V, bool PerImage = false>
__global__ __launch_bounds__(kSplitBlock) void lsr_fwd_split(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                            float *__restrict__ loss, Partials part,
                                                            const LsrParams p) {
    const bool Reduce = part.sum != nullptr;
    __shared__ float parts[4][kSplitWaves][kWave * V];
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
            float xv[KW];
            float mx = -INFINITY;
#pragma unroll
            for (int i = 0; i < KW; ++i) {
                xv[i] = (i < at.here) ? Pack<T, V>::get(raw[i], k) : -INFINITY;
                mx = fmaxf(mx, xv[i]);
            }
            const float c = mx * kLog2e;
            const float r = __builtin_fmaf(mx, kLog2e, -c);
            float s = 0.f, d = 0.f, x_y = 0.f;
#pragma unroll
            for (int i = 0; i < KW; ++i) {
                s += __builtin_amdgcn_exp2f(__builtin_fmaf(xv[i], kLog2e, -c));
                d += (i < at.here) ? xv[i] - mx : 0.f;
                x_y = (rel == i) ? xv[i] : x_y;
            }
            const int q = lane * V + k;
            parts[0][wave][q] = mx;
            parts[1][wave][q] = s * __builtin_amdgcn_exp2f(-r);      // 2^r is what the rounding of c left in every term
            parts[2][wave][q] = d;
            parts[3][wave][q] = x_y;
        }
    }
    __syncthreads();
    const int used = (p.C + KW - 1) / KW;               // wavefronts that hold channels
    const float fc = (float)p.C;
    if (wave >= V) return;                              // wavefront k finishes pixel k of every lane
    bool ign;
    PLH_SPLIT_MY_LABEL(my_lb, lb, wave, V)
    const int tgt = narrow_label(my_lb, p.ignore, p.C, ign);
    const int q = lane * V + wave;
    float M = parts[0][0][q];
    for (int w = 1; w < used; ++w) M = fmaxf(M, parts[0][w][q]);
    float S = 0.f, D = 0.f, x_y = 0.f;
    for (int w = 0; w < used; ++w) {
        const float shift = parts[0][w][q] - M;
        S = __builtin_fmaf(parts[1][w][q], fast_exp(shift), S);
        D += __builtin_fmaf((float)split_count(w, KW, p.C), shift, parts[2][w][q]);
        x_y += parts[3][w][q];
    }
    const float lse = fast_log(S);
    const float all = D - fc * lse;
    const float hot = (tgt >= 0) ? (p.w_pos - p.w_neg) * ((x_y - M) - lse) : 0.f;
    const float acc = -(p.w_neg * all + hot);
    const bool here = at.live && wave < at.nv;
    const bool valid = here && !ign;
    const float out = valid ? acc : 0.f;
    if (here && loss) loss[at.pix + wave] = out;
    if constexpr (sizeof(T) == 4) {
        if (here && p.lse) __builtin_nontemporal_store(M + lse, p.lse + at.pix + wave);      // LsrParams::lse
    }
    if (Reduce) split_block_partials<V>(out, valid, wave, lane, part);
}

template <class T, int KW, int V, bool PerImage = false>
__global__ __launch_bounds__(kSplitBlock) void lsr_bwd_split(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                            const Upstream up, T *__restrict__ grad,
                                                            const LsrParams p) {
    __shared__ float parts[2][kSplitWaves][kWave * V];
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
            float xv[KW];
            float mx = -INFINITY;
#pragma unroll
            for (int i = 0; i < KW; ++i) {
                xv[i] = (i < at.here) ? PK::get(raw[i], k) : -INFINITY;
                mx = fmaxf(mx, xv[i]);
            }
            const float c = mx * kLog2e;
            float s = 0.f;
#pragma unroll
            for (int i = 0; i < KW; ++i) s += __builtin_amdgcn_exp2f(__builtin_fmaf(xv[i], kLog2e, -c));
            parts[0][wave][lane * V + k] = c;
            parts[1][wave][lane * V + k] = s;
        }
    }
    __syncthreads();
    if (at.here == 0 || !at.live) return;
    const int used = (p.C + KW - 1) / KW;
    unsigned keep[V];      // all ones for a pixel that counts, 0 for an ignored one
#pragma unroll
    for (int k0 = 0; k0 < V; k0 += PK::kStep) {
        float g[KW][PK::kStep];
#pragma unroll
        for (int kk = 0; kk < PK::kStep; ++kk) {
            const int k = k0 + kk;
            bool ign;
            const int rel = narrow_label(lb[k], p.ignore, p.C, ign) - at.first;
            keep[k] = ign ? 0u : 0xFFFFFFFFu;
            const int q = lane * V + k;
            float cmax = parts[0][0][q];
            for (int w = 1; w < used; ++w) cmax = fmaxf(cmax, parts[0][w][q]);
            float S = 0.f;
            for (int w = 0; w < used; ++w)
                S = __builtin_fmaf(parts[1][w][q], __builtin_amdgcn_exp2f(parts[0][w][q] - cmax), S);
            const float gk = go[k];
            const float scale = p.sumw * gk * __builtin_amdgcn_rcpf(S);
            float n_pos = -p.w_pos * gk, n_neg = -p.w_neg * gk;
            asm("" : "+v"(n_pos), "+v"(n_neg));                             // formed per pixel, not per channel
#pragma unroll
            for (int i = 0; i < KW; ++i) {
                const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(PK::get(raw[i], k), kLog2e, -cmax));
                g[i][kk] = __builtin_fmaf(e, scale, (rel == i) ? n_pos : n_neg);
            }
        }
#pragma unroll
        for (int i = 0; i < KW; ++i) PK::set(raw[i], k0 / PK::kStep, g[i]);
    }
    // ignored pixels get exact zeros whatever their logits were (the bitwise AND also clears NaN)
    const typename PK::Raw mask = PK::mask(keep);
#pragma unroll
    for (int i = 0; i < KW; ++i) raw[i] = raw[i] & mask;
    at.store(grad, p.m_size, raw);
}

// -------------------------------------------------------------- stream ----
// Forward for more channels than the wavefronts of a block can hold in registers (beyond kMaxDeepChannels), fp32 logits
// in NCHW: a block of 8 wavefronts takes 256 consecutive pixels of an image, four per lane, and wavefront w walks the
// channels w, w + 8, w + 16, ... with four 16-byte loads in flight - whole kilobyte runs in every plane, where a lane per
// pixel reads 256 bytes per instruction ((4,600,256,256): 0.318 -> 0.113 ms). A wavefront keeps running statistics per
// pixel (maximum m, sum of exp(x - m), sum of x), rescaled once per batch of four channels; the eight sets meet in
// LDS, the first four wavefronts finish one pixel per lane (loss, log-sum-exp) and leave the block's partial sums.
constexpr int kStreamWaves = 8, kStreamPixels = 256;
struct StreamStats { float m, s, sx, xt; };

template <class T>
__global__ __launch_bounds__(kStreamWaves * 64) void lsr_fwd_stream(const T *__restrict__ x,
                                                                    const int64_t *__restrict__ lab,
                                                                    float *__restrict__ loss, Partials part,
                                                                    const LsrParams p, int tiles) {
    static_assert(sizeof(T) == 4, "fp32 logits");
    __shared__ StreamStats parts[kStreamWaves][kStreamPixels + 4];
    __shared__ float red[2][4];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int64_t n = blockIdx.x / tiles;
    const int64_t t0 = (int64_t)(blockIdx.x - n * tiles) * kStreamPixels;       // image-local first pixel of the tile
    const int64_t q = t0 + 4 * lane;                                            // this lane's four pixels
    const int have = (int)(p.m_size - q >= 4 ? 4 : (p.m_size - q > 0 ? p.m_size - q : 0));
    const int64_t at = n * p.m_size + (have ? q : 0);
    int tgt[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int64_t lb = k < have ? lab[at + k] : p.ignore;
        tgt[k] = (lb < 0 || lb >= p.C) ? -1 : (int)lb;
    }
    float m[4], sum[4], sx[4], xt[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        m[k] = -INFINITY;
        sum[k] = 0.f; sx[k] = 0.f; xt[k] = 0.f;
    }
    const T *xs = x + (n * p.C) * p.m_size + (have ? q : 0);
    constexpr int U = 4;
    for (int c0 = wave; c0 < p.C; c0 += kStreamWaves * U) {
        float v[U][4];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int c = c0 + kStreamWaves * u;
            const int cc = c < p.C ? c : c0;                   // a channel that exists; its values are not used
            const T *src = xs + (int64_t)cc * p.m_size;
            if (have == 4) {
                const plh_f4_a4 w = __builtin_nontemporal_load(reinterpret_cast<const plh_f4_a4 *>(src));
                v[u][0] = w.x; v[u][1] = w.y; v[u][2] = w.z; v[u][3] = w.w;
            } else {
#pragma unroll
                for (int k = 0; k < 4; ++k) v[u][k] = k < have ? src[k] : 0.f;
            }
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            float bm = m[k];
#pragma unroll
            for (int u = 0; u < U; ++u)
                if (c0 + kStreamWaves * u < p.C) bm = fmaxf(bm, v[u][k]);
            // exp(-inf - bm) = 0 on the first batch; while every channel so far is -inf (bm = -inf) the sum stays empty
            const bool empty = bm == -INFINITY;
            const float shift = bm * kLog2e;
            float acc = empty ? 0.f : sum[k] * __builtin_amdgcn_exp2f(__builtin_fmaf(m[k], kLog2e, -shift));
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int c = c0 + kStreamWaves * u;
                if (c < p.C) {
                    acc += empty ? 0.f : __builtin_amdgcn_exp2f(__builtin_fmaf(v[u][k], kLog2e, -shift));
                    sx[k] += v[u][k];
                    xt[k] = (tgt[k] == c) ? v[u][k] : xt[k];
                }
            }
            sum[k] = acc;
            m[k] = bm;
        }
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) parts[wave][4 * lane + k] = StreamStats{m[k], sum[k], sx[k], xt[k]};
    __syncthreads();
    if (wave >= 4) return;
    // thread i < 256 finishes pixel i of the tile
    const int i = threadIdx.x;
    const int64_t qi = t0 + i;
    const bool live = qi < p.m_size;
    float out = 0.f;
    bool valid = false;
    if (live) {
        const int64_t lb = lab[n * p.m_size + qi];
        const bool ign = lb == p.ignore;
        const int tg = (lb < 0 || lb >= p.C) ? -1 : (int)lb;
        float M = parts[0][i].m;
#pragma unroll
        for (int w = 1; w < kStreamWaves; ++w) M = fmaxf(M, parts[w][i].m);
        float S = 0.f, SX = 0.f;
#pragma unroll
        for (int w = 0; w < kStreamWaves; ++w) {
            const StreamStats st = parts[w][i];
            // a wavefront without channels (fewer than 8 channels never come here) or with -inf only: an empty sum
            S += st.s == 0.f ? 0.f : st.s * __builtin_amdgcn_exp2f((st.m - M) * kLog2e);
            SX += st.sx;
        }
        const float lse = __builtin_amdgcn_logf(S) * kLn2;
        const float fc = (float)p.C;
        const float all = (SX - fc * M) - fc * lse;
        const float x_y = tg >= 0 ? parts[tg & (kStreamWaves - 1)][i].xt : 0.f;
        const float hot = (tg >= 0) ? (p.w_pos - p.w_neg) * ((x_y - M) - lse) : 0.f;
        valid = !ign;
        out = valid ? -(p.w_neg * all + hot) : 0.f;
        if (loss) __builtin_nontemporal_store(out, loss + n * p.m_size + qi);
        if (p.lse) __builtin_nontemporal_store(M + lse, p.lse + n * p.m_size + qi);
    }
    if (part.sum) {
        // the four finishing wavefronts only: the others have left
        const float bs = group_reduce<64>(out, OpSum()), bc = group_reduce<64>(valid ? 1.f : 0.f, OpSum());
        if (lane == 0) {
            red[0][wave] = bs;
            red[1][wave] = bc;
        }
        __syncthreads();                                // the four wavefronts that are still here
        if (threadIdx.x == 0) {
            part.sum[blockIdx.x] = (red[0][0] + red[0][1]) + (red[0][2] + red[0][3]);
            part.cnt[blockIdx.x] = (int)((red[1][0] + red[1][1]) + (red[1][2] + red[1][3]));
        }
    }
}

// --------------------------------------------------------------- group ----
// G lanes per pixel, striding over its channels and re-reading global memory in each sweep (the
// preceding sweep has just pulled the slice into cache). Launched with G = 1: a lane per pixel.

template <class T, int G>
__global__ __launch_bounds__(256) void lsr_fwd_group(const T *__restrict__ x,
                                                     const int64_t *__restrict__ lab,
                                                     float *__restrict__ loss, Partials part,
                                                     const LsrParams p) {
    const bool Reduce = part.sum != nullptr;
    constexpr int kPix = 256 / G;
    __shared__ float red[4];
    const int sub = threadIdx.x % G;
    const int grp = threadIdx.x / G;

    float mine = 0.f, cnt = 0.f;
    // every lane of a group walks the same pixels, so the loop is group-uniform
    const int64_t rounds = ceil_div_dev(p.P, (int64_t)gridDim.x * kPix);
    for (int64_t r = 0; r < rounds; ++r) {
        const int64_t pix = (r * gridDim.x + blockIdx.x) * kPix + grp;
        const bool live = pix < p.P;
        const int64_t pc = live ? pix : 0;
        const int64_t n = pc / p.m_size;
        const T *xs = x + (pc + n * (int64_t)(p.C - 1) * p.m_size);
        const int64_t lb = lab[pc];

        float mx = -INFINITY;
#pragma unroll kGroupUnroll<G>
        for (int j = sub; j < p.C; j += G) {
            const float t = load_one(xs + (int64_t)j * p.m_size);
            mx = fmaxf(mx, t);
        }
        mx = group_reduce<G>(mx, OpMax());
        float s = 0.f;
#pragma unroll kGroupUnroll<G>
        for (int j = sub; j < p.C; j += G) {
            const float t = load_one(xs + (int64_t)j * p.m_size);
            s += fast_exp(t - mx);
        }
        s = group_reduce<G>(s, OpSum());
        const float lse = logf(s);
        float acc = 0.f;
#pragma unroll kGroupUnroll<G>
        for (int j = sub; j < p.C; j += G) {
            const float t = load_one(xs + (int64_t)j * p.m_size);
            acc -= ((t - mx) - lse) * ((lb == j) ? p.w_pos : p.w_neg);
        }
        acc = group_reduce<G>(acc, OpSum());
        const bool valid = live && (lb != p.ignore);
        if (live && sub == 0) {
            if (loss) loss[pix] = valid ? acc : 0.f;
            if constexpr (sizeof(T) == 4) {
                if (p.lse) p.lse[pix] = mx + lse;        // LsrParams::lse
            }
            mine += valid ? acc : 0.f;
            cnt += valid ? 1.f : 0.f;
        }
    }
    if (Reduce) {
        const float bs = block_sum_256(mine, red);
        const float bc = block_sum_256(cnt, red);     // exact while a block sees < 2^24 pixels
        if (threadIdx.x == 0) {
            part.sum[blockIdx.x] = bs;
            part.cnt[blockIdx.x] = (int)bc;
        }
    }
}

template <class T, int G>
__global__ __launch_bounds__(256) void lsr_bwd_group(const T *__restrict__ x,
                                                     const int64_t *__restrict__ lab,
                                                     const Upstream up, T *__restrict__ grad,
                                                     const LsrParams p) {
    constexpr int kPix = 256 / G;
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
        T *gs = grad + base;
        const int64_t lb = lab[pc];
        float go[1];
        load_upstream<1>(up, pc, go);

        float mx = -INFINITY;
#pragma unroll kGroupUnroll<G>
        for (int j = sub; j < p.C; j += G) {
            const float t = load_one(xs + (int64_t)j * p.m_size);
            mx = fmaxf(mx, t);
        }
        mx = group_reduce<G>(mx, OpMax());
        float s = 0.f;
#pragma unroll kGroupUnroll<G>
        for (int j = sub; j < p.C; j += G) {
            const float t = load_one(xs + (int64_t)j * p.m_size);
            const float e = fast_exp(t - mx);
            s += e;
        }
        s = group_reduce<G>(s, OpSum());
        if (live) {
            const float gk = (lb == p.ignore) ? 0.f : go[0];
            const float scale = p.sumw * gk / s;
#pragma unroll kGroupUnroll<G>
            for (int j = sub; j < p.C; j += G) {
                const float e = fast_exp(load_one(xs + (int64_t)j * p.m_size) - mx);
                store_one(gs + (int64_t)j * p.m_size, e * scale - ((lb == j) ? p.w_pos : p.w_neg) * gk);
            }
        }
    }
}

// ------------------------------------------------- wavefront per row, in registers ----
// (N, C) inputs with 33..2048 channels: a wavefront holds a whole row in registers (NI steps of 64 lanes,
// 16 bytes per lane and step where the rows allow it, else pieces of 8, 4 or 2 bytes), so the row is read once and
// every load of the row is in flight before the first one is used. Four rows per block at a time.

template <class T, int NI, int LP, int G>
__global__ __launch_bounds__(256) void lsr_fwd_wrow(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                    float *__restrict__ loss, Partials part, const LsrParams p) {
    const bool Reduce = part.sum != nullptr;
    __shared__ float red[4];
    constexpr int L = WaveRow<T, NI, LP, G>::L;
    const WaveRowAt<G> at;
    float mine = 0.f, cnt = 0.f;
    const float fc = (float)p.C;
    for (int64_t r0 = at.start; r0 < p.P; r0 += at.stride) {   // wave-uniform
        const bool live = r0 + at.grp < p.P;
        const int64_t row = live ? r0 + at.grp : p.P - 1;
        const T *xs = x + row * p.C;
        WaveRow<T, NI, LP, G> r;
        r.load(xs, p.C, at.sub);
        const float mx = r.max();
        float s = 0.f, d = 0.f;
#pragma unroll
        for (int i = 0; i < NI; ++i)
#pragma unroll
            for (int l = 0; l < L; ++l) {
                const float t = r.v[i][l] - mx;       // -inf beyond the row
                s += fast_exp(t);
                d += (t > -INFINITY) ? t : 0.f;
            }
        s = group_reduce<G>(s, OpSum());
        d = group_reduce<G>(d, OpSum());              // sum_j (x_j - mx)
        if (at.sub == 0 && live) {
            const int64_t lb = lab[row];
            const bool ign = (lb == p.ignore);
            const bool has_y = !ign && lb >= 0 && lb < p.C;
            const float x_y = has_y ? load_one(xs + lb) : 0.f;
            const float lse = fast_log(s);
            const float all = d - fc * lse;
            const float hot = has_y ? (p.w_pos - p.w_neg) * ((x_y - mx) - lse) : 0.f;
            const float acc = ign ? 0.f : -(p.w_neg * all + hot);
            if (loss) loss[row] = (loss == p.lse) ? mx + lse : acc;       // the slot takes the row's log-sum-exp (LsrParams::lse)
            mine += acc;
            cnt += ign ? 0.f : 1.f;
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

template <class T, int NI, int LP, int G, bool Cached = false>
__global__ __launch_bounds__(256) void lsr_bwd_wrow(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                    const Upstream up, T *__restrict__ grad, const LsrParams p) {
    constexpr int L = WaveRow<T, NI, LP, G>::L;
    using Span = WaveRowSpan<T, L, G, NI>;
    T *tile = Span::tile();
    const WaveRowAt<G> at;
    for (int64_t r0 = at.start; r0 < p.P; r0 += at.stride) {   // wave-uniform
        const bool live = r0 + at.grp < p.P;
        const int64_t row = live ? r0 + at.grp : p.P - 1;
        const T *xs = x + row * p.C;
        T *gs = grad + row * p.C;
        WaveRow<T, NI, LP, G> r;
        r.load(xs, p.C, at.sub);
        const int64_t lb = lab[row];
        float go[1];
        load_upstream<1>(up, row, go);
        const float mx = r.max();
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < NI; ++i)
#pragma unroll
            for (int l = 0; l < L; ++l) {
                r.v[i][l] = fast_exp(r.v[i][l] - mx);
                s += r.v[i][l];
            }
        s = group_reduce<G>(s, OpSum());
        const float gk = (lb == p.ignore) ? 0.f : go[0];
        const float scale = p.sumw * gk / s;
        const float n_pos = -p.w_pos * gk, n_neg = -p.w_neg * gk;
        const int tgt = (lb >= 0 && lb < p.C) ? (int)lb : -1;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int e0 = (at.sub + G * i) * L;
            if (e0 < p.C && live) {
                float g[L];
#pragma unroll
                for (int l = 0; l < L; ++l) g[l] = __builtin_fmaf(r.v[i][l], scale, (e0 + l == tgt) ? n_pos : n_neg);
                if constexpr (Span::kUse) Span::stage(tile, p.C, at.grp, e0, g);
                else RowPiece<T, L>::template store<Cached>(gs + e0, g);
            }
        }
        if constexpr (Span::kUse) {
            const int64_t left = p.P - r0;
            Span::flush(tile, grad + r0 * p.C, left < Span::kRows ? (int)left : Span::kRows, p.C);
        }
    }
}

// ----------------------------------------------------------------- row ----
// (N, C) inputs with rows longer than the staging buffer (a vocabulary): one block per row at a time,
// 16-byte loads, four of them in flight per lane, and a running (maximum, exponential sum) per lane
// that is rescaled when the maximum moves, so the forward reads the row once; the backward reads it a
// second time (from cache for all but the longest rows) to write the gradient.

template <class T>
__global__ __launch_bounds__(kRowBlock) void lsr_fwd_row(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                   float *__restrict__ loss, Partials part, const LsrParams p, int vec) {
    // vec: bit 0 - rows can be walked in 16-byte chunks; bit 1 - `loss` takes every row's log-sum-exp instead of its loss
    // (LsrParams::lse for rows: the reduced forward writes no per-row losses, so the one output slot serves; a second
    // conditional store per row, through the struct or an argument of its own, cost the kernel 40 %: (8192,32000) fp32
    // 0.167 -> 0.236 ms)
    const bool Reduce = part.sum != nullptr;
    __shared__ float red[kRowBlock / 64];
    float mine = 0.f;
    int cnt = 0;
    const float fc = (float)p.C;
    for (int64_t row = blockIdx.x; row < p.P; row += gridDim.x) {
        const T *xs = x + row * p.C;
        const RowStats st = row_combine(row_sweep<T>(xs, p.C, (vec & 1) != 0), red, true);
        if (threadIdx.x == 0) {
            const int64_t lb = lab[row];
            const bool ign = (lb == p.ignore);
            const bool has_y = !ign && lb >= 0 && lb < p.C;
            const float x_y = has_y ? load_one(xs + lb) : 0.f;
            const float lse = fast_log(st.s);
            const float all = (st.sx - fc * st.m) - fc * lse;
            const float hot = has_y ? (p.w_pos - p.w_neg) * ((x_y - st.m) - lse) : 0.f;
            const float acc = ign ? 0.f : -(p.w_neg * all + hot);
            if (loss) loss[row] = (vec & 2) ? st.m + lse : acc;
            mine += acc;
            cnt += ign ? 0 : 1;
        }
    }
    if (Reduce) {
        if (threadIdx.x == 0) {
            part.sum[blockIdx.x] = mine;
            part.cnt[blockIdx.x] = cnt;
        }
    }
}

// Backward of a long row from the forward's log-sum-exp: elementwise, g[j] = gk (sumw exp(x[j] - lse) - w(label == j)),
// so the row is read once and no reduction (two block-wide barriers per row) stands between the loads and the stores.
// One scalar upstream gradient, optionally the byte mask of an OHEM selection. Blocks take rows in turn; a thread has four
// 16-byte chunks in flight.
template <class T>
__global__ __launch_bounds__(kRowBlockShort) void lsr_bwd_row_lse(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                                  const Upstream up, T *__restrict__ grad, const LsrParams p,
                                                                  int vec) {
    constexpr int L = RowChunk<T>::kLen;
    float gk0 = up.gout ? *up.gout * up.scale : up.scale;
    if (up.divide_by) gk0 = gk0 / (float)(*up.divide_by);
    const int threads = row_threads();
    for (int64_t row = blockIdx.x; row < p.P; row += gridDim.x) {
        const T *xs = x + row * p.C;
        T *gs = grad + row * p.C;
        const RowSplit<T> sp(xs, p.C, vec != 0);
        const int64_t lb = lab[row];
        const bool dropped = lb == p.ignore || (up.keep && up.keep[row] == 0);
        const float gk = dropped ? 0.f : gk0;
        const float shift = -p.lse[row] * kLog2e;
        const float scale = p.sumw * gk, n_pos = -p.w_pos * gk, n_neg = -p.w_neg * gk;
        const int tgt = (lb >= 0 && lb < p.C) ? (int)lb : -1;
        auto one = [&](float xv, int j) {
            // ignored rows: exact zeros whatever the logits are (0 * inf would be NaN)
            const float g = __builtin_fmaf(__builtin_amdgcn_exp2f(__builtin_fmaf(xv, kLog2e, shift)), scale, (j == tgt) ? n_pos : n_neg);
            return dropped ? 0.f : g;
        };
        const T *body = xs + sp.head;
        T *gbody = gs + sp.head;
        // four chunks in flight per thread to the end of the row (the last trip's loads are masked, not serialised)
        for (int i = threadIdx.x; i < sp.chunks; i += 4 * threads) {
            float v[4][L];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int at = i + u * threads < sp.chunks ? i + u * threads : i;
                RowChunk<T>::load(body + (int64_t)at * L, v[u]);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int at = i + u * threads;
                if (at < sp.chunks) {
#pragma unroll
                    for (int e = 0; e < L; ++e) v[u][e] = one(v[u][e], sp.head + at * L + e);
                    RowChunk<T>::store(gbody + (int64_t)at * L, v[u]);
                }
            }
        }
        // the row's ends (and the whole row when it cannot be walked in chunks): element by element
        const int n_edge = sp.head + (p.C - sp.tail_from);
        for (int k = threadIdx.x; k < n_edge; k += threads) {
            const int j = k < sp.head ? k : sp.tail_from + (k - sp.head);
            store_one(gs + j, one(load_one(xs + j), j));
        }
    }
}

template <class T>
__global__ __launch_bounds__(kRowBlock) void lsr_bwd_row(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                   const Upstream up, T *__restrict__ grad, const LsrParams p, int vec) {
    __shared__ float red[kRowBlock / 64];
    constexpr int L = RowChunk<T>::kLen;
    for (int64_t row = blockIdx.x; row < p.P; row += gridDim.x) {
        const T *xs = x + row * p.C;
        T *gs = grad + row * p.C;
        const RowStats st = row_combine(row_sweep<T>(xs, p.C, vec != 0), red, false);
        const int64_t lb = lab[row];
        float go[1];
        load_upstream<1>(up, row, go);
        const float gk = (lb == p.ignore) ? 0.f : go[0];
        const float scale = p.sumw * gk / st.s;
        const float n_pos = -p.w_pos * gk, n_neg = -p.w_neg * gk;
        const int tgt = (lb >= 0 && lb < p.C) ? (int)lb : -1;
        const RowSplit<T> sp(xs, p.C, vec != 0);         // the gradient row sits at the same offset from its own boundary
        for (int i = threadIdx.x; i < sp.chunks; i += row_threads()) {
            float v[L];
            RowChunk<T>::load(xs + sp.head + (int64_t)i * L, v);
#pragma unroll
            for (int e = 0; e < L; ++e)
                v[e] = __builtin_fmaf(fast_exp(v[e] - st.m), scale, (sp.head + i * L + e == tgt) ? n_pos : n_neg);
            RowChunk<T>::store(gs + sp.head + (int64_t)i * L, v);
        }
        for (int j = threadIdx.x; j < sp.head; j += row_threads())
            store_one(gs + j, __builtin_fmaf(fast_exp(load_one(xs + j) - st.m), scale, (j == tgt) ? n_pos : n_neg));
        for (int j = sp.tail_from + threadIdx.x; j < p.C; j += row_threads())
            store_one(gs + j, __builtin_fmaf(fast_exp(load_one(xs + j) - st.m), scale, (j == tgt) ? n_pos : n_neg));
    }
}

// The same with the row kept in the block's registers between the two uses (NCH 16-byte chunks per
// thread, as loaded; widened where they are used): rows of up to 16 chunks per thread, i.e. 65536 fp32
// or 131072 16-bit elements with 1024 threads, are read from memory once, where the kernel above reads
// them twice (the second time through the caches, for as long as the rows in flight fit them). The few
// elements before the first and after the last 16-byte boundary of a row are re-read instead.
template <class T> __device__ __forceinline__ void chunk_widen(const plh_u4 &t, float (&v)[RowChunk<T>::kLen]) {
    if constexpr (sizeof(T) == 4) {
        v[0] = bits_f32(t.x); v[1] = bits_f32(t.y); v[2] = bits_f32(t.z); v[3] = bits_f32(t.w);
    } else {
        const unsigned d[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = widen_lo(d[i], T{});
            v[2 * i + 1] = widen_hi(d[i], T{});
        }
    }
}

// (16 chunks per thread are launched with 256 threads only: bounds of 1024 would cap the kernel at 128 registers, and it
// spilled 64 of its row's values to scratch memory under them)
template <class T, int NCH>
__global__ __launch_bounds__(NCH == 16 ? kRowBlockShort : kRowBlock) void lsr_bwd_rowregs(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                            const Upstream up, T *__restrict__ grad, const LsrParams p) {
    __shared__ float red[kRowBlock / 64];
    constexpr int L = RowChunk<T>::kLen;
    const int threads = row_threads();
    for (int64_t row = blockIdx.x; row < p.P; row += gridDim.x) {
        const T *xs = x + row * p.C;
        T *gs = grad + row * p.C;
        const RowSplit<T> sp(xs, p.C, true);
        plh_u4 raw[NCH];
#pragma unroll
        for (int u = 0; u < NCH; ++u) {
            const int i = threadIdx.x + u * threads;
            if (i < sp.chunks) raw[u] = __builtin_nontemporal_load(reinterpret_cast<const plh_u4 *>(xs + sp.head + (int64_t)i * L));
        }
        // the row's ends: at most L - 1 elements each, one per thread
        const int n_edge = sp.head + (p.C - sp.tail_from);
        const int edge_at = (int)threadIdx.x < sp.head ? (int)threadIdx.x : sp.tail_from + ((int)threadIdx.x - sp.head);
        const bool has_edge = (int)threadIdx.x < n_edge;
        const float edge = has_edge ? load_one(xs + edge_at) : -INFINITY;
        float mx = edge;
#pragma unroll
        for (int u = 0; u < NCH; ++u)
            if (threadIdx.x + u * threads < sp.chunks) {
                float v[L];
                chunk_widen<T>(raw[u], v);
#pragma unroll
                for (int e = 0; e < L; ++e) mx = fmaxf(mx, v[e]);
            }
        const float m = row_block_reduce(mx, red, OpMax());
        float s = fast_exp(edge - m);                                   // 0 for a thread without an edge element
#pragma unroll
        for (int u = 0; u < NCH; ++u)
            if (threadIdx.x + u * threads < sp.chunks) {
                float v[L];
                chunk_widen<T>(raw[u], v);
#pragma unroll
                for (int e = 0; e < L; ++e) s += fast_exp(v[e] - m);
            }
        const float total = row_block_reduce(s, red, OpSum());
        const int64_t lb = lab[row];
        float go[1];
        load_upstream<1>(up, row, go);
        const float gk = (lb == p.ignore) ? 0.f : go[0];
        const float scale = p.sumw * gk / total;
        const float n_pos = -p.w_pos * gk, n_neg = -p.w_neg * gk;
        const int tgt = (lb >= 0 && lb < p.C) ? (int)lb : -1;
#pragma unroll
        for (int u = 0; u < NCH; ++u) {
            const int i = threadIdx.x + u * threads;
            if (i < sp.chunks) {
                float v[L];
                chunk_widen<T>(raw[u], v);
#pragma unroll
                for (int e = 0; e < L; ++e)
                    v[e] = __builtin_fmaf(fast_exp(v[e] - m), scale, (sp.head + i * L + e == tgt) ? n_pos : n_neg);
                RowChunk<T>::store(gs + sp.head + (int64_t)i * L, v);
            }
        }
        if (has_edge) store_one(gs + edge_at, __builtin_fmaf(fast_exp(edge - m), scale, (edge_at == tgt) ? n_pos : n_neg));
    }
}

// The same over the flattened (rows x classes) tensor, for logits and gradient on 16-byte boundaries: a block takes 512
// consecutive 16-byte chunks (kFlatChunks = 2 per thread, coalesced: fp32 (8192,32000) 0.361 ms with four, 0.337 with
// two, 0.341 with one; bf16 alike with one to four) wherever rows begin and end, so the accesses are those of a copy; a chunk finds its row by one 32-bit division (the block's first element by a 64-bit one, block-uniform), and a
// chunk that straddles two rows goes element by element. Rows longer than a chunk (4097 classes at least).
template <class T>
__global__ __launch_bounds__(256) void lsr_bwd_flat_lse(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                        const Upstream up, T *__restrict__ grad, const LsrParams p,
                                                        int64_t chunks) {
    constexpr int L = RowChunk<T>::kLen, U = kFlatChunks;
    float gk0 = up.gout ? *up.gout * up.scale : up.scale;
    if (up.divide_by) gk0 = gk0 / (float)(*up.divide_by);
    const int64_t first = (int64_t)blockIdx.x * (256 * U);             // the block's first chunk
    const int64_t row0 = first * L / p.C;                               // block-uniform
    const unsigned col0 = (unsigned)(first * L - row0 * p.C);
    const unsigned C = (unsigned)p.C;
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
        auto row_terms = [&](int64_t r, float &shift, float &scale, float &n_pos, float &n_neg, int &tgt, bool &dropped) {
            const int64_t lb = lab[r];
            dropped = lb == p.ignore || (up.keep && up.keep[r] == 0);
            const float gk = dropped ? 0.f : gk0;
            shift = -p.lse[r] * kLog2e;
            scale = p.sumw * gk;
            n_pos = -p.w_pos * gk;
            n_neg = -p.w_neg * gk;
            tgt = (lb >= 0 && lb < p.C) ? (int)lb : -1;
        };
        float shift, scale, n_pos, n_neg;
        int tgt;
        bool dropped;
        row_terms(row, shift, scale, n_pos, n_neg, tgt, dropped);
        const int64_t ch = first + threadIdx.x + 256 * u;
        if (col + L <= C) {
#pragma unroll
            for (int e = 0; e < L; ++e) {
                const float g = __builtin_fmaf(__builtin_amdgcn_exp2f(__builtin_fmaf(v[u][e], kLog2e, shift)), scale,
                                               ((int)(col + e) == tgt) ? n_pos : n_neg);
                v[u][e] = dropped ? 0.f : g;            // ignored rows: exact zeros whatever the logits are
            }
        } else {                                        // the chunk crosses into the next row: both rows' terms, chosen per element
            float shift2, scale2, n_pos2, n_neg2;
            int tgt2;
            bool dropped2;
            row_terms(row + 1, shift2, scale2, n_pos2, n_neg2, tgt2, dropped2);
            tgt2 = tgt2 < 0 ? -1 : tgt2 + (int)C;       // in the first row's column numbers
#pragma unroll
            for (int e = 0; e < L; ++e) {
                const bool next = col + e >= C;
                const int t = next ? tgt2 : tgt;
                const float g = __builtin_fmaf(__builtin_amdgcn_exp2f(__builtin_fmaf(v[u][e], kLog2e, next ? shift2 : shift)),
                                               next ? scale2 : scale,
                                               ((int)(col + e) == t) ? (next ? n_pos2 : n_pos) : (next ? n_neg2 : n_neg));
                v[u][e] = (next ? dropped2 : dropped) ? 0.f : g;
            }
        }
        RowChunk<T>::store(grad + ch * L, v[u]);
    }
    // what is left after the last whole chunk: at most L - 1 elements of the last row
    if (blockIdx.x == gridDim.x - 1) {
        const int64_t done = chunks * L, total = p.P * p.C;
        const int64_t at = done + threadIdx.x;
        if (at < total) {
            const int64_t r = p.P - 1;
            const int64_t lb = lab[r];
            const bool dropped = lb == p.ignore || (up.keep && up.keep[r] == 0);
            const float gk = dropped ? 0.f : gk0;
            const int j = (int)(at - r * p.C);
            const float g = __builtin_fmaf(__builtin_amdgcn_exp2f((load_one(x + at) - p.lse[r]) * kLog2e), p.sumw * gk,
                                           (j == lb) ? -p.w_pos * gk : -p.w_neg * gk);
            store_one(grad + at, dropped ? 0.f : g);
        }
    }
}

// ------------------------------------------------------------ dispatch ----

inline LsrParams make_params(int64_t n_size, int64_t dimsize, int64_t m_size, int64_t ignore, float smooth,
                             size_t elem_bytes) {
    LsrParams p;
    p.P = n_size * m_size;
    p.m_size = m_size;
    p.C = (int)dimsize;
    p.ignore = ignore;
    p.w_pos = 1.f - smooth;                        // csrc/lsr_kernel.cu:83
    p.w_neg = smooth / (float)dimsize;             // csrc/lsr_kernel.cu:84
    p.sumw = p.w_neg * (float)(dimsize - 1) + p.w_pos;   // csrc/lsr_kernel.cu:125
    p.xcd_run = xcd_run_for(elem_bytes, m_size);
    return p;
}

template <class T, int V>
static unsigned launch_fwd_regs(const T *x, const int64_t *lab, float *loss, Partials part, const LsrParams &p,
                                hipStream_t st) {
    const unsigned grid = regs_grid<V>(p.P);
    const bool uni = tiles_are_uniform(p.m_size, V, sizeof(T));
    switch ((p.C + 3) / 4) {
#define PLH_CASE(K)                                                                                               \
    case K:                                                                                                       \
        if constexpr (V * sizeof(T) == 8) {                                                                       \
            if (uni) {                                                                                            \
                hipLaunchKernelGGL((lsr_fwd_regs<T, 4 * K, V, kUniform>), dim3(grid), dim3(kRegsBlock), 0,    \
                                   st, x, lab, loss, part, p);                                                    \
                break;                                                                                            \
            }                                                                                                     \
        }                                                                                                         \
        hipLaunchKernelGGL((lsr_fwd_regs<T, 4 * K, V, kGeneral>), dim3(grid), dim3(kRegsBlock), 0, st, x,    \
                           lab, loss, part, p);                                                                   \
        break;
        PLH_CASE(1) PLH_CASE(2) PLH_CASE(3) PLH_CASE(4) PLH_CASE(5) PLH_CASE(6) PLH_CASE(7) PLH_CASE(8)
#undef PLH_CASE
    }
    return grid;
}

template <class T, int V, bool WithLoss = false>
static unsigned launch_bwd_regs(const T *x, const int64_t *lab, const Upstream &up, T *grad, const LsrParams &p,
                                hipStream_t st, Partials part = Partials{nullptr, nullptr}) {
    const unsigned grid = regs_grid<V>(p.P);
    const bool uni = tiles_are_uniform(p.m_size, V, sizeof(T));
    switch ((p.C + 3) / 4) {
#define PLH_CASE(K)                                                                                              \
    case K:                                                                                                      \
        if constexpr (V * sizeof(T) == 8) {                                                                      \
            if (uni) {                                                                                           \
                hipLaunchKernelGGL((lsr_bwd_regs<T, 4 * K, V, kUniform, WithLoss>), dim3(grid), dim3(kRegsBlock), 0, \
                                   st, x, lab, up, grad, p, part);                                               \
                break;                                                                                           \
            }                                                                                                    \
        }                                                                                                        \
        hipLaunchKernelGGL((lsr_bwd_regs<T, 4 * K, V, kGeneral, WithLoss>), dim3(grid), dim3(kRegsBlock), 0, st, x, \
                           lab, up, grad, p, part);                                                              \
        break;
        PLH_CASE(1) PLH_CASE(2) PLH_CASE(3) PLH_CASE(4) PLH_CASE(5) PLH_CASE(6) PLH_CASE(7) PLH_CASE(8)
#undef PLH_CASE
    }
    return grid;
}

// `image`: tiles per image (channel planes that start on element boundaries only)
template <class T, int V>
static unsigned launch_fwd_split(const T *x, const int64_t *lab, float *loss, Partials part, const LsrParams &p,
                                 hipStream_t st, bool image = false) {
    if constexpr (V == ElemTraits<T>::kVec) if (image) {      // the deep form (V / 2) has no such variant
        if constexpr (sizeof(T) == 4) {
            if (split_image_wide(p.C)) {       // four fp32 pixels per lane
                const unsigned grid = split_image_grid<4>(p.P / p.m_size, p.m_size);
                switch (split_slots(p.C)) {
#define PLH_CASE(KW)                                                                                              \
    case KW:                                                                                                      \
        hipLaunchKernelGGL((lsr_fwd_split<T, KW, 4, true>), dim3(grid), dim3(kSplitBlock), 0, st, x, lab, \
                           loss, part, p);                                                                        \
        break;
                    PLH_CASE(16) PLH_CASE(20)
#undef PLH_CASE
                }
                return grid;
            }
        }
        const unsigned grid = split_image_grid<V>(p.P / p.m_size, p.m_size);
        switch (split_slots(p.C)) {
#define PLH_CASE(KW)                                                                                              \
    case KW:                                                                                                      \
        hipLaunchKernelGGL((lsr_fwd_split<T, KW, V, true>), dim3(grid), dim3(kSplitBlock), 0, st, x, lab, \
                           loss, part, p);                                                                        \
        break;
            PLH_SPLIT_SLOT_CASES
#undef PLH_CASE
        }
        return grid;
    }
    const unsigned grid = split_grid<V>(p.P);
    if constexpr (V < ElemTraits<T>::kVec) {        // the deep form
        switch (split_slots_deep(p.C)) {
#define PLH_CASE(KW)                                                                                              \
    case KW:                                                                                                      \
        hipLaunchKernelGGL((lsr_fwd_split<T, KW, V>), dim3(grid), dim3(kSplitBlock), 0, st, x, lab, loss, \
                           part, p);                                                                              \
        break;
            PLH_SPLIT_DEEP_CASES
#undef PLH_CASE
        }
        return grid;
    }
    switch (split_slots(p.C)) {
#define PLH_CASE(KW)                                                                                              \
    case KW:                                                                                                      \
        hipLaunchKernelGGL((lsr_fwd_split<T, KW, V>), dim3(grid), dim3(kSplitBlock), 0, st, x, lab, loss, \
                           part, p);                                                                              \
        break;
        PLH_SPLIT_SLOT_CASES
#undef PLH_CASE
    }
    return grid;
}

template <class T, int V>
static void launch_bwd_split(const T *x, const int64_t *lab, const Upstream &up, T *grad, const LsrParams &p,
                             hipStream_t st, bool image = false) {
    if constexpr (V == ElemTraits<T>::kVec) if (image) {      // the deep form (V / 2) has no such variant
        if constexpr (sizeof(T) == 4) {
            if (split_image_wide(p.C)) {       // four fp32 pixels per lane
                const unsigned grid = split_image_grid<4>(p.P / p.m_size, p.m_size);
                switch (split_slots(p.C)) {
#define PLH_CASE(KW)                                                                                              \
    case KW:                                                                                                      \
        hipLaunchKernelGGL((lsr_bwd_split<T, KW, 4, true>), dim3(grid), dim3(kSplitBlock), 0, st, x, lab, up, grad, \
                           p);                                                                                    \
        break;
                    PLH_CASE(16) PLH_CASE(20)
#undef PLH_CASE
                }
                return;
            }
        }
        const unsigned grid = split_image_grid<V>(p.P / p.m_size, p.m_size);
        switch (split_slots(p.C)) {
#define PLH_CASE(KW)                                                                                              \
    case KW:                                                                                                      \
        hipLaunchKernelGGL((lsr_bwd_split<T, KW, V, true>), dim3(grid), dim3(kSplitBlock), 0, st, x, lab, up, grad, \
                           p);                                                                                    \
        break;
            PLH_SPLIT_SLOT_CASES
#undef PLH_CASE
        }
        return;
    }
    const unsigned grid = split_grid<V>(p.P);
    if constexpr (V < ElemTraits<T>::kVec) {        // the deep form
        switch (split_slots_deep(p.C)) {
#define PLH_CASE(KW)                                                                                              \
    case KW:                                                                                                      \
        hipLaunchKernelGGL((lsr_bwd_split<T, KW, V>), dim3(grid), dim3(kSplitBlock), 0, st, x, lab, up, grad, p); \
        break;
            PLH_SPLIT_DEEP_CASES
#undef PLH_CASE
        }
        return;
    }
    switch (split_slots(p.C)) {
#define PLH_CASE(KW)                                                                                              \
    case KW:                                                                                                      \
        hipLaunchKernelGGL((lsr_bwd_split<T, KW, V>), dim3(grid), dim3(kSplitBlock), 0, st, x, lab, up, grad, p); \
        break;
        PLH_SPLIT_SLOT_CASES
#undef PLH_CASE
    }
}

// NCHW whose channel planes start on element boundaries only (odd lengths): the per-image form, four
// pixels per lane.
template <class T>
static unsigned launch_fwd_image(const T *x, const int64_t *lab, float *loss, Partials part, const LsrParams &p,
                                 hipStream_t st) {
    const unsigned grid = image_grid<4>(p.P / p.m_size, p.m_size);
    switch ((p.C + 3) / 4) {
#define PLH_CASE(K)                                                                                               \
    case K:                                                                                                       \
        if constexpr (4 * K <= kImageFormMaxChannels<T>)                                                          \
            hipLaunchKernelGGL((lsr_fwd_regs<T, 4 * K, 4, kPerImage>), dim3(grid), dim3(kRegsBlock), 0,   \
                               st, x, lab, loss, part, p);                                                        \
        break;
        PLH_CASE(1) PLH_CASE(2) PLH_CASE(3) PLH_CASE(4) PLH_CASE(5) PLH_CASE(6) PLH_CASE(7) PLH_CASE(8)
#undef PLH_CASE
    }
    return grid;
}

template <class T, bool WithLoss = false>
static unsigned launch_bwd_image(const T *x, const int64_t *lab, const Upstream &up, T *grad, const LsrParams &p,
                                 hipStream_t st, Partials part = Partials{nullptr, nullptr}) {
    const unsigned grid = image_grid<4>(p.P / p.m_size, p.m_size);
    switch ((p.C + 3) / 4) {
#define PLH_CASE(K)                                                                                              \
    case K:                                                                                                      \
        if constexpr (4 * K <= kImageFormMaxChannels<T>)                                                         \
            hipLaunchKernelGGL((lsr_bwd_regs<T, 4 * K, 4, kPerImage, WithLoss>), dim3(grid), dim3(kRegsBlock), 0, st, \
                               x, lab, up, grad, p, part);                                                       \
        break;
        PLH_CASE(1) PLH_CASE(2) PLH_CASE(3) PLH_CASE(4) PLH_CASE(5) PLH_CASE(6) PLH_CASE(7) PLH_CASE(8)
#undef PLH_CASE
    }
    return grid;
}

// Launches the forward; returns the number of blocks that wrote partials.
template <class T>
static unsigned forward_shape(const T *logits, const int64_t *labels, float *losses, Partials part, const LsrParams &p,
                        hipStream_t st) {
    constexpr int V = ElemTraits<T>::kVec;
    switch (pick_shape(p.C, p.m_size, V, sizeof(T), logits, nullptr, labels, losses, nullptr, true, true, true,
                       kImageFormMaxChannels<T>)) {
        case Shape::RegsVec: return launch_fwd_regs<T, V>(logits, labels, losses, part, p, st);
        case Shape::RegsOne:
            if (image_form_pays<T>(p.C, p.m_size)) return launch_fwd_image<T>(logits, labels, losses, part, p, st);
            return launch_fwd_regs<T, 1>(logits, labels, losses, part, p, st);
        case Shape::Split: return launch_fwd_split<T, V>(logits, labels, losses, part, p, st);
        case Shape::SplitImage: return launch_fwd_split<T, V>(logits, labels, losses, part, p, st, true);
        case Shape::SplitDeep: return launch_fwd_split<T, V / 2>(logits, labels, losses, part, p, st);
        case Shape::Wave: {
            const int piece = wrow_piece<T>(logits, nullptr, p.C);
            if (p.C > wrow_cap<T>(piece)) {
                const unsigned grid = (unsigned)(p.P < kMinPartialSlots ? p.P : kMinPartialSlots);
                // (the forward that keeps the log-sum-exp has no per-row losses to write: lsr.hip)
                const bool keep_lse = p.lse != nullptr && losses == nullptr;
                // rows of up to 12 KiB: one wavefront per row (fp32 (65536,3000) 0.158 -> 0.139 ms, (65536,2049) 0.143 ->
                // 0.100, bf16 (65536,3001) 0.148 -> 0.076)
                const int threads = (int64_t)p.C * (int64_t)sizeof(T) <= 12 * 1024 ? 64 : row_threads_for_sweep<T>(p.C);
                hipLaunchKernelGGL((lsr_fwd_row<T>), dim3(grid), dim3(threads), 0, st, logits, labels,
                                   keep_lse ? p.lse : losses, part, p,
                                   (row_chunks_ok<T>(logits, nullptr, p.C) ? 1 : 0) | (keep_lse ? 2 : 0));
                return grid;
            }
            unsigned grid = 0;
#define PLH_GO(NI, W, G)                                                                                            \
    do {                                                                                                            \
        grid = group_grid(p.P, WaveRowAt<G>::kRowsPerBlock);                                                        \
        hipLaunchKernelGGL((lsr_fwd_wrow<T, NI, W, G>), dim3(grid), dim3(256), 0, st, logits, labels, slot_w, \
                           part, p);                                                                                \
    } while (0)
            float *slot_w;
            slot_w = (p.lse != nullptr && losses == nullptr && lsr_lse_applies(sizeof(T), p.C, p.m_size)) ? p.lse : losses;
            PLH_WROW_DISPATCH(piece, p.C, PLH_GO);
#undef PLH_GO
            return grid;
        }
        case Shape::Lane: {
            if constexpr (sizeof(T) == 4) {
                // more channels than the split kernels hold, planes of some length: the wavefronts stream the channels
                const int64_t tiles = ceil_div(p.m_size, (int64_t)kStreamPixels);
                if (p.C > kMaxDeepChannels && p.m_size >= kStreamPixels && p.P / p.m_size * tiles < ((int64_t)1 << 31)) {
                    const unsigned grid = (unsigned)(p.P / p.m_size * tiles);
                    hipLaunchKernelGGL(lsr_fwd_stream<T>, dim3(grid), dim3(kStreamWaves * 64), 0, st, logits, labels, losses,
                                       part, p, (int)tiles);
                    return grid;
                }
            }
            const unsigned grid = group_grid(p.P, 256);
            hipLaunchKernelGGL((lsr_fwd_group<T, 1>), dim3(grid), dim3(256), 0, st, logits, labels, losses, part, p);
            return grid;
        }
    }
    return 0;
}

template <class T>
void lsr_backward_typed(const T *logits, const int64_t *labels, const Upstream &up, T *grad_logits,
                           const LsrParams &p, hipStream_t st) {
    constexpr int V = ElemTraits<T>::kVec;
    const float *go_vec = (up.gout && up.stride == 1) ? up.gout : nullptr;
    if (p.lse && p.m_size == 1 && !go_vec && lsr_lse_applies(sizeof(T), p.C, p.m_size)) {
        // long rows, from the forward's log-sum-exp: elementwise - over the flattened tensor when both tensors sit on
        // 16-byte boundaries, else row by row
        constexpr int L = RowChunk<T>::kLen;
        const int64_t chunks = p.P * p.C / L, blocks = ceil_div(chunks, (int64_t)(256 * kFlatChunks));
        if (!misaligned(logits, 16) && !misaligned(grad_logits, 16) && blocks >= 1 && blocks < ((int64_t)1 << 31)) {
            hipLaunchKernelGGL((lsr_bwd_flat_lse<T>), dim3((unsigned)blocks), dim3(256), 0, st, logits, labels, up,
                               grad_logits, p, chunks);
            return;
        }
        if (p.C > 2 * kWaveRowCap) {
            const unsigned grid = (unsigned)(p.P < kMinPartialSlots ? p.P : kMinPartialSlots);
            hipLaunchKernelGGL((lsr_bwd_row_lse<T>), dim3(grid), dim3(kRowBlockShort), 0, st, logits, labels, up, grad_logits, p, 0);
            return;
        }
        // (shorter rows off the 16-byte boundaries: the kernels below, which recompute)
    }
    if constexpr (sizeof(T) == 4) {
        // from the forward's log-sum-exp, plane by plane: one scalar upstream gradient, logits and gradient at the same
        // offset into a 128-byte line (whole lines of the one are whole lines of the other)
        const int64_t tiles = ceil_div(p.m_size + PlaneGeom<T>::kHalo - 1, (int64_t)PlaneGeom<T>::kTile);
        if (p.lse && !go_vec && lsr_lse_applies(sizeof(T), p.C, p.m_size) &&
            ((reinterpret_cast<uintptr_t>(logits) ^ reinterpret_cast<uintptr_t>(grad_logits)) & 127) == 0 &&
            !misaligned(logits, sizeof(T)) && p.P / p.m_size * tiles < ((int64_t)1 << 31)) {
            // planes per block (a multiple of the four in flight): all of them up to 32 channels; beyond, 16 on planes of
            // 1 MiB and more and 4 on smaller ones, where short blocks measured better (backward at (8,300,256,256)
            // 0.229 -> 0.213 ms, (8,300,384,384) 0.532 -> 0.491, (8,150,385,385) 0.251 -> 0.241; on 1 MiB planes
            // (8,150,512,512) 0.439 -> 0.488) - 8 when the tiles alone outnumber the blocks the chip holds at once
            // ((64,40,256,256) 4: 0.261, 8: 0.239 ms)
            const int64_t tiles_all = p.P / p.m_size * tiles;
            const int per = p.C <= kMaxRegsChannels                      ? p.C
                            : p.m_size * (int64_t)sizeof(T) >= (1 << 20) ? 16
                            : tiles_all <= 2048                          ? 4
                                                                         : 8;
            hipLaunchKernelGGL(lsr_bwd_planes<T>, dim3((unsigned)tiles_all, (unsigned)ceil_div(p.C, per)),
                               dim3(256), 0, st, logits, labels, up, grad_logits, p, (int)tiles, per);
            return;
        }
    }
    switch (pick_shape(p.C, p.m_size, V, sizeof(T), logits, grad_logits, labels, go_vec, nullptr, true, true, true,
                       kImageFormMaxChannels<T>)) {
        case Shape::RegsVec: launch_bwd_regs<T, V>(logits, labels, up, grad_logits, p, st); break;
        case Shape::RegsOne:
            if (image_form_pays<T>(p.C, p.m_size)) {
                launch_bwd_image<T>(logits, labels, up, grad_logits, p, st);
                break;
            }
            launch_bwd_regs<T, 1>(logits, labels, up, grad_logits, p, st);
            break;
        case Shape::Split: launch_bwd_split<T, V>(logits, labels, up, grad_logits, p, st); break;
        case Shape::SplitImage: launch_bwd_split<T, V>(logits, labels, up, grad_logits, p, st, true); break;
        case Shape::SplitDeep: launch_bwd_split<T, V / 2>(logits, labels, up, grad_logits, p, st); break;
        case Shape::Wave:
            if (p.C > wrow_cap<T>(wrow_piece<T>(logits, grad_logits, p.C))) {
                const unsigned grid = (unsigned)(p.P < kMinPartialSlots ? p.P : kMinPartialSlots);
                // chunks a row can have at most, and the threads that share them: 256 while 16 chunks per thread do
                const int chunks = p.C / RowChunk<T>::kLen + 1;
                const int threads = chunks <= kRowBlockShort * 16 ? kRowBlockShort : kRowBlock;
                const int per = (chunks + threads - 1) / threads;
                // 16 chunks per thread only in the 256-thread blocks: with 1024 threads they leave one block per
                // compute unit and lose to the two sweeps below (fp32 (4096, 50257) 0.641 against 0.365 ms,
                // (6144, 40000) 0.849 against 0.419; bf16 (2048, 128256) 0.276 against 0.246)
                if (row_chunks_ok<T>(logits, grad_logits, p.C) && per <= (threads == kRowBlockShort ? 16 : 8)) {
                    if (per <= 4)
                        hipLaunchKernelGGL((lsr_bwd_rowregs<T, 4>), dim3(grid), dim3(threads), 0, st, logits, labels, up,
                                           grad_logits, p);
                    else if (per <= 8)
                        hipLaunchKernelGGL((lsr_bwd_rowregs<T, 8>), dim3(grid), dim3(threads), 0, st, logits, labels, up,
                                           grad_logits, p);
                    else
                        hipLaunchKernelGGL((lsr_bwd_rowregs<T, 16>), dim3(grid), dim3(threads), 0, st, logits, labels, up,
                                           grad_logits, p);
                    break;
                }
                hipLaunchKernelGGL((lsr_bwd_row<T>), dim3(grid), dim3(row_threads_for(p.C)), 0, st, logits, labels, up, grad_logits, p,
                                   row_chunks_ok<T>(logits, grad_logits, p.C));
                break;
            }
            {
#define PLH_GO(NI, W, G)                                                                                           \
    do {                                                                                                           \
        if constexpr (wrow_cached_form<T>(W, G)) {                                                                 \
            if (wrow_rows_end_inside_lines<T>(p.C)) {                                                              \
                hipLaunchKernelGGL((lsr_bwd_wrow<T, NI, W, G, true>), dim3(group_grid(p.P, WaveRowAt<G>::kRowsPerBlock)), \
                                   dim3(256), 0, st, logits, labels, up, grad_logits, p);                          \
                break;                                                                                             \
            }                                                                                                      \
        }                                                                                                          \
        hipLaunchKernelGGL((lsr_bwd_wrow<T, NI, W, G>), dim3(group_grid(p.P, WaveRowAt<G>::kRowsPerBlock)), dim3(256), 0, \
                           st, logits, labels, up, grad_logits, p);                                                \
    } while (0)
                PLH_WROW_DISPATCH_IF(wrow_piece<T>(logits, grad_logits, p.C), p.C, PLH_GO, 1);
#undef PLH_GO
            }
            break;
        case Shape::Lane:
            hipLaunchKernelGGL((lsr_bwd_group<T, 1>), dim3(group_grid(p.P, 256)), dim3(256), 0, st, logits, labels, up,
                               grad_logits, p);
            break;
    }
}

// Loss partials and gradient from one pass, where the register-resident kernels run (up to kMaxRegsChannels channels in
// NCHW); returns the number of blocks that left partials, 0 for every other shape (nothing launched: the caller runs
// the forward and the backward one after the other).
template <class T>
unsigned lsr_fused_typed(const T *logits, const int64_t *labels, const Upstream &up, T *grad_logits, Partials part,
                         const LsrParams &p, hipStream_t st) {
    constexpr int V = ElemTraits<T>::kVec;
    switch (pick_shape(p.C, p.m_size, V, sizeof(T), logits, grad_logits, labels, nullptr, nullptr, true, true, true,
                       kImageFormMaxChannels<T>)) {
        case Shape::RegsVec: return launch_bwd_regs<T, V, true>(logits, labels, up, grad_logits, p, st, part);
        case Shape::RegsOne:
            if (image_form_pays<T>(p.C, p.m_size)) return launch_bwd_image<T, true>(logits, labels, up, grad_logits, p, st, part);
            return launch_bwd_regs<T, 1, true>(logits, labels, up, grad_logits, p, st, part);
        default: return 0;
    }
}

// Per-dtype entries into the kernels of this header; explicitly instantiated per element type and direction
// (lsr_f32_fwd.hip, lsr_f32_bwd.hip, lsr_f32_both.hip, ...) so that the nine parts compile in parallel.
template <class T>
unsigned lsr_forward_typed(const T *logits, const int64_t *labels, float *losses, Partials part, bool reduce,
                           const LsrParams &p, hipStream_t st) {
    if (!reduce) part = Partials{nullptr, nullptr};      // the kernels leave partial sums where they are given a place
    return forward_shape<T>(logits, labels, losses, part, p, st);
}

#define PLH_LSR_FWD_SIGNATURE(T)                                                                                    \
    unsigned lsr_forward_typed<T>(const T *, const int64_t *, float *, Partials, bool, const LsrParams &, hipStream_t);
#define PLH_LSR_BWD_SIGNATURE(T)                                                                                    \
    void lsr_backward_typed<T>(const T *, const int64_t *, const Upstream &, T *, const LsrParams &, hipStream_t);

#define PLH_LSR_BOTH_SIGNATURE(T)                                                                                   \
    unsigned lsr_fused_typed<T>(const T *, const int64_t *, const Upstream &, T *, Partials, const LsrParams &, hipStream_t);
#define PLH_LSR_EXTERN(T)                  \
    extern template PLH_LSR_FWD_SIGNATURE(T) \
    extern template PLH_LSR_BWD_SIGNATURE(T) \
    extern template PLH_LSR_BOTH_SIGNATURE(T)

// one translation unit per element type and direction (lsr_<type>_fwd.hip, lsr_<type>_bwd.hip)
#define PLH_LSR_INSTANTIATE_FWD(T) template PLH_LSR_FWD_SIGNATURE(T)
#define PLH_LSR_INSTANTIATE_BWD(T) template PLH_LSR_BWD_SIGNATURE(T)
#define PLH_LSR_INSTANTIATE_BOTH(T) template PLH_LSR_BOTH_SIGNATURE(T)

}  // namespace plh
