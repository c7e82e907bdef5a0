// Layer norm over the channel dimension of (N, C, M) tensors on gfx950 (csrc/layer_norm.cu:53-257).
//   forward   out = (x - mean) * rsqrt(var + eps),  mean / var (population) over C per (n, m)   (:102-129)
//   backward  res = -rsqrt(v) * (1/C + (x - mean) * (x - 1/C) * mean * v) * grad,  v = var + eps  (:200-216)
// The backward is the reference's expression, kept as it is (it is not the derivative of the forward).
//
// The op has to see a slice twice (statistics, then the normalised values), and a slice of C
// channels times a wavefront's pixels is far more than caches keep per wave, so the slice stays in
// REGISTERS between the two uses: lanes run along pixels (8 bytes per lane and channel), and for
// C > 32 the four (C > 64: eight) waves of a block split the channels of one pixel group between
// them and exchange per-wave (mean, centred square sum) pairs through LDS, merged by the
// pairwise-variance rule. A wave holds at most 96 packed channels, which covers C <= 768; C <= 1024
// runs one pixel per lane; anything larger, and m_size == 1 (rows contiguous), takes a two-sweep
// kernel whose second sweep is served by cache.
#pragma once
#include <type_traits>
#include "plh_common.hpp"

namespace plh {

struct LnParams {
    int64_t P;          // n_size * m_size
    int64_t m_size;
    int C;
    int per_wave;       // channels per wave when the waves of a block share a pixel group
    float eps;
};

constexpr int kLnBlock = 256;

// KW = channel slots per wave (>= the channels it holds), V = pixels per lane, WS = waves sharing a
// pixel group (1: each of a block's four waves has its own group and all channels; 4 or 8: the block
// is WS waves with 1/WS of the channels each).
// PerImage: pixel groups that never straddle two images (groups = images x groups per image), for channel planes
// that start on element boundaries only (odd lengths): a lane's V pixels are moved with accesses of the same
// width from element boundaries; the last lane of an image may hold fewer and goes pixel by pixel.
template <class T, int KW, int V, int WS, bool Bwd, bool PerImage = false>
__global__ __launch_bounds__(WS > 4 ? 64 * WS : kLnBlock) void ln_regs(const T *__restrict__ x, const T *__restrict__ g,
                                                    T *__restrict__ out, const LnParams p) {
    using PK = Pack<T, V>;
    __shared__ float ex[WS][2][V][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t group = WS > 1 ? (int64_t)blockIdx.x : (int64_t)blockIdx.x * 4 + wave;
    bool live;
    int nv = V;                                        // pixels this lane has
    int64_t pc, n;
    if constexpr (PerImage) {
        const int64_t per_image = ceil_div_dev(p.m_size, (int64_t)64 * V);
        n = group / per_image;
        const int64_t local = ((group - n * per_image) * 64 + lane) * V;
        const int64_t left = p.m_size - local;
        nv = left >= V ? V : (left > 0 ? (int)left : 0);
        live = nv > 0 && n * p.m_size < p.P;
        if (!live) { n = 0; nv = V; }                  // dead lanes read pixel 0 and store nothing
        pc = live ? n * p.m_size + local : 0;
    } else {
        const int64_t pix = (group * 64 + lane) * V;
        live = pix < p.P;
        pc = live ? pix : 0;                           // dead lanes read pixel 0 and store nothing
        n = pc / p.m_size;
    }
    const int c0 = WS > 1 ? wave * p.per_wave : 0;
    int cnt = WS > 1 ? p.C - c0 : p.C;
    cnt = cnt < 1 ? 1 : (WS > 1 && cnt > p.per_wave ? p.per_wave : cnt);   // a split always leaves every wave >= 1 channel
    cnt = __builtin_amdgcn_readfirstlane(cnt);
    const int64_t base = pc + n * (int64_t)(p.C - 1) * p.m_size + (int64_t)c0 * p.m_size;
    auto fetch = [&](const T *at) {
        if constexpr (PerImage) {
            if (nv < V) {
                float one[V];
#pragma unroll
                for (int k = 0; k < V; ++k) one[k] = k < nv ? load_one(at + k) : 0.f;
                return PK::put(one);
            }
            return PK::load_unaligned(at);
        } else {
            return PK::load(at);
        }
    };
    auto put_back = [&](T *at, const float (&r)[V]) {
        if constexpr (PerImage) {
            if (nv < V) {
#pragma unroll
                for (int k = 0; k < V; ++k)
                    if (k < nv) store_one(at + k, r[k]);
                return;
            }
            PK::store_unaligned(at, PK::put(r));
        } else {
            PK::store(at, PK::put(r));
        }
    };

    // Slots past the wave's last channel re-read that channel (same address, served by cache) and are
    // weighted out of the sums: straight-line code, no per-slot control flow.
    typename PK::Raw raw[KW];
#pragma unroll
    for (int j = 0; j < KW; ++j) raw[j] = fetch(x + base + (int64_t)(j < cnt ? j : cnt - 1) * p.m_size);

    const float inv_c = 1.f / (float)p.C;
    float mean[V], v[V];
#pragma unroll
    for (int k = 0; k < V; ++k) {
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < KW; ++j) s += j < cnt ? PK::get(raw[j], k) : 0.f;
        const float mw = s / (float)cnt;
        // every sweep widens the packed slice again: kept apart for the optimiser, which would
        // otherwise hold all widened values of the first sweep in registers for the later ones
#pragma unroll
        for (int j = 0; j < KW; ++j) forget_origin(raw[j]);
        float q = 0.f;
#pragma unroll
        for (int j = 0; j < KW; ++j) {
            const float d = j < cnt ? PK::get(raw[j], k) - mw : 0.f;
            q = __builtin_fmaf(d, d, q);
        }
        if constexpr (WS > 1) {
            ex[wave][0][k][lane] = mw;
            ex[wave][1][k][lane] = q;
        } else {
            mean[k] = mw;
            v[k] = q * inv_c + p.eps;
        }
    }
    if constexpr (WS > 1) {
        __syncthreads();
#pragma unroll
        for (int k = 0; k < V; ++k) {
            float mw[WS], cw[WS], tot = 0.f;
#pragma unroll
            for (int w = 0; w < WS; ++w) {
                int c = p.C - w * p.per_wave;
                c = c < 0 ? 0 : (c > p.per_wave ? p.per_wave : c);
                cw[w] = (float)c;
                mw[w] = ex[w][0][k][lane];
                tot = __builtin_fmaf(cw[w], mw[w], tot);
            }
            const float m = tot * inv_c;
            float m2 = 0.f;
#pragma unroll
            for (int w = 0; w < WS; ++w) {
                const float d = mw[w] - m;
                m2 += ex[w][1][k][lane] + cw[w] * d * d;
            }
            mean[k] = m;
            v[k] = m2 * inv_c + p.eps;
        }
    }
    float rstd[V], mv[V];
#pragma unroll
    for (int k = 0; k < V; ++k) {
        rstd[k] = 1.f / sqrtf(v[k]);
        mv[k] = mean[k] * v[k];
    }
#pragma unroll
    for (int j = 0; j < KW; ++j) forget_origin(raw[j]);

    if constexpr (!Bwd) {
#pragma unroll
        for (int j = 0; j < KW; ++j) {
            float r[V];
#pragma unroll
            for (int k = 0; k < V; ++k) r[k] = (PK::get(raw[j], k) - mean[k]) * rstd[k];
            if (live && j < cnt) put_back(out + base + (int64_t)j * p.m_size, r);
        }
    } else {
        constexpr int kChunk = KW < 8 ? KW : 8;        // gradient slices in flight per trip
#pragma unroll
        for (int j0 = 0; j0 < KW; j0 += kChunk) {
            typename PK::Raw graw[kChunk];
#pragma unroll
            for (int jj = 0; jj < kChunk; ++jj)
                graw[jj] = fetch(g + base + (int64_t)(j0 + jj < cnt ? j0 + jj : cnt - 1) * p.m_size);
#pragma unroll
            for (int jj = 0; jj < kChunk; ++jj) {
                float r[V];
#pragma unroll
                for (int k = 0; k < V; ++k) {
                    const float val = PK::get(raw[j0 + jj], k);
                    const float inner = __builtin_fmaf((val - mean[k]) * (val - inv_c), mv[k], inv_c);
                    r[k] = -rstd[k] * inner * PK::get(graw[jj], k);
                }
                if (live && j0 + jj < cnt) put_back(out + base + (int64_t)(j0 + jj) * p.m_size, r);
            }
        }
    }
}

// Any C: G lanes share one slice and stride over it (G = 64: a wavefront per contiguous row;
// G = 1: a lane per slice). Statistics from sums shifted by the mean of the slice's first elements, which keeps
// the one-pass variance well conditioned; the second sweep re-reads the slice through cache.
template <class T, int G, bool Bwd>
__global__ __launch_bounds__(256) void ln_group(const T *__restrict__ x, const T *__restrict__ g, T *__restrict__ out,
                                                const LnParams p) {
    constexpr int kPix = 256 / G;
    const int sub = threadIdx.x % G, grp = threadIdx.x / G;
    const float inv_c = 1.f / (float)p.C;
    const int64_t rounds = ceil_div_dev(p.P, (int64_t)gridDim.x * kPix);
    for (int64_t rd = 0; rd < rounds; ++rd) {
        const int64_t pix = (rd * gridDim.x + blockIdx.x) * kPix + grp;
        const bool live = pix < p.P;
        const int64_t pc = live ? pix : 0;
        const int64_t n = pc / p.m_size;
        const int64_t base = pc + n * (int64_t)(p.C - 1) * p.m_size;
        // The shift is the mean of the slice's first (up to) 8 elements: a single element can sit several standard
        // deviations from the mean, and E[d^2] - E[d]^2 then cancels digits (shifted by its first element, a slice
        // of 1317 channels missed 1e-5 by a factor of 4). Four independent partial sums per lane keep the rounding
        // of the long sums down and eight loads in flight.
        const int n_shift = p.C < 8 ? p.C : 8;
        float shift = 0.f;
        for (int j = 0; j < n_shift; ++j) shift += load_one(x + base + (int64_t)j * p.m_size);
        shift *= 1.f / (float)n_shift;
        float a1[4] = {0.f, 0.f, 0.f, 0.f}, a2[4] = {0.f, 0.f, 0.f, 0.f};
        int j = sub;
#pragma unroll 2
        for (; j + 3 * G < p.C; j += 4 * G) {
            float d[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) d[u] = load_one(x + base + (int64_t)(j + u * G) * p.m_size) - shift;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                a1[u] += d[u];
                a2[u] = __builtin_fmaf(d[u], d[u], a2[u]);
            }
        }
        for (; j < p.C; j += G) {
            const float d = load_one(x + base + (int64_t)j * p.m_size) - shift;
            a1[0] += d;
            a2[0] = __builtin_fmaf(d, d, a2[0]);
        }
        float s1 = (a1[0] + a1[1]) + (a1[2] + a1[3]), s2 = (a2[0] + a2[1]) + (a2[2] + a2[3]);
        s1 = group_reduce<G>(s1, OpSum());
        s2 = group_reduce<G>(s2, OpSum());
        const float dm = s1 * inv_c;
        const float mean = shift + dm;
        const float var = fmaxf(s2 * inv_c - dm * dm, 0.f);
        const float v = var + p.eps;
        const float rstd = 1.f / sqrtf(v), mv = mean * v;
        if (!live) continue;
#pragma unroll 8
        for (int j = sub; j < p.C; j += G) {
            const int64_t at = base + (int64_t)j * p.m_size;
            const float val = load_one(x + at);
            if constexpr (Bwd) {
                const float inner = __builtin_fmaf((val - mean) * (val - inv_c), mv, inv_c);
                store_one(out + at, -rstd * inner * load_one(g + at));
            } else {
                store_one(out + at, (val - mean) * rstd);
            }
        }
    }
}

template <class T, bool Bwd>
void ln_launch(const T *x, const T *g, T *out, int64_t n_size, int64_t dimsize, int64_t m_size, float eps,
               hipStream_t st) {
    constexpr int VT = ElemTraits<T>::kVec;
    LnParams p;
    p.P = n_size * m_size;
    p.m_size = m_size;
    p.C = (int)dimsize;
    p.eps = eps;
    // Channels per wave: all of them up to 32, a quarter up to 64, an eighth beyond (smaller register
    // chunks in more waves measured better: they overlap one wave's loads with another's stores).
    // With 4 waves and C > 32, or 8 waves and C > 64, every wave holds at least one channel.
    const int ws = dimsize > 64 ? 8 : (dimsize > 32 ? 4 : 1);
    p.per_wave = (int)ceil_div(dimsize, ws);
    if (m_size == 1 || dimsize > 1024) {
        if (m_size == 1) {
            hipLaunchKernelGGL((ln_group<T, 64, Bwd>), dim3(group_grid(p.P, 4)), dim3(256), 0, st, x, g, out, p);
        } else {
            hipLaunchKernelGGL((ln_group<T, 1, Bwd>), dim3(group_grid(p.P, 256)), dim3(256), 0, st, x, g, out, p);
        }
        return;
    }
    const bool vec = dimsize <= 768 && m_size % VT == 0 && !misaligned(x, VT * sizeof(T)) &&
                     !misaligned(out, VT * sizeof(T)) && !(Bwd && misaligned(g, VT * sizeof(T)));
    // planes that start on element boundaries only (odd lengths, misaligned tensors) and are long enough that
    // the partly filled last group of every image is a small share: the same pixels per lane in groups per image
    const bool image = !vec && dimsize <= 768 && m_size >= 4096;
    const int slots = p.per_wave;
    // 16-bit elements, more than 48 slots per wave: 64 and 96 slots of four pixels are 256 and 384 values per lane, and
    // where the kernel spills them (up to 1168 bytes per lane: the per-image form, and fp16 with 96 slots) two pixels per
    // lane are faster: fp16 (32,768,4098) forward 0.565 -> 0.174 ms, backward 0.739 -> 0.271; (32,768,4096) 0.109 -> 0.092
    // and 0.180 -> 0.172. (bf16 on aligned planes keeps four: 0.129 against 0.192 ms backward at (32,768,4096).)
    constexpr int VN = (sizeof(T) == 2) ? 2 : VT;
    const bool narrow = sizeof(T) == 2 && ws == 8 && slots > 48 && slots <= 96 &&
                        (image || (vec && std::is_same<T, f16>::value && slots > 64));
    const int vv = narrow ? VN : VT;
    const int64_t groups = image ? n_size * ceil_div(m_size, 64 * vv) : ceil_div(p.P, 64 * (vec ? vv : 1));
    const unsigned grid = (unsigned)(ws > 1 ? groups : ceil_div(groups, 4));
#define PLH_LN(KW, VV, WS) \
    hipLaunchKernelGGL((ln_regs<T, KW, VV, WS, Bwd>), dim3(grid), dim3(WS > 4 ? 64 * WS : kLnBlock), 0, st, x, g, out, p)
#define PLH_LN_IMAGE(KW, WS) \
    hipLaunchKernelGGL((ln_regs<T, KW, VT, WS, Bwd, true>), dim3(grid), dim3(WS > 4 ? 64 * WS : kLnBlock), 0, st, x, g, out, p)
#define PLH_LN_V(KW, WS) do { if (vec) PLH_LN(KW, VT, WS); else if (image) PLH_LN_IMAGE(KW, WS); else PLH_LN(KW, 1, WS); } while (0)
#define PLH_LN_NARROW(KW, WS)                                                                                              \
    do {                                                                                                                   \
        if (vec) PLH_LN(KW, VN, WS);                                                                                       \
        else if (image)                                                                                                    \
            hipLaunchKernelGGL((ln_regs<T, KW, VN, WS, Bwd, true>), dim3(grid), dim3(64 * WS), 0, st, x, g, out, p);       \
        else PLH_LN(KW, 1, WS);                                                                                            \
    } while (0)
    // Slot counts in steps of about 1.5x: a wave whose channels fall short of its slots re-reads its last
    // channel for the rest, and at 12 channels in 16 slots that cost a third of the bandwidth.
    if (ws == 1) {
        if (slots <= 8) PLH_LN_V(8, 1);
        else if (slots <= 12) PLH_LN_V(12, 1);
        else if (slots <= 16) PLH_LN_V(16, 1);
        else if (slots <= 24) PLH_LN_V(24, 1);
        else PLH_LN_V(32, 1);
    } else if (ws == 4) {
        if (slots <= 12) PLH_LN_V(12, 4);
        else PLH_LN_V(16, 4);
    } else if (slots <= 12) PLH_LN_V(12, 8);
    else if (slots <= 16) PLH_LN_V(16, 8);
    else if (slots <= 24) PLH_LN_V(24, 8);
    else if (slots <= 32) PLH_LN_V(32, 8);
    else if (slots <= 48) PLH_LN_V(48, 8);
    else if (slots <= 64) { if (narrow) PLH_LN_NARROW(64, 8); else PLH_LN_V(64, 8); }
    else if (slots <= 96) { if (narrow) PLH_LN_NARROW(96, 8); else PLH_LN_V(96, 8); }      // C <= 768
    else PLH_LN(128, 1, 8);                            // 768 < C <= 1024: one pixel per lane
#undef PLH_LN_NARROW
#undef PLH_LN_V
#undef PLH_LN_IMAGE
#undef PLH_LN
}

// Per-dtype entry, instantiated in layernorm_f32.hip / layernorm_f16.hip / layernorm_bf16.hip.
template <class T>
void ln_run_typed(bool bwd, const T *x, const T *g, T *out, int64_t n_size, int64_t dimsize, int64_t m_size, float eps,
                  hipStream_t st) {
    if (bwd) ln_launch<T, true>(x, g, out, n_size, dimsize, m_size, eps, st);
    else ln_launch<T, false>(x, g, out, n_size, dimsize, m_size, eps, st);
}

#define PLH_LN_SIGNATURE(T) void ln_run_typed<T>(bool, const T *, const T *, T *, int64_t, int64_t, int64_t, float, hipStream_t);
#define PLH_LN_EXTERN(T) extern template PLH_LN_SIGNATURE(T)
#define PLH_LN_INSTANTIATE(T) template PLH_LN_SIGNATURE(T)

}  // namespace plh
