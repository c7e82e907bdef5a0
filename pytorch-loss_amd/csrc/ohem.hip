// Online hard example mining by score for gfx950: softmax probability at the label, then the
// relabelling rule "beyond the n_min lowest scores, a pixel whose score exceeds the threshold
// becomes ignore_index" (csrc/ohem_label_kernel.cu:112-168, 171-263).
//
// The reference sorts all P scores with their indices (thrust::sort_by_key, :247) only to learn,
// per pixel, whether its sorted position is below n_min. That is an order-statistic question, so
// nothing is sorted here:
//   1. scores      one pass over the logits (channel slice in registers), P fp32 scores out;
//   2. select      a 3-digit (10 bits each) radix select over the score bit patterns finds v, the
//                  n_min-th smallest score, and how many pixels with exactly that score still
//                  fall below position n_min (`keep_ties`); the histogram kernel of a digit first
//                  resolves the digit before it (every block for itself, from the finished table);
//   3. ties        pixels equal to v are ranked in pixel order (what a stable key sort gives): a
//                  wavefront per run of tiles counts them (running count per tile, total per run),
//                  the relabelling adds up the runs before its own, in-tile ranks from ballots;
//   4. relabel     drop = score > thresh && (score > v || (score == v && tie_rank >= keep_ties)).
// When v <= thresh every pixel above the threshold lies beyond position n_min, so steps 3 is
// skipped on the device (the kernels return at once). Scores are positive floats, whose bit
// patterns order like the values; patterns are clamped to that of 1.0f, so a NaN score ranks as
// 1 and, failing `score > thresh`, is never relabelled.
#include "plh_common.hpp"

namespace plh {

constexpr int kOhemBins = 1024;                 // 10 bits per digit, 3 digits cover [0, 0x3F800000]
constexpr int kOhemTile = 1024;                 // pixels per block in the tie-ranking passes (256 threads x 4)
constexpr int kOhemZeroWords = 3 * kOhemBins + 16;   // histograms and state of the selection: zero before use
constexpr uint32_t kOneBits = 0x3F800000u;


__device__ __forceinline__ uint32_t score_key(float s) {
    const uint32_t b = __builtin_bit_cast(uint32_t, s);
    return b > kOneBits ? kOneBits : b;
}
__device__ __forceinline__ int key_digit(uint32_t key, int pass) { return (int)((key >> (20 - 10 * pass)) & 1023u); }

// ------------------------------------------------------------------ scores ----
// `none` is what a pixel without a target (ignored, or a label outside [0, C)) scores: 1, as the reference
// writes it (csrc/ohem_label_kernel.cu:131-134), or kNoTargetMark for the forwards that hand their selection
// on as a mask and have to tell such a pixel from a valid one that scores exactly 1 without reading the labels
// again. Both sort last (score_key clamps at 1) and tie with each other in pixel order.
constexpr float kNoTargetMark = 2.f;

constexpr int kEarlyFlag = 8;       // index into OhemTables::state: raised when the threshold rule decided (OhemEarly)


template <class T, int CP, int V, int Form>
__global__ __launch_bounds__(kRegsBlock) void ohem_scores_regs(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                              float *__restrict__ scores, float *__restrict__ ce,
                                                              int64_t P, int64_t m_size, int C, int64_t ignore,
                                                              unsigned xcd_run, uint32_t *__restrict__ tables, float none,
                                                              const OhemEarly ev) {
    __shared__ float red[4];
    const bool early = ev.kept != nullptr;              // uniform over the grid
    // the selection's tables start at zero; the kernels that fill them are launched after this one
    if (tables && blockIdx.x == 0)
        for (int i = threadIdx.x; i < kOhemZeroWords; i += kRegsBlock) tables[i] = 0;
    const PixelRef<V, Form> at(P, m_size, C, xcd_run);
    if (!early && !at.live) return;
    // labels (and the upstream gradient) first: in the rows form the slice arrives through LDS behind a wait
    int64_t lb[V];
    at.labels(lab, ignore, lb);
    typename Pack<T, V>::Raw raw[CP];
    at.load_slice(x, C, m_size, raw);
    float out[V], loss[V];
    bool kp[V];
    float kept_sum = 0.f;
    int kept_cnt = 0, below_cnt = 0;
#pragma unroll
    for (int k = 0; k < V; ++k) {
        bool ign;
        const int tgt = narrow_label(lb[k], ignore, C, ign);
        float xv[CP];
        const float mx = widen_and_max<T, V, CP>(raw, k, C, xv);
        const float c = mx * kLog2e;
        float s = 0.f, e_y = 0.f, x_y = mx;
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (chan_ok<CP>(j, C)) {
                const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(xv[j], kLog2e, -c));
                s += e;
                e_y = (tgt == j) ? e : e_y;
                x_y = (tgt == j) ? xv[j] : x_y;
            }
        // ignored pixels score 1 (ohem_label_kernel.cu:131-134); so does a label outside [0, C),
        // which the reference leaves undefined
        out[k] = (tgt < 0) ? none : fminf(e_y * __builtin_amdgcn_rcpf(s), 1.f);
        // the pixel's cross entropy from the same sums, exact also where the score underflows
        loss[k] = (tgt < 0) ? 0.f : __builtin_fmaf(__builtin_amdgcn_logf(s), kLn2, mx - x_y);
        if (early) {
            const bool real = at.live && k < at.nv;
            kp[k] = real && tgt >= 0 && !(out[k] > ev.thresh);
            kept_sum += kp[k] ? loss[k] : 0.f;
            kept_cnt += kp[k] ? 1 : 0;
            below_cnt += (real && fminf(out[k], 1.f) <= ev.thresh) ? 1 : 0;      // fminf: a NaN score counts as 1
        }
    }
    if (at.live) {
        // the selection kernels read both back several times: leave them to the caches (in the threshold-rule case
        // nothing reads them again; stores that bypass the caches measured the same there)
        at.store_f32_cached(scores, out);
        if (ce) at.store_f32_cached(ce, loss);
    }
    if (early) {
        if (at.live) store_kept<V>(ev.kept, at.pix, at.nv, kp);
        const float bs = block_sum_256(kept_sum, red);
        const float bk = block_sum_256((float)kept_cnt, red);         // at most 1024 per block: exact in fp32
        const float bb = block_sum_256((float)below_cnt, red);
        if (threadIdx.x == 0) {
            ev.sum[blockIdx.x] = bs;
            ev.cnt[blockIdx.x] = (int)bk;
            ev.below[blockIdx.x] = (int)bb;
        }
    }
}

// 33..256 channels in NCHW (SplitSlice): per wavefront the maximum, the exponential sum and the target's
// logit of its channels; wavefront 0 combines them into the pixel's score and cross entropy.
template <class T, int KW, int V, bool PerImage = false>
__global__ __launch_bounds__(kSplitBlock) void ohem_scores_split(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                                float *__restrict__ scores, float *__restrict__ ce,
                                                                int64_t P, int64_t m_size, int C, int64_t ignore,
                                                                unsigned xcd_run, uint32_t *__restrict__ tables, float none) {
    __shared__ float parts[3][kSplitWaves][kWave * V];
    if (tables && blockIdx.x == 0)
        for (int i = threadIdx.x; i < kOhemZeroWords; i += kSplitBlock) tables[i] = 0;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const SplitSlice<T, V, KW, PerImage> at(P, m_size, C, xcd_run);
    int64_t lb[V];
    at.labels(lab, ignore, lb);
    if (at.here > 0) {                                  // wave-uniform
        typename Pack<T, V>::Raw raw[KW];
        at.load(x, C, m_size, raw);
#pragma unroll
        for (int k = 0; k < V; ++k) {
            bool ign;
            const int rel = narrow_label(lb[k], ignore, C, ign) - at.first;
            float xv[KW];
            float mx = -INFINITY, x_y = -INFINITY;
#pragma unroll
            for (int i = 0; i < KW; ++i) {
                xv[i] = (i < at.here) ? Pack<T, V>::get(raw[i], k) : -INFINITY;
                mx = fmaxf(mx, xv[i]);
                x_y = (rel == i) ? xv[i] : x_y;
            }
            float s = 0.f;
#pragma unroll
            for (int i = 0; i < KW; ++i) s += fast_exp(xv[i] - mx);
            const int q = lane * V + k;
            parts[0][wave][q] = mx;
            parts[1][wave][q] = s;
            parts[2][wave][q] = x_y;
        }
    }
    __syncthreads();
    if (wave >= V || !at.live || wave >= at.nv) return;     // wavefront k finishes pixel k of every lane
    const int used = (C + KW - 1) / KW;
    bool ign;
    PLH_SPLIT_MY_LABEL(my_lb, lb, wave, V)
    const int tgt = narrow_label(my_lb, ignore, C, ign);
    const int q = lane * V + wave;
    float M = parts[0][0][q];
    for (int w = 1; w < used; ++w) M = fmaxf(M, parts[0][w][q]);
    float S = 0.f, x_y = -INFINITY;
    for (int w = 0; w < used; ++w) {
        S = __builtin_fmaf(parts[1][w][q], fast_exp(parts[0][w][q] - M), S);
        x_y = fmaxf(x_y, parts[2][w][q]);
    }
    scores[at.pix + wave] = (tgt < 0) ? none : fminf(fast_exp(x_y - M) * __builtin_amdgcn_rcpf(S), 1.f);
    if (ce) ce[at.pix + wave] = (tgt < 0) ? 0.f : fast_log(S) + (M - x_y);
}

// Any channel count: a lane per pixel, two sweeps over the slice (the second one hits cache).
template <class T>
__global__ __launch_bounds__(256) void ohem_scores_lane(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                        float *__restrict__ scores, float *__restrict__ ce, int64_t P,
                                                        int64_t m_size, int C, int64_t ignore,
                                                        uint32_t *__restrict__ tables, float none) {
    if (tables && blockIdx.x == 0)
        for (int i = threadIdx.x; i < kOhemZeroWords; i += 256) tables[i] = 0;
    for (int64_t pix = (int64_t)blockIdx.x * 256 + threadIdx.x; pix < P; pix += (int64_t)gridDim.x * 256) {
        const int64_t lb = lab[pix];
        if (lb == ignore || lb < 0 || lb >= C) {
            scores[pix] = none;
            if (ce) ce[pix] = 0.f;
            continue;
        }
        const int64_t n = pix / m_size;
        const T *xs = x + (pix + n * (int64_t)(C - 1) * m_size);
        float mx = -INFINITY;
#pragma unroll 8
        for (int j = 0; j < C; ++j) mx = fmaxf(mx, load_one(xs + (int64_t)j * m_size));
        float s = 0.f;
#pragma unroll 8
        for (int j = 0; j < C; ++j) s += fast_exp(load_one(xs + (int64_t)j * m_size) - mx);
        const float x_y = load_one(xs + lb * m_size);
        scores[pix] = fminf(fast_exp(x_y - mx) / s, 1.f);
        if (ce) ce[pix] = logf(s) + (mx - x_y);
    }
}

// (N, C) inputs with 33..2048 channels: a wavefront per row, the row in its registers (one read of HBM,
// every access a contiguous run), where the lane-per-pixel kernel would have each lane walk its own row.
template <class T, int NI, int LP, int G>
__global__ __launch_bounds__(256) void ohem_scores_wrow(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                        float *__restrict__ scores, float *__restrict__ ce, int64_t P,
                                                        int C, int64_t ignore, uint32_t *__restrict__ tables, float none) {
    if (tables && blockIdx.x == 0)
        for (int i = threadIdx.x; i < kOhemZeroWords; i += 256) tables[i] = 0;
    constexpr int L = WaveRow<T, NI, LP, G>::L;
    const WaveRowAt<G> at;
    for (int64_t r0 = at.start; r0 < P; r0 += at.stride) {   // wave-uniform
        const bool live = r0 + at.grp < P;
        const int64_t row = live ? r0 + at.grp : P - 1;
        const int64_t lb = lab[row];
        const bool no_target = (lb == ignore || lb < 0 || lb >= C);
        if constexpr (G == 64) {                              // the wavefront has one row: skip its loads
            if (no_target) {
                if (at.sub == 0) {
                    scores[row] = none;
                    if (ce) ce[row] = 0.f;
                }
                continue;
            }
        }
        const T *xs = x + row * C;
        WaveRow<T, NI, LP, G> r;
        r.load(xs, C, at.sub);
        const float mx = r.max();
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < NI; ++i)
#pragma unroll
            for (int l = 0; l < L; ++l) s += fast_exp(r.v[i][l] - mx);      // -inf beyond the row
        s = group_reduce<G>(s, OpSum());
        if (at.sub == 0 && live) {
            const float x_y = load_one(xs + (no_target ? 0 : lb));
            scores[row] = no_target ? none : fminf(fast_exp(x_y - mx) / s, 1.f);
            if (ce) ce[row] = no_target ? 0.f : logf(s) + (mx - x_y);
        }
    }
}

// (N, C) inputs with longer rows (a vocabulary): a 1024-thread block per row at a time, the row read once
// with running (maximum, exponential sum) statistics per lane.
template <class T>
__global__ __launch_bounds__(kRowBlock) void ohem_scores_row(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                             float *__restrict__ scores, float *__restrict__ ce,
                                                             int64_t P, int C, int64_t ignore,
                                                             uint32_t *__restrict__ tables, int vec, float none) {
    __shared__ float red[kRowBlock / 64];
    if (tables && blockIdx.x == 0)
        for (int i = threadIdx.x; i < kOhemZeroWords; i += row_threads()) tables[i] = 0;
    for (int64_t row = blockIdx.x; row < P; row += gridDim.x) {       // block-uniform
        const int64_t lb = lab[row];
        if (lb == ignore || lb < 0 || lb >= C) {
            if (threadIdx.x == 0) {
                scores[row] = none;
                if (ce) ce[row] = 0.f;
            }
            continue;
        }
        const T *xs = x + row * C;
        const RowStats st = row_combine(row_sweep<T>(xs, C, vec != 0), red, false);
        if (threadIdx.x == 0) {
            const float x_y = load_one(xs + lb);
            scores[row] = fminf(fast_exp(x_y - st.m) / st.s, 1.f);
            if (ce) ce[row] = logf(st.s) + (st.m - x_y);
        }
    }
}

// ------------------------------------------------------------------ select ----

// Tables of the selection, all in the caller's workspace. `state` (16 words, zeroed with the
// histograms): [2*pass] = key prefix after `pass`+1 digits, [2*pass+1] = 1-based rank of the
// n_min-th smallest key among the keys sharing that prefix.
struct OhemTables {
    uint32_t *hist;        // [3][kOhemBins]
    uint32_t *state;       // [16]
    uint32_t *tile_ties;   // [tiles]: ties in the earlier tiles of the same run; then [kTieRuns]: ties per run
};

// The tie count: kTieRuns runs of consecutive tiles, a wavefront per run.
constexpr int kTieRuns = 1024;
__host__ __device__ inline int tie_run_tiles(int tiles) { return (tiles + kTieRuns - 1) / kTieRuns; }

__global__ void ohem_zero(uint32_t *p, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

// One digit of the selection, by one 256-thread block: in histogram `h` (kOhemBins counts) find the
// bin where the running count first reaches `rank` (1-based) and the rank left inside that bin.
// Every thread gets the result. `lds` holds at least 260 words.
__device__ void ohem_pick_digit(const uint32_t *h, uint32_t rank, uint32_t *lds, uint32_t &digit, uint32_t &rank_in_bin) {
    const int t = threadIdx.x;
    uint32_t b[4];                               // 4 consecutive bins per thread, then a scan over the 256 sums
#pragma unroll
    for (int i = 0; i < 4; ++i) b[i] = h[t * 4 + i];
    const uint32_t mine = b[0] + b[1] + b[2] + b[3];
    lds[t] = mine;
    if (t == 0) { lds[256] = 0; lds[257] = 1; }
    __syncthreads();
    for (int off = 1; off < 256; off <<= 1) {
        const uint32_t add = (t >= off) ? lds[t - off] : 0u;
        __syncthreads();
        lds[t] += add;
        __syncthreads();
    }
    const uint32_t incl = lds[t], excl = incl - mine;
    if (excl < rank && rank <= incl) {           // exactly one thread owns the bin
        uint32_t run = excl;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (run < rank && rank <= run + b[i]) {
                lds[256] = (uint32_t)(t * 4 + i);
                lds[257] = rank - run;
            }
            run += b[i];
        }
    }
    __syncthreads();
    digit = lds[256];
    rank_in_bin = lds[257];
    __syncthreads();
}

// Digit `pass` of the selection from its finished histogram: returns the key prefix including that
// digit. Every block of a kernel may call it (same inputs, same answer); the one with `publish`
// stores prefix and remaining rank for the kernels launched later.
__device__ uint32_t ohem_resolve_digit(const OhemTables &tb, int pass, uint32_t n_min, uint32_t *lds, bool publish) {
    const uint32_t before = pass == 0 ? 0u : tb.state[2 * (pass - 1)];
    const uint32_t rank = pass == 0 ? n_min : tb.state[2 * (pass - 1) + 1];
    uint32_t digit, rank_in_bin;
    ohem_pick_digit(tb.hist + pass * kOhemBins, rank, lds, digit, rank_in_bin);
    const uint32_t prefix = before | (digit << (20 - 10 * pass));
    if (publish && threadIdx.x == 0) {
        tb.state[2 * pass] = prefix;
        tb.state[2 * pass + 1] = rank_in_bin;
    }
    return prefix;
}

__device__ __forceinline__ void hist_add(uint32_t *bins, float s, uint32_t high_mask, uint32_t prefix, int pass) {
    const uint32_t key = score_key(s);
    if ((key & high_mask) == prefix) atomicAdd(&bins[key_digit(key, pass)], 1u);
}

// Histogram of digit `pass` over the keys that share the leading digits, the last of which the
// block resolves first. (A device-wide "last block resolves it" would need a release fence in every
// block, which costs more than this redundant scan of 1024 counts on a GPU whose XCDs have separate
// L2s; so does a launch of its own.)
// Once the digits resolved so far put the n_min-th smallest score at or below the threshold whatever its
// remaining digits are, the rule is "drop what lies above the threshold" and nothing finer is needed: the
// later passes leave their histograms empty (every block returns before it reads a score), the digits they
// resolve from those come out as 0, and the key that ohem_ties publishes stays below the threshold.
__global__ __launch_bounds__(256) void ohem_hist(const float *__restrict__ scores, OhemTables tb, int P, int pass,
                                                 uint32_t n_min, float thresh, int vec,
                                                 const int *__restrict__ below, unsigned below_blocks) {
    __shared__ uint32_t bins[kOhemBins];
    __shared__ uint32_t scan[260];
    if (pass > 0 && tb.state[kEarlyFlag]) return;            // uniform over the grid
    if (pass == 0 && below) {
        // the score kernel counted, per block, the pixels that score within the threshold: with n_min or more of them
        // the threshold rule is the whole selection (every block adds the numbers up for itself, block 0 says so)
        // (the array is 16-byte aligned: four 16-byte loads in flight per thread and trip)
        __shared__ float red[4];
        typedef int i4 __attribute__((ext_vector_type(4)));
        int mine = 0;
        const i4 *b4 = reinterpret_cast<const i4 *>(below);
        const unsigned quads = below_blocks / 4;
        for (unsigned i = threadIdx.x; i < quads; i += 1024) {
            i4 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = i + u * 256 < quads ? b4[i + u * 256] : i4{0, 0, 0, 0};
#pragma unroll
            for (int u = 0; u < 4; ++u) mine += (v[u].x + v[u].y) + (v[u].z + v[u].w);
        }
        if (threadIdx.x < below_blocks - quads * 4) mine += below[quads * 4 + threadIdx.x];
        // per thread at most 2^31 / 256 pixels, in whole numbers a float holds up to 2^24: sum as two halves
        const float lo = block_sum_256((float)(mine & 0xFFFF), red), hi = block_sum_256((float)(mine >> 16), red);
        const uint64_t total = (uint64_t)lo + ((uint64_t)hi << 16);
        if (total >= n_min) {
            if (blockIdx.x == 0 && threadIdx.x == 0) tb.state[kEarlyFlag] = 1;
            return;
        }
    }
    for (int i = threadIdx.x; i < kOhemBins; i += 256) bins[i] = 0;
    const uint32_t prefix = pass == 0 ? 0u : ohem_resolve_digit(tb, pass - 1, n_min, scan, blockIdx.x == 0);
    if (pass > 0) {
        const uint32_t largest = prefix | ((1u << (30 - 10 * pass)) - 1u);      // block-uniform
        if (__builtin_bit_cast(float, largest) <= thresh) return;
    }
    __syncthreads();
    const uint32_t high_mask = pass == 0 ? 0u : (0xFFFFFFFFu << (30 - 10 * pass));
    const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x, stride = (int64_t)gridDim.x * 256;
    if (vec) {
        const int64_t quads = P / 4;
        const plh_f4 *s4 = reinterpret_cast<const plh_f4 *>(scores);
        int64_t i = gid;
        for (; i + 3 * stride < quads; i += 4 * stride) {        // four loads in flight per lane
            plh_f4 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = s4[i + u * stride];     // scores are read again: ordinary loads
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                hist_add(bins, v[u].x, high_mask, prefix, pass);
                hist_add(bins, v[u].y, high_mask, prefix, pass);
                hist_add(bins, v[u].z, high_mask, prefix, pass);
                hist_add(bins, v[u].w, high_mask, prefix, pass);
            }
        }
        for (; i < quads; i += stride) {
            const plh_f4 v = s4[i];
            hist_add(bins, v.x, high_mask, prefix, pass);
            hist_add(bins, v.y, high_mask, prefix, pass);
            hist_add(bins, v.z, high_mask, prefix, pass);
            hist_add(bins, v.w, high_mask, prefix, pass);
        }
        if (gid < P - quads * 4) hist_add(bins, scores[quads * 4 + gid], high_mask, prefix, pass);
    } else {
        for (int64_t i = gid; i < P; i += stride) hist_add(bins, scores[i], high_mask, prefix, pass);
    }
    __syncthreads();
    uint32_t *out = tb.hist + pass * kOhemBins;
    for (int i = threadIdx.x; i < kOhemBins; i += 256)
        if (bins[i]) atomicAdd(out + i, bins[i]);
}

// This thread's 4 consecutive scores and their keys; pixels beyond the end match no key.
__device__ __forceinline__ void load_tile_keys(const float *scores, int P, int base, bool vec, float (&s)[4],
                                               uint32_t (&key)[4]) {
    if (vec && base + 3 < P) {
        const plh_f4 v = *reinterpret_cast<const plh_f4 *>(scores + base);
        s[0] = v.x; s[1] = v.y; s[2] = v.z; s[3] = v.w;
#pragma unroll
        for (int k = 0; k < 4; ++k) key[k] = score_key(s[k]);
        return;
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int i = base + k;
        s[k] = i < P ? scores[i] : 2.f;
        key[k] = i < P ? score_key(s[k]) : 0xFFFFFFFFu;
    }
}

// The last digit (every block for itself, block 0 publishes: state[4] = v, the n_min-th smallest key,
// state[5] = how many pixels equal to it lie below sorted position n_min), then, only when v exceeds
// the threshold (otherwise no rank among the ties is ever looked at), the ties in pixel order: each
// wavefront walks one run of consecutive tiles and leaves, per tile, the ties in the run's earlier
// tiles, and per run its total. One launch where a pick, a count and a scan kernel were three.
__global__ __launch_bounds__(256) void ohem_ties(const float *__restrict__ scores, OhemTables tb, int P, int tiles,
                                                 uint32_t n_min, float thresh, int vec) {
    __shared__ uint32_t scan[260];
    if (tb.state[kEarlyFlag]) return;                           // uniform over the grid
    const uint32_t v = ohem_resolve_digit(tb, 2, n_min, scan, blockIdx.x == 0);
    if (!(__builtin_bit_cast(float, v) > thresh)) return;       // block-uniform
    const int lane = threadIdx.x & 63;
    const int run = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int per = tie_run_tiles(tiles);
    uint32_t before = 0;
    for (int t = run * per; t < min(tiles, (run + 1) * per); ++t) {      // wave-uniform
        uint32_t n = 0;
#pragma unroll
        for (int q = 0; q < kOhemTile / 256; ++q) {             // a tile is 1024 pixels: 4 x (64 lanes x 4)
            float s[4];
            uint32_t key[4];
            load_tile_keys(scores, P, t * kOhemTile + (q * 64 + lane) * 4, vec != 0, s, key);
#pragma unroll
            for (int k = 0; k < 4; ++k) n += key[k] == v ? 1u : 0u;
        }
        n = (uint32_t)group_reduce<64>((float)n, OpSum());      // <= 1024: exact
        if (lane == 0) tb.tile_ties[t] = before;
        before += n;
    }
    if (lane == 0 && run < kTieRuns) tb.tile_ties[tiles + run] = before;
}

// With `part`, the block also leaves the sum of `ce` over the pixels that keep a label other than
// `ignore`, and their number: the mean cross entropy of the relabelled batch needs no further pass
// over the logits.
// With `kept`, the labels are neither read nor written: the kernel leaves one byte per pixel instead, 1 where
// the pixel keeps a label other than `ignore` (pixels without a target carry kNoTargetMark as their score).
__global__ __launch_bounds__(256) void ohem_relabel(const float *__restrict__ scores, const int64_t *__restrict__ lab,
                                                    int64_t *__restrict__ out, OhemTables tb, int P, int tiles, uint32_t n_min,
                                                    float thresh, int64_t ignore, int vec,
                                                    const float *__restrict__ ce, Partials part,
                                                    uint8_t *__restrict__ kept_out) {
    __shared__ uint32_t wave_ties[4], run_ties[4];
    __shared__ float red[4];
    if (n_min != 0 && tb.state[kEarlyFlag]) return;     // uniform over the grid: the score kernel has left mask and sums
    const int base = blockIdx.x * kOhemTile + threadIdx.x * 4;
    float s[4];
    uint32_t key[4];
    load_tile_keys(scores, P, base, vec != 0, s, key);
    bool drop[4];
    const uint32_t v = n_min == 0 ? 0u : tb.state[4];
    if (n_min == 0 || !(__builtin_bit_cast(float, v) > thresh)) {
        // every position is beyond n_min, or the n_min-th smallest score is within the threshold:
        // all scores above the threshold lie beyond position n_min
#pragma unroll
        for (int k = 0; k < 4; ++k) drop[k] = s[k] > thresh;
    } else {
        // rank of this thread's ties in pixel order: tiles before, waves before, lanes before
        const uint32_t keep_ties = tb.state[5];
        int mine = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) mine += key[k] == v ? 1 : 0;
        int lane_incl = mine;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int up = __shfl_up(lane_incl, off, 64);
            if ((threadIdx.x & 63) >= off) lane_incl += up;
        }
        if ((threadIdx.x & 63) == 63) wave_ties[threadIdx.x >> 6] = (uint32_t)lane_incl;
        // ties in the runs of tiles before this tile's run (ohem_ties): kTieRuns totals, 4 per thread
        const int my_run = blockIdx.x / tie_run_tiles(tiles);
        uint32_t earlier = 0;
#pragma unroll
        for (int q = 0; q < kTieRuns / 256; ++q) {
            const int r = q * 256 + threadIdx.x;
            earlier += r < my_run ? tb.tile_ties[tiles + r] : 0u;
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) earlier += (uint32_t)__shfl_xor((int)earlier, off, 64);
        if ((threadIdx.x & 63) == 0) run_ties[threadIdx.x >> 6] = earlier;
        __syncthreads();                                           // also what wave_ties needs
        const uint32_t runs_before = (run_ties[0] + run_ties[1]) + (run_ties[2] + run_ties[3]);
        uint32_t before = runs_before + tb.tile_ties[blockIdx.x] + (uint32_t)(lane_incl - mine);
        for (int w = 0; w < (int)(threadIdx.x >> 6); ++w) before += wave_ties[w];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const bool tie = key[k] == v;
            drop[k] = key[k] != 0xFFFFFFFFu && (key[k] > v || (tie && before >= keep_ties)) && s[k] > thresh;
            before += tie ? 1u : 0u;
        }
    }
    bool kept[4] = {false, false, false, false};
    if (kept_out) {                                     // uniform over the grid
#pragma unroll
        for (int k = 0; k < 4; ++k) kept[k] = base + k < P && !drop[k] && !(s[k] > 1.5f);
        if (base + 3 < P) {
            *reinterpret_cast<uint32_t *>(kept_out + base) =
                (uint32_t)kept[0] | ((uint32_t)kept[1] << 8) | ((uint32_t)kept[2] << 16) | ((uint32_t)kept[3] << 24);
        } else {
#pragma unroll
            for (int k = 0; k < 4; ++k)
                if (base + k < P) kept_out[base + k] = kept[k] ? 1 : 0;
        }
    } else if (vec && base + 3 < P) {
        const plh_l2 *in2 = reinterpret_cast<const plh_l2 *>(lab + base);
        plh_l2 *out2 = reinterpret_cast<plh_l2 *>(out + base);
        plh_l2 a = __builtin_nontemporal_load(in2), b = __builtin_nontemporal_load(in2 + 1);
        a.x = drop[0] ? ignore : a.x; a.y = drop[1] ? ignore : a.y;
        b.x = drop[2] ? ignore : b.x; b.y = drop[3] ? ignore : b.y;
        __builtin_nontemporal_store(a, out2);
        __builtin_nontemporal_store(b, out2 + 1);
        kept[0] = a.x != ignore; kept[1] = a.y != ignore; kept[2] = b.x != ignore; kept[3] = b.y != ignore;
    } else {
#pragma unroll
        for (int k = 0; k < 4; ++k)
            if (base + k < P) {
                const int64_t nl = drop[k] ? ignore : lab[base + k];
                out[base + k] = nl;
                kept[k] = nl != ignore;
            }
    }
    if (part.sum == nullptr) return;            // uniform over the grid
    float mine = 0.f, cnt = 0.f;
#pragma unroll
    for (int k = 0; k < 4; ++k)
        if (kept[k]) {
            mine += ce[base + k];
            cnt += 1.f;
        }
    const float bs = block_sum_256(mine, red);
    const float bc = block_sum_256(cnt, red);
    if (threadIdx.x == 0) {
        part.sum[blockIdx.x] = bs;
        part.cnt[blockIdx.x] = (int)bc;
    }
}

// The mean over the kept pixels from whichever pass produced the final sums: the score kernel's (threshold rule,
// kEarlyFlag raised) or the relabelling pass's.
__global__ __launch_bounds__(1024) void ohem_finish(const uint32_t *__restrict__ state, Partials early, unsigned early_blocks,
                                                    Partials late, unsigned late_blocks, float *__restrict__ loss_out,
                                                    int64_t *__restrict__ count_out) {
    const bool e = state[kEarlyFlag] != 0;              // uniform
    finish_block(e ? early.sum : late.sum, e ? early.cnt : late.cnt, e ? early_blocks : late_blocks, loss_out, count_out,
                 kFinishMeanOverCount, 0);
}

__global__ void ohem_copy_labels(const int64_t *__restrict__ in, int64_t *__restrict__ out, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        out[i] = in[i];
}

// ------------------------------------------------------------ host side ----

constexpr int64_t kOhemMaxPixels = ((int64_t)1 << 31) - kOhemTile;

static int64_t align256(int64_t v) { return (v + 255) / 256 * 256; }
static int64_t ohem_tiles(int64_t P) { return ceil_div(P > 0 ? P : 1, kOhemTile); }

static int launch_scores(const void *logits, int32_t dtype, const int64_t *labels, float *scores, float *ce,
                         int64_t n_size, int64_t dimsize, int64_t m_size, int64_t ignore_index, hipStream_t st,
                         uint32_t *tables = nullptr, float none = 1.f, const OhemEarly *early = nullptr,
                         unsigned *early_blocks = nullptr) {
    // `early`: taken up by the kernels that keep a pixel's channels in a lane's registers; *early_blocks then is their
    // grid (0: the launch shape produces none of it)
    const int64_t P = n_size * m_size;
    const int C = (int)dimsize;
    const OhemEarly ev = early ? *early : OhemEarly{nullptr, nullptr, nullptr, nullptr, 0.f};
    if (early_blocks) *early_blocks = 0;
    dispatch_dtype(dtype, [&](auto tag) {
        using T = decltype(tag);
        const T *x = static_cast<const T *>(logits);
        constexpr int VT = ElemTraits<T>::kVec;
        const Shape shape = pick_shape(dimsize, m_size, VT, sizeof(T), x, nullptr, labels, scores, ce, true, true, true,
                                       kImageFormMaxChannels<T>);
        if (shape == Shape::SplitDeep) {            // 257..512 channels: up to 64 slots per wavefront, half the pixels per lane
            constexpr int VD = VT / 2;
            const unsigned grid = split_grid<VD>(P);
            const unsigned run = xcd_run_for(sizeof(T), m_size);
            switch (split_slots_deep(dimsize)) {
#define PLH_CASE(KW)                                                                                                  \
    case KW:                                                                                                          \
        hipLaunchKernelGGL((ohem_scores_split<T, KW, VD>), dim3(grid), dim3(kSplitBlock), 0, st, x, labels, scores, ce, \
                           P, m_size, C, ignore_index, run, tables, none);                                                  \
        break;
                PLH_SPLIT_DEEP_CASES
#undef PLH_CASE
            }
        } else if (shape == Shape::SplitImage) {    // tiles per image: channel planes that start on element boundaries only
            const unsigned grid = split_image_grid<VT>(n_size, m_size);
            const unsigned run = xcd_run_for(sizeof(T), m_size);
            switch (split_slots(dimsize)) {
#define PLH_CASE(KW)                                                                                                  \
    case KW:                                                                                                          \
        hipLaunchKernelGGL((ohem_scores_split<T, KW, VT, true>), dim3(grid), dim3(kSplitBlock), 0, st, x, labels, scores, \
                           ce, P, m_size, C, ignore_index, run, tables, none);                                              \
        break;
                PLH_SPLIT_SLOT_CASES
#undef PLH_CASE
            }
        } else if (shape == Shape::Split) {
            const unsigned grid = split_grid<VT>(P);
            const unsigned run = xcd_run_for(sizeof(T), m_size);
            switch (split_slots(dimsize)) {
#define PLH_CASE(KW)                                                                                                  \
    case KW:                                                                                                          \
        hipLaunchKernelGGL((ohem_scores_split<T, KW, VT>), dim3(grid), dim3(kSplitBlock), 0, st, x, labels, scores, ce, \
                           P, m_size, C, ignore_index, run, tables, none);                                                  \
        break;
                PLH_SPLIT_SLOT_CASES
#undef PLH_CASE
            }
        } else if (shape == Shape::RegsVec || shape == Shape::RegsOne) {
            const bool vec = (shape == Shape::RegsVec);
            const bool uni = vec && tiles_are_uniform(m_size, VT, sizeof(T));
            // planes that start on element boundaries only: tiles per image, four pixels per lane
            const bool image = !vec && image_form_pays<T>(C, m_size);
            const unsigned grid = vec ? regs_grid<VT>(P) : (image ? image_grid<4>(n_size, m_size) : regs_grid<1>(P));
            const unsigned run = xcd_run_for(sizeof(T), m_size);
            if (early_blocks && ev.kept) *early_blocks = grid;
            switch ((C + 3) / 4) {
#define PLH_CASE(K)                                                                                                   \
    case K:                                                                                                           \
        if (uni) hipLaunchKernelGGL((ohem_scores_regs<T, 4 * K, VT, kUniform>), dim3(grid), dim3(kRegsBlock), 0, st,  \
                                    x, labels, scores, ce, P, m_size, C, ignore_index, run, tables, none, ev);              \
        else if (vec) hipLaunchKernelGGL((ohem_scores_regs<T, 4 * K, VT, kGeneral>), dim3(grid), dim3(kRegsBlock), 0, \
                                         st, x, labels, scores, ce, P, m_size, C, ignore_index, run, tables, none, ev);     \
        else if (image) {                                                                                             \
            if constexpr (4 * K <= kImageFormMaxChannels<T>)                                                          \
                hipLaunchKernelGGL((ohem_scores_regs<T, 4 * K, 4, kPerImage>), dim3(grid), dim3(kRegsBlock), 0, st,   \
                                   x, labels, scores, ce, P, m_size, C, ignore_index, run, tables, none, ev);               \
        } else hipLaunchKernelGGL((ohem_scores_regs<T, 4 * K, 1, kGeneral>), dim3(grid), dim3(kRegsBlock), 0, st, x,  \
                                  labels, scores, ce, P, m_size, C, ignore_index, run, tables, none, ev);                   \
        break;
                PLH_CASE(1) PLH_CASE(2) PLH_CASE(3) PLH_CASE(4) PLH_CASE(5) PLH_CASE(6) PLH_CASE(7) PLH_CASE(8)
#undef PLH_CASE
            }
        } else if (shape == Shape::Wave && C <= wrow_cap<T>(wrow_piece<T>(x, (const T *)nullptr, C))) {
#define PLH_GO(NI, W, G)                                                                                            \
    hipLaunchKernelGGL((ohem_scores_wrow<T, NI, W, G>), dim3(group_grid(P, WaveRowAt<G>::kRowsPerBlock)), dim3(256), 0, \
                       st, x, labels, scores, ce, P, C, ignore_index, tables, none)
            PLH_WROW_DISPATCH(wrow_piece<T>(x, (const T *)nullptr, C), C, PLH_GO);
#undef PLH_GO
        } else if (shape == Shape::Wave) {
            const unsigned grid = (unsigned)(P < 1 ? 1 : (P < kMinPartialSlots ? P : kMinPartialSlots));
            hipLaunchKernelGGL(ohem_scores_row<T>, dim3(grid), dim3(row_threads_for_sweep<T>(C)), 0, st, x, labels, scores, ce, P, C,
                               ignore_index, tables, row_chunks_ok<T>(x, nullptr, C), none);
        } else {
            hipLaunchKernelGGL(ohem_scores_lane<T>, dim3(group_grid(P, 256)), dim3(256), 0, st, x, labels, scores, ce, P,
                               m_size, C, ignore_index, tables, none);
        }
    });
    return check_launch();
}

// The score kernels that leave the threshold rule's sums give a block 256 pixels or more (a multiple of 64 slots keeps
// the three arrays 256-byte aligned).
static int64_t early_blocks_max(int64_t P) { return ceil_div(ceil_div(P > 0 ? P : 1, kRegsBlock), 64) * 64; }

static int64_t select_workspace(int64_t P) {
    return align256(kOhemZeroWords * 4) + align256((ohem_tiles(P) + kTieRuns) * 4);
}

// The tables are needed unless the labels pass through unchanged (n_min >= P).
static int check_workspace(const void *workspace, int64_t workspace_bytes, int64_t P, int64_t n_min) {
    if (n_min >= P) return PLH_OK;
    if (!workspace || misaligned(workspace, 256) || workspace_bytes < select_workspace(P)) return PLH_ERR_WORKSPACE;
    return PLH_OK;
}

static int launch_select(const float *scores, const int64_t *labels, int64_t *out_labels, void *workspace,
                         int64_t P, int64_t ignore_index, float score_thresh, int64_t n_min, hipStream_t st,
                         const float *ce = nullptr, Partials part = Partials{nullptr, nullptr},
                         bool tables_zeroed = false, uint8_t *kept_out = nullptr, const int *below = nullptr,
                         unsigned below_blocks = 0) {
    if (n_min >= P && part.sum) {                // nothing is relabelled, the loss is still wanted
        n_min = 0;
        score_thresh = INFINITY;
    }
    if (n_min >= P) {                            // csrc/ohem_label_kernel.cu:189: labels are returned as they are
        if (out_labels != labels)
            hipLaunchKernelGGL(ohem_copy_labels, dim3((unsigned)(ceil_div(P, 256) < 4096 ? ceil_div(P, 256) : 4096)),
                               dim3(256), 0, st, labels, out_labels, P);
        return check_launch();
    }
    const int64_t tiles = ohem_tiles(P);
    OhemTables tb;
    tb.hist = static_cast<uint32_t *>(workspace);
    tb.state = tb.hist + 3 * kOhemBins;
    tb.tile_ties = reinterpret_cast<uint32_t *>(static_cast<char *>(workspace) + align256(kOhemZeroWords * 4));
    const uint32_t k = n_min > 0 ? (uint32_t)n_min : 0u;
    const int Pi = (int)P;
    // 16-byte accesses when every tensor allows them (tile bases are multiples of 4 pixels)
    const int vec = !misaligned(scores, 16) && (kept_out || (!misaligned(labels, 16) && !misaligned(out_labels, 16)));
    if (k > 0) {
        if (!tables_zeroed)     // the score kernel of the one-call entry points has done it
            hipLaunchKernelGGL(ohem_zero, dim3((kOhemZeroWords + 255) / 256), dim3(256), 0, st, tb.hist, kOhemZeroWords);
        // every block ends with one global atomic per non-empty bin, all blocks on the same few hundred
        // addresses: 512 blocks (two per compute unit) measured 30 us faster than 2048 on 8 M scores
        const unsigned hgrid = (unsigned)(ceil_div(P, 256 * 16) < 512 ? ceil_div(P, 256 * 16) : 512);
        for (int pass = 0; pass < 3; ++pass)
            hipLaunchKernelGGL(ohem_hist, dim3(hgrid), dim3(256), 0, st, scores, tb, Pi, pass, k, score_thresh, vec,
                               pass == 0 ? below : nullptr, below_blocks);
        hipLaunchKernelGGL(ohem_ties, dim3(kTieRuns / 4), dim3(256), 0, st, scores, tb, Pi, (int)tiles, k, score_thresh, vec);
    }
    hipLaunchKernelGGL(ohem_relabel, dim3((unsigned)tiles), dim3(256), 0, st, scores, labels, out_labels, tb, Pi, (int)tiles, k,
                       score_thresh, ignore_index, vec, ce, part, kept_out);
    return check_launch();
}

}  // namespace plh

using namespace plh;

extern "C" int64_t plh_ohem_workspace_bytes(int64_t n_pixels) {
    if (n_pixels < 0 || n_pixels > kOhemMaxPixels) return PLH_ERR_BAD_SIZE;
    return select_workspace(n_pixels);
}

extern "C" int plh_ohem_scores(const void *logits, int32_t dtype, const int64_t *labels, float *scores,
                               int64_t n_size, int64_t dimsize, int64_t m_size, int64_t ignore_index, void *stream) {
    if (!dtype_ok(dtype)) return PLH_ERR_BAD_DTYPE;
    const int rc = check_slice_args(logits, labels, scores, n_size, dimsize, m_size, dtype_size(dtype), 4);
    if (rc != PLH_OK) return rc;
    if (n_size * dimsize * m_size == 0) return PLH_OK;
    return launch_scores(logits, dtype, labels, scores, nullptr, n_size, dimsize, m_size, ignore_index,
                         (hipStream_t)stream);
}

extern "C" int plh_ohem_select_labels(const float *scores, const int64_t *labels, int64_t *out_labels,
                                      void *workspace, int64_t workspace_bytes, int64_t n_pixels,
                                      int64_t ignore_index, float score_thresh, int64_t n_min, void *stream) {
    if (n_pixels < 0 || n_pixels > kOhemMaxPixels) return PLH_ERR_BAD_SIZE;
    if (n_pixels == 0) return PLH_OK;
    if (!scores || !labels || !out_labels) return PLH_ERR_NULL_POINTER;
    if (misaligned(scores, 4) || misaligned(labels, 8) || misaligned(out_labels, 8)) return PLH_ERR_MISALIGNED;
    const int rc = check_workspace(workspace, workspace_bytes, n_pixels, n_min);
    if (rc != PLH_OK) return rc;
    return launch_select(scores, labels, out_labels, workspace, n_pixels, ignore_index, score_thresh, n_min,
                         (hipStream_t)stream);
}

extern "C" int plh_ohem_score_label(const void *logits, int32_t dtype, const int64_t *labels, int64_t *out_labels,
                                    float *scores, void *workspace, int64_t workspace_bytes,
                                    int64_t n_size, int64_t dimsize, int64_t m_size, int64_t ignore_index,
                                    float score_thresh, int64_t n_min, void *stream) {
    if (!dtype_ok(dtype)) return PLH_ERR_BAD_DTYPE;
    int rc = check_slice_args(logits, labels, out_labels, n_size, dimsize, m_size, dtype_size(dtype), 8);
    if (rc != PLH_OK) return rc;
    if (n_size * m_size > kOhemMaxPixels) return PLH_ERR_BAD_SIZE;
    if (n_size * dimsize * m_size == 0) return PLH_OK;
    const int64_t P = n_size * m_size;
    rc = check_workspace(workspace, workspace_bytes, P, n_min);
    if (rc != PLH_OK) return rc;
    if (n_min < P) {
        if (!scores) return PLH_ERR_NULL_POINTER;
        if (misaligned(scores, 4)) return PLH_ERR_MISALIGNED;
        rc = launch_scores(logits, dtype, labels, scores, nullptr, n_size, dimsize, m_size, ignore_index,
                           (hipStream_t)stream, static_cast<uint32_t *>(workspace));
        if (rc != PLH_OK) return rc;
    }
    return launch_select(scores, labels, out_labels, workspace, P, ignore_index, score_thresh, n_min,
                         (hipStream_t)stream, nullptr, Partials{nullptr, nullptr}, n_min < P);
}

extern "C" int64_t plh_ohem_ce_workspace_bytes(int64_t n_pixels) {
    if (n_pixels < 0 || n_pixels > kOhemMaxPixels) return PLH_ERR_BAD_SIZE;
    // the selection's tables, the relabelling pass's partial sums (8 bytes per tile), the score kernel's (12 bytes per block)
    return select_workspace(n_pixels) + align256(8 * ohem_tiles(n_pixels)) + align256(12 * early_blocks_max(n_pixels));
}

// The one-call forwards: scores and per-pixel loss in one pass over the logits (cross entropy: the
// score kernel itself; large margin: that loss's forward kernel, which then also leaves the scores),
// relabelling that adds up the kept pixels' losses, fixed-order finish.
// With `kept` (and no out_labels) the selection leaves the byte mask that plh_lsr_backward_kept and
// plh_lmargin_backward_kept read, instead of relabelled labels: the relabelling pass then neither reads the
// labels nor writes new ones.
static int ohem_loss_forward(bool large_margin, float lam, const void *logits, int32_t dtype, const int64_t *labels,
                             int64_t *out_labels, float *scores, float *pixel_loss, float *loss_out,
                             int64_t *n_valid_out, void *workspace, int64_t workspace_bytes, int64_t n_size,
                             int64_t dimsize, int64_t m_size, int64_t ignore_index, float score_thresh, int64_t n_min,
                             void *stream, uint8_t *kept = nullptr) {
    if (!dtype_ok(dtype)) return PLH_ERR_BAD_DTYPE;
    int rc = kept ? check_slice_args(logits, labels, kept, n_size, dimsize, m_size, dtype_size(dtype), 4)
                  : check_slice_args(logits, labels, out_labels, n_size, dimsize, m_size, dtype_size(dtype), 8);
    if (rc != PLH_OK) return rc;
    if (n_size * m_size > kOhemMaxPixels) return PLH_ERR_BAD_SIZE;
    if (!loss_out) return PLH_ERR_NULL_POINTER;
    if (misaligned(loss_out, 4) || misaligned(n_valid_out, 8)) return PLH_ERR_MISALIGNED;
    const int64_t P = n_size * m_size;
    hipStream_t st = (hipStream_t)stream;
    if (n_size * dimsize * m_size == 0) {        // the mean over no pixels, as the other reduced entry points give it
        finish_partials(Partials{nullptr, nullptr}, 0, loss_out, n_valid_out, kFinishMeanOverCount, 0, st);
        return check_launch();
    }
    if (!scores || !pixel_loss) return PLH_ERR_NULL_POINTER;
    if (misaligned(scores, 4) || misaligned(pixel_loss, 4)) return PLH_ERR_MISALIGNED;
    if (!workspace || misaligned(workspace, 256) || workspace_bytes < plh_ohem_ce_workspace_bytes(P))
        return PLH_ERR_WORKSPACE;
    const int64_t tiles = ohem_tiles(P);
    Partials part;
    part.sum = reinterpret_cast<float *>(static_cast<char *>(workspace) + select_workspace(P));
    part.cnt = reinterpret_cast<int *>(part.sum + tiles);
    const float none = kept ? kNoTargetMark : 1.f;
    if (n_min >= P) {                            // nothing is dropped (launch_select says the same), the loss is still wanted
        n_min = 0;
        score_thresh = INFINITY;
    }
    // with the byte mask the score pass also leaves what the threshold rule gives (OhemEarly)
    OhemEarly ev{nullptr, nullptr, nullptr, nullptr, score_thresh};
    unsigned early_blocks = 0;
    if (kept) {
        const int64_t slots = early_blocks_max(P);
        ev.kept = kept;
        ev.sum = reinterpret_cast<float *>(static_cast<char *>(workspace) + select_workspace(P) + align256(8 * tiles));
        ev.cnt = reinterpret_cast<int *>(ev.sum + slots);
        ev.below = ev.cnt + slots;
    }
    if (large_margin)
        rc = lmargin_forward_with_scores(logits, dtype, labels, pixel_loss, scores, n_size, dimsize, m_size, ignore_index,
                                         lam, st, none, &ev, &early_blocks);
    else
        rc = launch_scores(logits, dtype, labels, scores, pixel_loss, n_size, dimsize, m_size, ignore_index, st,
                           static_cast<uint32_t *>(workspace), none, &ev, &early_blocks);
    if (rc != PLH_OK) return rc;
    if (early_blocks && n_min <= 0) {            // no position lies below n_min: the threshold rule is the selection
        finish_partials(Partials{ev.sum, ev.cnt}, early_blocks, loss_out, n_valid_out, kFinishMeanOverCount, 0, st);
        return check_launch();
    }
    rc = launch_select(scores, labels, out_labels, workspace, P, ignore_index, score_thresh, n_min, st, pixel_loss, part,
                       /*tables_zeroed=*/!large_margin, kept, early_blocks ? ev.below : nullptr, early_blocks);
    if (rc != PLH_OK) return rc;
    if (early_blocks)
        hipLaunchKernelGGL(ohem_finish, dim3(1), dim3(1024), 0, st,
                           static_cast<const uint32_t *>(workspace) + 3 * kOhemBins, Partials{ev.sum, ev.cnt}, early_blocks,
                           part, (unsigned)tiles, loss_out, n_valid_out);
    else
        finish_partials(part, (unsigned)tiles, loss_out, n_valid_out, kFinishMeanOverCount, 0, st);
    return check_launch();
}

extern "C" int plh_ohem_ce_forward(const void *logits, int32_t dtype, const int64_t *labels, int64_t *out_labels,
                                   float *scores, float *pixel_ce, float *loss_out, int64_t *n_valid_out,
                                   void *workspace, int64_t workspace_bytes,
                                   int64_t n_size, int64_t dimsize, int64_t m_size, int64_t ignore_index,
                                   float score_thresh, int64_t n_min, void *stream) {
    return ohem_loss_forward(false, 0.f, logits, dtype, labels, out_labels, scores, pixel_ce, loss_out, n_valid_out,
                             workspace, workspace_bytes, n_size, dimsize, m_size, ignore_index, score_thresh, n_min, stream);
}

extern "C" int plh_ohem_lmargin_forward(const void *logits, int32_t dtype, const int64_t *labels, int64_t *out_labels,
                                        float *scores, float *pixel_loss, float *loss_out, int64_t *n_valid_out,
                                        void *workspace, int64_t workspace_bytes,
                                        int64_t n_size, int64_t dimsize, int64_t m_size, int64_t ignore_index,
                                        float lam, float score_thresh, int64_t n_min, void *stream) {
    return ohem_loss_forward(true, lam, logits, dtype, labels, out_labels, scores, pixel_loss, loss_out, n_valid_out,
                             workspace, workspace_bytes, n_size, dimsize, m_size, ignore_index, score_thresh, n_min, stream);
}

extern "C" int plh_ohem_ce_forward_kept(const void *logits, int32_t dtype, const int64_t *labels, uint8_t *kept,
                                        float *scores, float *pixel_ce, float *loss_out, int64_t *n_valid_out,
                                        void *workspace, int64_t workspace_bytes,
                                        int64_t n_size, int64_t dimsize, int64_t m_size, int64_t ignore_index,
                                        float score_thresh, int64_t n_min, void *stream) {
    if (!kept && n_size * dimsize * m_size != 0) return PLH_ERR_NULL_POINTER;
    return ohem_loss_forward(false, 0.f, logits, dtype, labels, nullptr, scores, pixel_ce, loss_out, n_valid_out,
                             workspace, workspace_bytes, n_size, dimsize, m_size, ignore_index, score_thresh, n_min, stream,
                             kept);
}

extern "C" int plh_ohem_lmargin_forward_kept(const void *logits, int32_t dtype, const int64_t *labels, uint8_t *kept,
                                             float *scores, float *pixel_loss, float *loss_out, int64_t *n_valid_out,
                                             void *workspace, int64_t workspace_bytes,
                                             int64_t n_size, int64_t dimsize, int64_t m_size, int64_t ignore_index,
                                             float lam, float score_thresh, int64_t n_min, void *stream) {
    if (!kept && n_size * dimsize * m_size != 0) return PLH_ERR_NULL_POINTER;
    return ohem_loss_forward(true, lam, logits, dtype, labels, nullptr, scores, pixel_loss, loss_out, n_valid_out,
                             workspace, workspace_bytes, n_size, dimsize, m_size, ignore_index, score_thresh, n_min, stream,
                             kept);
}
