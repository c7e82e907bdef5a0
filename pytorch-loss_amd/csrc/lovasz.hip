// Lovasz-softmax forward and backward for gfx950.
//
// Per class c over all P = n_size*m_size pixels (csrc/lovasz_softmax.cu:71-152,182-239):
//   e_i   = |1[y_i = c] - softmax(x_i)_c|                   ignored pixels take no part
//   sort e descending; cs_k = number of positives among the first k+1
//   J_k   = 1 - (n_pos - cs_k) / (n_pos - cs_k + k + 1),    dJ_k = J_k - J_{k-1}  (dJ_0 = J_0)
//   loss_c = sum_k e_(k) * dJ_k ;  jacc[c, pixel] = dJ of that pixel (0 when ignored)
// Backward (csrc/lovasz_softmax.cu:242-278,379-417):
//   d_ic = (c == y_i ? -1 : +1) * jacc[c,i] * grad_out[c];  g_ic = p_ic * (d_ic - sum_k p_ik d_ik)
//
// Pipeline (all launches on the caller's stream, nothing allocated here):
//   1. keys           one pass over the logits: softmax in registers, one 32-bit key per
//                     (class, pixel):  bit 31 = positive flag, bits 0..30 = 0x3F800000 - bits(e)
//                     (ascending key order = descending error; e lies in [0,1] so its bit
//                     pattern is monotone), ignored pixel = 0x7FFFFFFF (sorts last). Also the
//                     largest positive key per class (per-block table + lov_class_max): keys
//                     beyond it have dJ = 0 exactly and are left out of the sort (keep_key).
//   2. 3 x (tile_hist, row_scan, scatter): stable LSD radix passes, 8 bits each, batched over
//                     classes with blockIdx.y. Ranking inside a tile is done per wavefront with
//                     ballot-built match masks, tiles are re-ordered in LDS so that the global
//                     writes are runs of consecutive addresses. The positive flag rides along in
//                     bit 31; the payload (pixel index) is generated from the position in the
//                     first pass, which also drops the keys that take no part and counts the rest.
//   3. tile_hist<hot>, row_scan, final: the last (top-digit) pass is not written out: a key's
//                     destination is its rank k, the positives counted the same way give cs_k,
//                     so J, dJ and the tile's share of the loss follow at once; dJ goes to
//                     pixel order through region-binned staging (final) and an in-LDS permute
//                     per region (unbin), which also writes the zeros of the keys left out.
//   4. loss per class fixed-order sum of the per-tile partials (no floating-point atomics, so
//                     results are deterministic): by the first unbin block of the class, or by
//                     reduce_loss when the rows are too long for the staging regions.
// A 4096-key tile is handled by 512 threads with 8 keys each; neighbouring tiles of a class row run
// on the same XCD (sort_tile) so that the sectors they share merge in one L2.
// Equal errors keep pixel order (the sort is stable); the reference leaves tie order open.
#include "plh_common.hpp"

namespace plh {

constexpr uint32_t kOne = 0x3F800000u;          // bits of 1.0f
constexpr uint32_t kIgnoredKey = 0x7FFFFFFFu;
constexpr uint32_t kHotBit = 0x80000000u;

constexpr int kSortThreads = 512;
constexpr int kSortItems = 8;
constexpr int kSortTile = kSortThreads * kSortItems;   // 4096 keys per block
constexpr int kSortWaves = kSortThreads / kWave;
constexpr int kRadixBits = 8;                    // widest digit of a pass
constexpr int kRadix = 1 << kRadixBits;          // bins per (class, tile) table row set
constexpr int kRankGroup = 2;     // rounds whose match masks are formed together (see lov_scatter)

__device__ __forceinline__ uint32_t make_key(float prob, bool hot, bool ignored) {
    const float err = hot ? fabsf(1.f - prob) : fabsf(prob);
    const uint32_t bits = __builtin_bit_cast(uint32_t, err);
    const uint32_t key = (kOne - (bits > kOne ? kOne : bits)) | (hot ? kHotBit : 0u);
    return ignored ? kIgnoredKey : key;
}

__device__ __forceinline__ float key_error(uint32_t key) {
    return __builtin_bit_cast(float, kOne - (key & 0x7FFFFFFFu));
}

// ------------------------------------------------------ 1. build keys ----

// Besides the keys, both kernels leave per block and class the largest key among the block's
// positives of that class, plus 1 (0 = none), in block_table[block][C]; lov_class_max folds the
// table into pos_max[c], the error of the class's lowest-ranked positive. Everything sorted after
// that one has a Jaccard difference of exactly 0 (see keep_key), so the sort never sees it.
__device__ __forceinline__ void publish_block_max(const uint32_t *block_max, uint32_t *block_table, int C) {
    uint32_t *row = block_table + (int64_t)blockIdx.x * C;
    for (int j = threadIdx.x; j < C; j += blockDim.x) row[j] = block_max[j];
}

// It also leaves, per class, the number of key bits the sort has to look at: keys that take part are
// not above the limit, so the bits above the limit's highest set bit are zero in every one of them.
__global__ __launch_bounds__(256) void lov_class_max(const uint32_t *__restrict__ block_table, int blocks, int C,
                                                     uint32_t *__restrict__ pos_max, uint32_t *__restrict__ cursors,
                                                     int regions) {
    __shared__ uint32_t wave_max[4];
    const int c = blockIdx.x;
    // the class's staging cursors start at zero (they are first used by the last pass)
    for (int i = threadIdx.x; i < regions; i += 256) cursors[(int64_t)c * regions + i] = 0;
    uint32_t m = 0;
    for (int b = threadIdx.x; b < blocks; b += 256) m = max(m, block_table[(int64_t)b * C + c]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = max(m, (uint32_t)__shfl_xor((int)m, off, 64));
    if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t top = max(max(wave_max[0], wave_max[1]), max(wave_max[2], wave_max[3]));
        pos_max[c] = top;
        pos_max[2 * C + c] = 0xFFFFFFFFu;       // all_min[c], for lov_absent_min
        // key_bits[c]: a class without positives keeps a single key value, wherever it lies
        pos_max[3 * C + c] = (top > 1u) ? (uint32_t)(32 - __builtin_clz(top - 1u)) : (top ? 1u : 30u);
    }
}

// A class without positives has J = 1 from the first sorted key on: only its largest error (smallest
// key) has a non-zero Jaccard difference. For such classes (blocks of the others return at once)
// this finds the smallest key of the row, which then serves as the class's limit.
constexpr int kAbsentBlocks = 64;
__global__ __launch_bounds__(256) void lov_absent_min(const uint32_t *__restrict__ keys, const uint32_t *pos_max,
                                                      uint32_t *all_min, int P) {
    __shared__ uint32_t wave_min[4];
    const int c = blockIdx.y;
    if (pos_max[c] != 0) return;                // block-uniform
    const uint32_t *row = keys + (int64_t)c * P;
    uint32_t m = 0xFFFFFFFFu;
    for (int i = blockIdx.x * 256 + threadIdx.x; i < P; i += kAbsentBlocks * 256) m = min(m, row[i] & 0x7FFFFFFFu);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = min(m, (uint32_t)__shfl_xor((int)m, off, 64));
    if ((threadIdx.x & 63) == 0) wave_min[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) atomicMin(all_min + c, min(min(wave_min[0], wave_min[1]), min(wave_min[2], wave_min[3])));
}

template <class T, int CP, int V>
__global__ __launch_bounds__(kRegsBlock) void lov_keys_regs(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                           uint32_t *__restrict__ keys, uint32_t *__restrict__ block_table,
                                                           int64_t P, int64_t m_size, int C,
                                                           int64_t ignore, unsigned xcd_run) {
    __shared__ uint32_t block_max[kMaxRegsChannels];
    if (threadIdx.x < kMaxRegsChannels) block_max[threadIdx.x] = 0;
    __syncthreads();
    const int64_t want = (tile_of_block(xcd_run) * kRegsBlock + threadIdx.x) * V;
    const bool live = want < P;
    const int64_t pix = live ? want : 0;
    const int64_t n = pix / m_size;
    const T *xs = x + (pix + n * (int64_t)(C - 1) * m_size);
    float v[CP][V];
#pragma unroll
    for (int j = 0; j < CP; ++j)
        if (chan_ok<CP>(j, C)) load_vec<V>(xs + (int64_t)j * m_size, v[j]);
    int64_t lb[V];
    load_labels<V>(lab + pix, lb);
#pragma unroll
    for (int k = 0; k < V; ++k) {
        float mx = v[0][k];
#pragma unroll
        for (int j = 1; j < CP; ++j)
            if (chan_ok<CP>(j, C)) mx = fmaxf(mx, v[j][k]);
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (chan_ok<CP>(j, C)) {
                v[j][k] = expf(v[j][k] - mx);
                s += v[j][k];
            }
        const bool ign = (lb[k] == ignore);
        uint32_t key_y = 0;                     // the positive's key, if the pixel has one
        bool has_y = false;
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (chan_ok<CP>(j, C)) {
                const bool hot = (lb[k] == j);
                const uint32_t key = make_key(v[j][k] / s, hot, ign);
                key_y = hot ? key : key_y;
                has_y = has_y || hot;
                v[j][k] = __builtin_bit_cast(float, key);
            }
        if (live && !ign && has_y) atomicMax(&block_max[(int)lb[k]], (key_y & 0x7FFFFFFFu) + 1u);
    }
    if (live) {
#pragma unroll
        for (int j = 0; j < CP; ++j)
            // cache-allocating stores: the radix passes read the keys next, partly out of the last-level cache
            if (chan_ok<CP>(j, C)) store_vec_cached<V>(reinterpret_cast<float *>(keys) + (int64_t)j * P + pix, v[j]);
    }
    __syncthreads();
    publish_block_max(block_max, block_table, C);
}

// Any channel count: a lane per pixel, three sweeps over the slice (the later ones hit cache).
template <class T>
__global__ __launch_bounds__(256) void lov_keys_lane(const T *__restrict__ x, const int64_t *__restrict__ lab,
                                                     uint32_t *__restrict__ keys, uint32_t *__restrict__ block_table,
                                                     int64_t P, int64_t m_size, int C, int64_t ignore) {
    __shared__ uint32_t block_max[512];              // C < 512
    for (int j = threadIdx.x; j < C; j += 256) block_max[j] = 0;
    __syncthreads();
    for (int64_t pix = (int64_t)blockIdx.x * 256 + threadIdx.x; pix < P; pix += (int64_t)gridDim.x * 256) {
        const int64_t n = pix / m_size;
        const T *xs = x + (pix + n * (int64_t)(C - 1) * m_size);
        const int64_t lb = lab[pix];
        float mx = -INFINITY;
#pragma unroll 8
        for (int j = 0; j < C; ++j) mx = fmaxf(mx, load_one(xs + (int64_t)j * m_size));
        float s = 0.f;
#pragma unroll 8
        for (int j = 0; j < C; ++j) s += expf(load_one(xs + (int64_t)j * m_size) - mx);
#pragma unroll 8
        for (int j = 0; j < C; ++j) {
            const uint32_t key = make_key(expf(load_one(xs + (int64_t)j * m_size) - mx) / s, lb == j, lb == ignore);
            keys[(int64_t)j * P + pix] = key;
            if (lb == j && lb != ignore) atomicMax(&block_max[j], (key & 0x7FFFFFFFu) + 1u);
        }
    }
    __syncthreads();
    publish_block_max(block_max, block_table, C);
}

// --------------------------------------------------- 2. radix sort pass ----

struct SortArgs {
    const uint32_t *keys_in;
    const uint32_t *vals_in;     // nullptr in the first pass: payload = position
    uint32_t *keys_out;
    uint32_t *vals_out;
    const uint32_t *keys_alt;    // last pass only: where the rows of classes with two scatter passes are
    const uint32_t *vals_alt;    //   (keys_alt, vals_alt); the others are in (keys_in, vals_in)
    uint32_t *tile_hist;         // [C][kRadix][tiles_pad]: keys per (digit, tile); row-scanned in place
    uint32_t *digit_total;       // [C][kRadix]: keys per digit
    uint32_t *tile_hot;          // last pass only: the same two tables for the positives
    uint32_t *hot_total;
    const uint32_t *pos_max;     // first pass only: per class, largest positive key + 1 (see keep_key)
    const uint32_t *all_min;     // first pass only: per class without positives, its smallest key
    const uint32_t *kept_in;     // later passes: keys per class that the first pass let through
    uint32_t *kept_out;          // first pass: where that count goes
    const uint32_t *key_bits;    // per class: key bits that the sort has to look at (see DigitPlan)
    int P;                       // row stride; keys per class row in the first pass
    int tiles;                   // ceil(P / kSortTile)
    int tiles_pad;               // tiles rounded up to a multiple of kSortWaves: row length of the tile tables
    int pass;                    // 0, 1, 2: scatter pass; the last (fused) pass of a class is passes - 1
    // decoupled look-back variant only (see lov_look_back): this pass's tile descriptors [C][tiles][kRadix] (64-bit
    // ones in the last pass), its per-class ticket counters and the word that a timed-out wait sets
    uint32_t *desc;
    unsigned long long *desc_wide;
    uint32_t *tickets;
    uint32_t *timed_out;
};

// The digits of a class. Keys that take part in a class's sort are below 2^bits (bits from the
// class's limit, lov_class_max), so the sort runs over `bits` bits only: in 2, 3 or 4 stable passes
// of at most kRadixBits bits each, the first passes - 1 of them scatter passes and the last one
// fused with the Jaccard step (16 bits or fewer, i.e. a best positive's error above 0.99: two
// passes; up to 24 bits, error above 0.008: three). The bits are shared out evenly: 27 bits (best
// error around 1e-4) are 7 + 7 + 7 + 6. Measured on the benchmark's rows, forward in us: 7+7+7+6
// 682, 7+8+8+4 684, 5+8+7+7 688, 8+8+8+6 (all 30 bits) 701, 9+9+9 735: a pass costs by the bit
// (a scatter pass 70 us at 7 bits, 79 at 8, 104 at 9: the runs a tile writes per digit halve with
// every bit), so what counts is the number of bits, not how they are cut.
struct DigitPlan {
    int passes, shift, width;
    uint32_t mask;
};
__device__ __forceinline__ DigitPlan digit_plan(uint32_t bits, int pass) {
    const int np = bits <= 2u * kRadixBits ? 2 : (bits <= 3u * kRadixBits ? 3 : 4);
    const int base = (int)bits / np, rem = (int)bits % np;       // the first `rem` passes take one bit more
    const int p = pass < 0 ? np - 1 : pass;
    const int width = base + (p < rem ? 1 : 0);
    return DigitPlan{np, p * base + min(p, rem), width, (1u << width) - 1u};
}
constexpr int kLastPass = -1;

// A key takes part in the sort iff its error is not below that of the class's lowest-ranked positive
// (error bits of the key <= limit). What is left out would be sorted after every positive, where
// the intersection is empty: J = 1 - 0/(k+1) = 1 on both sides of the difference, so its Jaccard
// difference is exactly 0 and it adds exactly 0 to the loss; lov_unbin writes those zeros. Ignored
// pixels (error bits 0x7FFFFFFF) are always left out. A class without positives has J = 1 from the
// first key on, so only its largest error counts: its limit is the smallest key of the row. Keys
// equal to the limit stay in, so ties with the last positive (or at the largest error) keep their
// pixel order.
__device__ __forceinline__ uint32_t keep_limit(const SortArgs &a, int c) {
    if (!a.pos_max) return 0x7FFFFFFFu;          // later passes: everything that is there takes part
    const uint32_t m = a.pos_max[c];
    if (m) return m - 1u;
    const uint32_t lowest = a.all_min[c];
    return lowest <= kOne ? lowest : kOne;       // no valid key at all: nothing passes anyway
}
__device__ __forceinline__ bool keep_key(uint32_t key, uint32_t limit) { return (key & 0x7FFFFFFFu) <= limit; }

// Keys of class c that enter this pass.
__device__ __forceinline__ int row_items(const SortArgs &a, int c) { return a.kept_in ? (int)a.kept_in[c] : a.P; }

// Tile of this block. Workgroups go to the 8 XCDs round-robin, each with an L2 of its own; taking
// the tiles of a class row in 8 contiguous chunks, one per XCD, puts neighbouring tiles behind the
// same L2, where what they share merges: the table words of consecutive tiles (4-byte stores into
// one sector) and the sectors in which one tile's run of a digit ends and the next tile's begins.
// Only the tiles that hold keys are permuted (the rest of a pruned row exits at once, and would
// leave the XCDs of the last chunks idle).
__device__ __forceinline__ int sort_tile(int items, int tile_keys = kSortTile) {
    const int x = blockIdx.x, q = ((items + tile_keys - 1) / tile_keys) >> 3;
    return x < 8 * q ? (x & 7) * q + (x >> 3) : x;
}

// Inclusive scan over the 64 lanes of a wave.
__device__ __forceinline__ uint32_t wave_incl_scan(uint32_t v) {
    const int lane = __lane_id();
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const uint32_t up = (uint32_t)__builtin_amdgcn_ds_bpermute(((lane - d) & 63) << 2, (int)v);
        if (lane >= d) v += up;
    }
    return v;
}

// Exclusive scan of one value per thread over the whole block (kSortThreads threads);
// `total` = block sum. lds must hold kSortWaves words. Contains barriers: every thread calls it.
__device__ __forceinline__ uint32_t block_excl_scan(uint32_t v, uint32_t *lds, uint32_t &total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t incl = wave_incl_scan(v);
    if (lane == 63) lds[wave] = incl;
    __syncthreads();
    uint32_t before = 0, all = 0;
#pragma unroll
    for (int w = 0; w < kSortWaves; ++w) {
        const uint32_t t = lds[w];
        before += (w < wave) ? t : 0u;
        all += t;
    }
    total = all;
    __syncthreads();
    return before + incl - v;
}

// Two independent exclusive scans behind one pair of barriers. lds must hold 2 * kSortWaves words.
__device__ __forceinline__ void block_excl_scan2(uint32_t a, uint32_t b, uint32_t *lds, uint32_t &excl_a,
                                                 uint32_t &total_a, uint32_t &excl_b, uint32_t &total_b) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t incl_a = wave_incl_scan(a), incl_b = wave_incl_scan(b);
    if (lane == 63) {
        lds[wave] = incl_a;
        lds[kSortWaves + wave] = incl_b;
    }
    __syncthreads();
    uint32_t before_a = 0, all_a = 0, before_b = 0, all_b = 0;
#pragma unroll
    for (int w = 0; w < kSortWaves; ++w) {
        const uint32_t ta = lds[w], tb = lds[kSortWaves + w];
        before_a += (w < wave) ? ta : 0u;
        before_b += (w < wave) ? tb : 0u;
        all_a += ta;
        all_b += tb;
    }
    total_a = all_a;
    total_b = all_b;
    excl_a = before_a + incl_a - a;
    excl_b = before_b + incl_b - b;
    __syncthreads();
}

// Match mask: the valid lanes of the wave whose digit equals this lane's. One ballot per digit bit;
// each lane ORs up, in two 32-bit halves, the lanes that differ from it in that bit
// (vote XOR own bit splatted), so a bit costs one field extract, one compare, two XORs and its share
// of two 3-input ORs.
// The same with a number of digit bits that is known at run time only (wave-uniform), for the last
// pass's histogram. (In lov_final the loop costs more than the ballots it leaves out: 138 us against 132.)
__device__ __forceinline__ uint64_t wave_peers_n(uint32_t digit, bool valid, int bits) {
    uint32_t diff_lo = 0, diff_hi = 0;
#pragma unroll 1
    for (int b = 0; b < bits; ++b) {
        uint32_t splat = 0u - ((digit >> b) & 1u);
        asm("" : "+v"(splat));
        const uint64_t vote = __builtin_amdgcn_ballot_w64(splat != 0u);
        diff_lo |= (uint32_t)vote ^ splat;
        diff_hi |= (uint32_t)(vote >> 32) ^ splat;
    }
    const uint64_t diff = ((uint64_t)diff_hi << 32) | diff_lo;
    return __builtin_amdgcn_ballot_w64(valid) & ~diff;
}

__device__ __forceinline__ uint64_t wave_peers(uint32_t digit, bool valid) {
    uint32_t diff_lo = 0, diff_hi = 0;
#pragma unroll
    for (int b = 0; b < kRadixBits; ++b) {
        uint32_t splat = (uint32_t)((int32_t)(digit << (31 - b)) >> 31);   // bit b splatted: 0 or ~0
        asm("" : "+v"(splat));      // the vote is taken from the splat itself: one field extract serves both
        const uint64_t vote = __builtin_amdgcn_ballot_w64(splat != 0u);
        diff_lo |= (uint32_t)vote ^ splat;
        diff_hi |= (uint32_t)(vote >> 32) ^ splat;
    }
    const uint64_t diff = ((uint64_t)diff_hi << 32) | diff_lo;
    return __builtin_amdgcn_ballot_w64(valid) & ~diff;
}

// Stable rank of this lane's key among the equal digits the wave has seen so far (earlier rounds
// through the wave's private counters, this round through the match mask). With Hot, the same for
// the positives only (hrank = positives with this digit before this key).
// Peers of this lane that sit in lower lanes: the masked bit count does the AND with "lanes below me"
// and the population count in two instructions.
__device__ __forceinline__ uint32_t peers_below(uint64_t peers) {
    return __builtin_amdgcn_mbcnt_hi((uint32_t)(peers >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)peers, 0u));
}

template <bool Hot>
__device__ __forceinline__ void wave_rank_of(uint64_t peers, uint32_t digit, bool valid, bool hot, uint16_t *counts,
                                             uint16_t *counts_hot, uint32_t &rank, uint32_t &hrank) {
    // Every lane of a group reads the group's counter (one LDS address: a broadcast), then the group's
    // first lane moves it on. LDS executes a wave's instructions in issue order, so the reads see the
    // value from before this round, and the next round's reads see the update.
    const uint32_t before = peers_below(peers);
    uint64_t hot_peers = 0;
    uint32_t hot_before = 0;
    if constexpr (Hot) {
        hot_peers = peers & __builtin_amdgcn_ballot_w64(hot && valid);
        hot_before = peers_below(hot_peers);
    }
    uint32_t seen = 0, seen_hot = 0;
    if (valid) {
        seen = counts[digit];
        if constexpr (Hot) seen_hot = counts_hot[digit];
    }
    __builtin_amdgcn_wave_barrier();
    if (valid && before == 0u) {
        counts[digit] = (uint16_t)(seen + __builtin_popcountll(peers));
        if constexpr (Hot) counts_hot[digit] = (uint16_t)(seen_hot + __builtin_popcountll(hot_peers));
    }
    __builtin_amdgcn_wave_barrier();
    rank = seen + before;
    if constexpr (Hot) hrank = seen_hot + hot_before;
}

template <bool Hot>
__device__ __forceinline__ void wave_rank(uint32_t digit, bool valid, bool hot, uint16_t *counts,
                                          uint16_t *counts_hot, uint32_t &rank, uint32_t &hrank) {
    wave_rank_of<Hot>(wave_peers(digit, valid), digit, valid, hot, counts, counts_hot, rank, hrank);
}

// Where the rows of class c are when its last pass starts: after an odd number of scatter passes in
// (keys_in, vals_in), after two in (keys_alt, vals_alt); the other value buffer is free for staging.
struct LastPassRows {
    const uint32_t *keys, *vals;
    uint32_t *stage;
};
__device__ __forceinline__ LastPassRows last_pass_rows(const SortArgs &a, int passes) {
    const bool alt = (passes - 1) == 2;
    return LastPassRows{alt ? a.keys_alt : a.keys_in, alt ? a.vals_alt : a.vals_in,
                        const_cast<uint32_t *>(alt ? a.vals_in : a.vals_alt)};
}

// Per-tile digit counts (and, for the last pass, the same for the positives): a block per tile,
// per-wave tables, all loads up front. The lower digits are spread evenly: LDS atomics per lane, and
// a round whose keys all share one digit (a row of equal keys) is added by a single lane. The top
// digit clusters (a handful of values per round with soft predictions, dozens of binades with
// confident ones), so per-lane atomics would queue on a few addresses: the lowest lane of every
// group of equal digits, found through the match mask, adds the group.
template <bool Top>
__global__ __launch_bounds__(kSortThreads) void lov_tile_hist(const SortArgs a) {
    // A block counts two neighbouring tiles, the first with its wavefronts 0..3 and the second with 4..7: twice
    // the loads in flight per block and half the blocks (a block of one tile spends most of its life waiting
    // for its 8 loads per lane), and the two table words of a digit leave in one 8-byte store.
    constexpr int kPair = 2, kItems = kPair * kSortItems, kWavesPerTile = kSortWaves / kPair;
    __shared__ uint32_t counts[kSortWaves][kRadix];
    __shared__ uint32_t counts_hot[Top ? kSortWaves : 1][kRadix];
    const int c = blockIdx.y, pair = sort_tile(row_items(a, c), kPair * kSortTile);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const DigitPlan dp = digit_plan(a.key_bits[c], Top ? kLastPass : a.pass);
    if (!Top && a.pass >= dp.passes - 1) return;        // block-uniform: this class has fewer scatter passes
    const int begin = pair * (kPair * kSortTile);
    const int count = min(kPair * kSortTile, row_items(a, c) - begin);
    const int64_t cell = ((int64_t)c * kRadix + threadIdx.x) * a.tiles_pad + kPair * pair;
    const bool in_table = kPair * pair < a.tiles_pad;   // the grid covers the padded row in pairs: it may end one pair late
    if (count <= 0) {                           // block-uniform: the row ends before these tiles; lov_row_scan
        if (threadIdx.x <= dp.mask && in_table) {       // reads the live tiles in whole groups of kSortWaves
            *reinterpret_cast<uint2 *>(a.tile_hist + cell) = make_uint2(0u, 0u);
            if constexpr (Top) *reinterpret_cast<uint2 *>(a.tile_hot + cell) = make_uint2(0u, 0u);
        }
        return;
    }
    for (int i = threadIdx.x; i < kSortWaves * kRadix; i += kSortThreads) {
        (&counts[0][0])[i] = 0;
        if constexpr (Top) (&counts_hot[0][0])[i] = 0;
    }
    const uint32_t limit = keep_limit(a, c);
    const uint32_t *rows = Top ? last_pass_rows(a, dp.passes).keys : a.keys_in;
    const uint32_t *kin = rows + (int64_t)c * a.P + begin;
    uint32_t key[kItems];
#pragma unroll
    for (int r = 0; r < kItems; ++r) {          // all loads in flight before the first one is used
        const int li = wave * (kItems * kWave) + r * kWave + lane;
        key[r] = (li < count) ? kin[li] : kIgnoredKey;
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kItems; ++r) {
        const int li = wave * (kItems * kWave) + r * kWave + lane;
        const bool valid = li < count && keep_key(key[r], limit);
        const uint32_t digit = (key[r] >> dp.shift) & dp.mask;
        const uint64_t vmask = __builtin_amdgcn_ballot_w64(valid);
        if (vmask == 0) continue;               // wave-uniform
        if constexpr (Top) {
            const uint64_t peers = wave_peers_n(digit, valid, dp.width);
            const uint64_t hot_peers = peers & __builtin_amdgcn_ballot_w64(valid && (key[r] >> 31));
            if (valid && peers_below(peers) == 0u) {
                atomicAdd(&counts[wave][digit], (uint32_t)__builtin_popcountll(peers));
                if (hot_peers) atomicAdd(&counts_hot[wave][digit], (uint32_t)__builtin_popcountll(hot_peers));
            }
            continue;
        }
        const uint32_t value = (uint32_t)__builtin_amdgcn_readlane((int)digit, __builtin_ctzll(vmask));
        if (__builtin_amdgcn_ballot_w64(valid && digit == value) == vmask) {        // wave-uniform
            if (lane == 0) atomicAdd(&counts[wave][value], (uint32_t)__builtin_popcountll(vmask));
        } else if (valid) {
            atomicAdd(&counts[wave][digit], 1u);
        }
    }
    __syncthreads();
    if (threadIdx.x <= dp.mask) {
        const int d = threadIdx.x;
        uint32_t n[kPair] = {0, 0}, nh[kPair] = {0, 0};
#pragma unroll
        for (int w = 0; w < kSortWaves; ++w) {
            n[w / kWavesPerTile] += counts[w][d];
            if constexpr (Top) nh[w / kWavesPerTile] += counts_hot[w][d];
        }
        *reinterpret_cast<uint2 *>(a.tile_hist + cell) = make_uint2(n[0], n[1]);
        if constexpr (Top) *reinterpret_cast<uint2 *>(a.tile_hot + cell) = make_uint2(nh[0], nh[1]);
    }
}

// One block per (digit, class) row of a tile table: exclusive scan over the row's live tiles in
// place, row total to totals[c][d]. blockIdx.z selects the table (keys / positives). pass as in
// SortArgs (kLastPass for the fused pass); kept = nullptr in the first pass (every tile is live).
__global__ __launch_bounds__(256) void lov_row_scan(uint32_t *table0, uint32_t *totals0, uint32_t *table1,
                                                    uint32_t *totals1, int tiles_pad, const uint32_t *key_bits, int pass,
                                                    const uint32_t *kept, int P) {
    __shared__ uint32_t wave_tot[4];
    uint32_t *table = blockIdx.z ? table1 : table0;
    uint32_t *totals = blockIdx.z ? totals1 : totals0;
    const int c = blockIdx.y;
    const DigitPlan dp = digit_plan(key_bits[c], pass);
    if (pass >= 0 && pass >= dp.passes - 1) return;
    const int64_t rid = (int64_t)c * kRadix + blockIdx.x;
    if (blockIdx.x > dp.mask) {                     // no key has this digit; the tile table has no row for it
        if (threadIdx.x == 0) totals[rid] = 0;
        return;
    }
    const int items = kept ? (int)kept[c] : P;
    const int tiles = ((items + kSortTile - 1) / kSortTile + kSortWaves - 1) / kSortWaves * kSortWaves;
    uint32_t *row = table + rid * tiles_pad;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t carry = 0;
    for (int base = 0; base < tiles; base += 256) {
        const int i = base + threadIdx.x;
        const uint32_t v = (i < tiles) ? row[i] : 0u;
        const uint32_t incl = wave_incl_scan(v);
        if (lane == 63) wave_tot[wave] = incl;
        __syncthreads();
        uint32_t before = 0, all = 0;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            before += (w < wave) ? wave_tot[w] : 0u;
            all += wave_tot[w];
        }
        if (i < tiles) row[i] = carry + before + incl - v;
        carry += all;
        __syncthreads();
    }
    if (threadIdx.x == 0) totals[rid] = carry;
}

// ---- the decoupled look-back variant of the passes (plh_lovasz_forward_lookback) ------------------------
// Instead of a histogram kernel and a row scan in front of every pass, a tile learns how many keys of each digit
// the tiles before it hold by walking back over their descriptors: every tile publishes, per digit, first its own
// count ("aggregate") and, once it knows the sum over all its predecessors, the inclusive sum ("prefix"); a walk
// adds aggregates until it meets a prefix. The count travels in the same word as the state, so plain device-scope
// atomic loads and stores carry it (no fence). Tiles are handed out by a ticket counter per class, in the order
// in which blocks start, so every predecessor of a waiting block is resident and gets to publish: the waits end.
// They are bounded all the same; a wait that runs out sets `timed_out`, which turns the class losses into NaN.
// The digit totals of all passes come from one pass over the keys up front (lov_hist_all, lov_hist_reduce).
constexpr uint32_t kDescAggregate = 1u << 30, kDescPrefix = 2u << 30, kDescValue = (1u << 30) - 1u;
constexpr int kLookBackSpins = 1 << 22;

__device__ __forceinline__ uint32_t lov_look_back(uint32_t *desc_row, int tile, int d, uint32_t mine, uint32_t *timed_out) {
    uint32_t *me = desc_row + (int64_t)tile * kRadix + d;
    __hip_atomic_store(me, kDescAggregate | mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    uint32_t before = 0;
    for (int t = tile - 1; t >= 0; --t) {
        const uint32_t *at = desc_row + (int64_t)t * kRadix + d;
        uint32_t v = 0;
        for (int spin = 0; spin < kLookBackSpins; ++spin) {
            v = __hip_atomic_load(at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (v >> 30) break;
        }
        if ((v >> 30) == 0) {
            *timed_out = 1u;
            break;
        }
        before += v & kDescValue;
        if ((v >> 30) == 2u) break;
    }
    __hip_atomic_store(me, kDescPrefix | (before + mine), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return before;
}

// The same for two counts at once (keys and positives of the last pass): state in bits 62-63, positives in
// bits 31-61, keys in bits 0-30.
constexpr unsigned long long kWideAggregate = 1ull << 62, kWidePrefix = 2ull << 62, kWideField = (1ull << 31) - 1ull;
__device__ __forceinline__ void lov_look_back2(unsigned long long *desc_row, int tile, int d, uint32_t mine, uint32_t mine_hot,
                                               uint32_t &before, uint32_t &before_hot, uint32_t *timed_out) {
    unsigned long long *me = desc_row + (int64_t)tile * kRadix + d;
    __hip_atomic_store(me, kWideAggregate | ((unsigned long long)mine_hot << 31) | mine, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
    unsigned long long sum = 0;         // both fields at once: neither can carry into the other (counts stay below 2^31)
    for (int t = tile - 1; t >= 0; --t) {
        const unsigned long long *at = desc_row + (int64_t)t * kRadix + d;
        unsigned long long v = 0;
        for (int spin = 0; spin < kLookBackSpins; ++spin) {
            v = __hip_atomic_load(at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (v >> 62) break;
        }
        if ((v >> 62) == 0) {
            *timed_out = 1u;
            break;
        }
        sum += v & ((1ull << 62) - 1ull);
        if ((v >> 62) == 2ull) break;
    }
    before = (uint32_t)(sum & kWideField);
    before_hot = (uint32_t)((sum >> 31) & kWideField);
    __hip_atomic_store(me, kWidePrefix | ((unsigned long long)(before_hot + mine_hot) << 31) | (before + mine),
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The tile of a block in the look-back variant: the next ticket of its class.
__device__ __forceinline__ int lov_take_ticket(uint32_t *tickets, int c) {
    __shared__ int ticket;
    if (threadIdx.x == 0) ticket = (int)atomicAdd(&tickets[c], 1u);
    __syncthreads();
    return ticket;
}

// Digit counts of every pass of a class in one sweep over its keys: a block per two tiles, tables per pass in LDS,
// one table set per block in `partial` [C][blocks][kHistTables][kRadix]; slot p < 3 = scatter pass p, slot 3 = the
// class's last pass, slot 4 = the positives of the last pass.
constexpr int kHistTables = 5;
__global__ __launch_bounds__(kSortThreads) void lov_hist_all(const SortArgs a, uint32_t *__restrict__ partial, int blocks) {
    __shared__ uint32_t counts[kHistTables][kRadix];
    const int c = blockIdx.y;
    for (int i = threadIdx.x; i < kHistTables * kRadix; i += kSortThreads) (&counts[0][0])[i] = 0;
    __syncthreads();
    const uint32_t bits = a.key_bits[c];
    const int np = digit_plan(bits, 0).passes;
    const uint32_t limit = keep_limit(a, c);
    const int begin = blockIdx.x * (2 * kSortTile);
    const uint32_t *kin = a.keys_in + (int64_t)c * a.P;
    for (int i = begin + threadIdx.x; i < min(a.P, begin + 2 * kSortTile); i += kSortThreads) {
        const uint32_t key = kin[i];
        if (!keep_key(key, limit)) continue;
        for (int p = 0; p < np; ++p) {
            const DigitPlan dp = digit_plan(bits, p);
            const uint32_t digit = (key >> dp.shift) & dp.mask;
            const int slot = (p == np - 1) ? 3 : p;
            atomicAdd(&counts[slot][digit], 1u);
            if (p == np - 1 && (key >> 31)) atomicAdd(&counts[4][digit], 1u);
        }
    }
    __syncthreads();
    uint32_t *out = partial + ((int64_t)c * blocks + blockIdx.x) * (kHistTables * kRadix);
    for (int i = threadIdx.x; i < kHistTables * kRadix; i += kSortThreads) out[i] = (&counts[0][0])[i];
}

// totals[slot][C][kRadix] = sum over the blocks' tables.
__global__ __launch_bounds__(kRadix) void lov_hist_reduce(const uint32_t *__restrict__ partial, int blocks, int C,
                                                          uint32_t *__restrict__ totals) {
    const int c = blockIdx.y, slot = blockIdx.x, d = threadIdx.x;
    uint32_t sum = 0;
    for (int b = 0; b < blocks; ++b) sum += partial[(((int64_t)c * blocks + b) * kHistTables + slot) * kRadix + d];
    totals[((int64_t)slot * C + c) * kRadix + d] = sum;
}

template <bool LookBack>
__global__ __launch_bounds__(kSortThreads) void lov_scatter(const SortArgs a) {
    __shared__ uint32_t s_keys[kSortTile];
    __shared__ uint32_t s_vals[kSortTile];
    // per-wave digit counts, then exclusive over waves: never more than the tile's 4096 keys, so 16 bits
    // do (only a wave's leader lane updates an entry, with plain loads and stores); the smaller tables
    // let one more block fit a CU's LDS
    __shared__ __align__(4) uint16_t counts[kSortWaves][kRadix];
    __shared__ uint32_t digit_start[kRadix];          // first local position of each digit
    __shared__ uint32_t out_base[kRadix];             // global minus local position of each digit's run in this tile
    __shared__ uint32_t scan_tmp[2 * kSortWaves];

    const int c = blockIdx.y;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const DigitPlan dp = digit_plan(a.key_bits[c], a.pass);
    if (a.pass >= dp.passes - 1) return;        // block-uniform: this class has fewer scatter passes
    const int tile = LookBack ? lov_take_ticket(a.tickets, c) : sort_tile(row_items(a, c));
    const int begin = tile * kSortTile;
    const int count = min(kSortTile, row_items(a, c) - begin);
    if (count <= 0) return;                     // block-uniform: the row ends before this tile

    const uint32_t limit = keep_limit(a, c);
    const int64_t row = (int64_t)c * a.P;
    const uint32_t *kin = a.keys_in + row + begin;
    const uint32_t *vin = a.vals_in ? a.vals_in + row + begin : nullptr;

    // Every global read of the block is issued up front, so that the table entries (needed only after
    // the ranking) and the keys travel together. Keys beyond the row's end read as ignored, which
    // keep_key never lets through.
    uint32_t key[kSortItems], val[kSortItems], rank[kSortItems];
#pragma unroll
    for (int r = 0; r < kSortItems; ++r) {
        const int li = wave * (kSortItems * kWave) + r * kWave + lane;
        const bool valid = li < count;
        key[r] = valid ? kin[li] : kIgnoredKey;
        val[r] = vin ? (valid ? vin[li] : 0u) : (uint32_t)(begin + li);
    }
    uint32_t dtot = 0, tile_before = 0;         // thread d < kRadix: digit d's total in the row, and in the tiles before this one
    if (threadIdx.x < kRadix) {
        dtot = a.digit_total[(int64_t)c * kRadix + threadIdx.x];
        if constexpr (!LookBack) {
            if (threadIdx.x <= dp.mask) tile_before = a.tile_hist[((int64_t)c * kRadix + threadIdx.x) * a.tiles_pad + tile];
        }
    }
    for (int i = threadIdx.x; i < kSortWaves * kRadix / 2; i += kSortThreads) reinterpret_cast<uint32_t *>(&counts[0][0])[i] = 0;
    __syncthreads();
    // kRankGroup rounds at a time: their match masks do not depend on each other, so the compiler can fill
    // the wait between a vote and its use in one round with the other round's instructions; only the
    // counter updates have to follow the rounds' order.
    static_assert(kSortItems % kRankGroup == 0, "rounds are ranked in groups");
#pragma unroll
    for (int r = 0; r < kSortItems; r += kRankGroup) {
        bool valid[kRankGroup];
        uint32_t digit[kRankGroup];
        uint64_t peers[kRankGroup];
#pragma unroll
        for (int h = 0; h < kRankGroup; ++h) {
            const int li = wave * (kSortItems * kWave) + (r + h) * kWave + lane;
            valid[h] = li < count && keep_key(key[r + h], limit);
            digit[h] = (key[r + h] >> dp.shift) & dp.mask;
        }
        bool any = false;
#pragma unroll
        for (int h = 0; h < kRankGroup; ++h) any = any || valid[h];
        if (__builtin_amdgcn_ballot_w64(any) == 0) {        // wave-uniform: nothing of these rounds takes part
#pragma unroll
            for (int h = 0; h < kRankGroup; ++h) rank[r + h] = 0;
            continue;
        }
#pragma unroll
        for (int h = 0; h < kRankGroup; ++h) peers[h] = wave_peers(digit[h], valid[h]);
#pragma unroll
        for (int h = 0; h < kRankGroup; ++h) {
            uint32_t unused;
            wave_rank_of<false>(peers[h], digit[h], valid[h], false, counts[wave], nullptr, rank[r + h], unused);
        }
    }
    __syncthreads();

    uint32_t n_local;                           // keys of this tile that take part
    {
        uint32_t mine = 0;
        const int d = threadIdx.x;
        if (d < kRadix) {
            uint32_t run = 0;
#pragma unroll
            for (int w = 0; w < kSortWaves; ++w) {
                const uint32_t t = counts[w][d];
                counts[w][d] = (uint16_t)run;
                run += t;
            }
            mine = run;
            if constexpr (LookBack) {
                if (d <= (int)dp.mask)
                    tile_before = lov_look_back(a.desc + (int64_t)c * a.tiles * kRadix, tile, d, mine, a.timed_out);
            }
        }
        uint32_t row_total, local_start, global_start;
        block_excl_scan2(mine, dtot, scan_tmp, local_start, n_local, global_start, row_total);
        if (d < kRadix) {
            digit_start[d] = local_start;
            out_base[d] = global_start + tile_before - local_start;   // global position minus local one (mod 2^32)
        }
        // the digit totals of the row add up to the keys this pass lets through
        if (a.kept_out && tile == 0 && threadIdx.x == 0) a.kept_out[c] = row_total;
    }
    __syncthreads();

#pragma unroll
    for (int r = 0; r < kSortItems; ++r) {
        const int li = wave * (kSortItems * kWave) + r * kWave + lane;
        if (li < count && keep_key(key[r], limit)) {
            const uint32_t d = (key[r] >> dp.shift) & dp.mask;
            const uint32_t pos = digit_start[d] + counts[wave][d] + rank[r];
            s_keys[pos] = key[r];
            s_vals[pos] = val[r];
        }
    }
    __syncthreads();

    uint32_t *kout = a.keys_out + row;
    uint32_t *vout = a.vals_out + row;
    for (int i = threadIdx.x; i < (int)n_local; i += kSortThreads) {
        const uint32_t k = s_keys[i];
        const uint32_t d = (k >> dp.shift) & dp.mask;
        const uint32_t dst = out_base[d] + (uint32_t)i;
        kout[dst] = k;
        vout[dst] = s_vals[i];
    }
}

// ----------------------------- 3. last radix pass fused with the Jaccard step ----
// The last pass knows every key's final position k (its scatter destination) and, with the
// positives counted the same way as the keys, the number of positives sorted before it. That is
// all J_k needs, so instead of writing the sorted row the kernel evaluates the Jaccard difference
// and scatters it straight to pixel order, and leaves the tile's share of sum e_(k) dJ_k behind.

//
// Scattering 4 bytes per key to a random pixel is the slow part (each store is its own memory
// transaction). Binned = true splits it in two: pixels are grouped in regions of kRegion; every
// class row holds each pixel exactly once, so region b of a row receives exactly its own number of
// values and can be staged in place: the kernel appends (value -> jacc, pixel offset -> idx_stage)
// at a cursor inside the region's own range [b*kRegion, ...), in runs per (tile, region); a second
// kernel (lov_unbin) then permutes each region inside LDS and writes it back coalesced.
// The region size grows with the row so that a 4096-key tile still sends runs of ~16 values to a
// region: 2^13 pixels (32 KiB of fp32 in lov_unbin's LDS) up to 2^15 (128 KiB).
constexpr int kMinRegionBits = 13, kMaxRegionBits = 15;
constexpr int kMaxRegions = 1024;             // per class row; larger rows take the direct scatter

template <bool Binned, bool LookBack = false>
__global__ __launch_bounds__(kSortThreads) void lov_final(const SortArgs a, float *__restrict__ jacc,
                                                          float *__restrict__ tile_loss,
                                                          uint32_t *__restrict__ cursors, int regions, int region_bits) {
    __shared__ uint32_t region_cnt[Binned ? kMaxRegions : 1];    // keys of this tile per region
    __shared__ uint16_t region_start[Binned ? kMaxRegions : 1];  // first position of the region in the re-ordered tile (< 4096)
    __shared__ uint32_t region_base[Binned ? kMaxRegions : 1];   // this tile's run inside the region's staging range
    __shared__ float s_dj[Binned ? kSortTile : 1];               // tile re-ordered by region, so that the stores
    __shared__ uint32_t s_val[Binned ? kSortTile : 1];           // of neighbouring threads fall into the same run
    __shared__ __align__(4) uint16_t counts[kSortWaves][kRadix];       // 16 bits: see lov_scatter
    __shared__ __align__(4) uint16_t counts_hot[kSortWaves][kRadix];
    __shared__ uint32_t out_base[kRadix];     // global position of the tile's first key with digit d
    __shared__ uint32_t hot_base[kRadix];     // positives sorted before that position
    __shared__ uint32_t scan_tmp[2 * kSortWaves];
    __shared__ float wave_loss[kSortWaves];

    const int c = blockIdx.y, tile = LookBack ? lov_take_ticket(a.tickets, c) : sort_tile(row_items(a, c));
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int begin = tile * kSortTile;
    const int count = min(kSortTile, row_items(a, c) - begin);
    if (count <= 0) {                           // block-uniform: the row ends before this tile
        if (threadIdx.x == 0) tile_loss[(int64_t)c * a.tiles + tile] = 0.f;
        return;
    }
    const DigitPlan dp = digit_plan(a.key_bits[c], kLastPass);
    const LastPassRows in = last_pass_rows(a, dp.passes);
    const int64_t row = (int64_t)c * a.P;
    const uint32_t *kin = in.keys + row + begin;
    const uint32_t *vin = in.vals + row + begin;
    uint32_t *idx_stage = in.stage;

    // every global read of the block is issued up front (the table entries are needed only after the ranking)
    uint32_t key[kSortItems], val[kSortItems], rank[kSortItems], hrank[kSortItems];
    uint32_t slot[Binned ? kSortItems : 1];
#pragma unroll
    for (int r = 0; r < kSortItems; ++r) {
        const int li = wave * (kSortItems * kWave) + r * kWave + lane;
        const bool valid = li < count;
        key[r] = valid ? kin[li] : kIgnoredKey;
        val[r] = valid ? vin[li] : 0u;
    }
    uint32_t dtot = 0, htot = 0, tile_before = 0, hot_before = 0;
    if (threadIdx.x < kRadix) {
        const int64_t at = (int64_t)c * kRadix + threadIdx.x;
        dtot = a.digit_total[at];
        htot = a.hot_total[at];
        if constexpr (!LookBack) {
            if (threadIdx.x <= dp.mask) {
                tile_before = a.tile_hist[at * a.tiles_pad + tile];
                hot_before = a.tile_hot[at * a.tiles_pad + tile];
            }
        }
    }
    for (int i = threadIdx.x; i < kSortWaves * kRadix / 2; i += kSortThreads) {
        reinterpret_cast<uint32_t *>(&counts[0][0])[i] = 0;
        reinterpret_cast<uint32_t *>(&counts_hot[0][0])[i] = 0;
    }
    if constexpr (Binned)
        for (int i = threadIdx.x; i < regions; i += kSortThreads) region_cnt[i] = 0;
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kSortItems; r += kRankGroup) {      // in groups, as in lov_scatter
        uint64_t peers[kRankGroup];
#pragma unroll
        for (int h = 0; h < kRankGroup; ++h) {
            const int li = wave * (kSortItems * kWave) + (r + h) * kWave + lane;
            peers[h] = wave_peers((key[r + h] >> dp.shift) & dp.mask, li < count);
        }
#pragma unroll
        for (int h = 0; h < kRankGroup; ++h) {
            const int li = wave * (kSortItems * kWave) + (r + h) * kWave + lane;
            wave_rank_of<true>(peers[h], (key[r + h] >> dp.shift) & dp.mask, li < count, key[r + h] >> 31, counts[wave],
                               counts_hot[wave], rank[r + h], hrank[r + h]);
            if constexpr (Binned) {
                // order inside a region's staging range is irrelevant: lov_unbin puts every value at its pixel
                if (li < count) slot[r + h] = atomicAdd(&region_cnt[val[r + h] >> region_bits], 1u);
            }
        }
    }
    __syncthreads();
    if constexpr (Binned) {
        // exclusive scan of the per-region counts (each thread owns `per` consecutive regions), and one
        // cursor reservation per region the tile touches
        const int per = (regions + kSortThreads - 1) / kSortThreads;
        const int r0 = threadIdx.x * per;
        uint32_t mine = 0;
        for (int i = r0; i < min(regions, r0 + per); ++i) mine += region_cnt[i];
        uint32_t total;
        uint32_t run = block_excl_scan(mine, scan_tmp, total);
        for (int i = r0; i < min(regions, r0 + per); ++i) {
            const uint32_t n = region_cnt[i];
            region_start[i] = (uint16_t)run;
            run += n;
            region_base[i] = n ? atomicAdd(&cursors[(int64_t)c * regions + i], n) : 0u;
        }
    }

    uint32_t n_pos_u;
    {
        const int d = threadIdx.x;
        if (d < kRadix) {
            uint32_t run = 0, run_hot = 0;
#pragma unroll
            for (int w = 0; w < kSortWaves; ++w) {
                const uint32_t t = counts[w][d], th = counts_hot[w][d];
                counts[w][d] = (uint16_t)run;
                counts_hot[w][d] = (uint16_t)run_hot;
                run += t;
                run_hot += th;
            }
            if constexpr (LookBack) {
                if (d <= (int)dp.mask)
                    lov_look_back2(a.desc_wide + (int64_t)c * a.tiles * kRadix, tile, d, run, run_hot, tile_before, hot_before,
                                   a.timed_out);
            }
        }
        uint32_t total, global_start, hot_start;
        block_excl_scan2(dtot, htot, scan_tmp, global_start, total, hot_start, n_pos_u);
        if (d < kRadix) {
            out_base[d] = global_start + tile_before;
            hot_base[d] = hot_start + hot_before;
        }
    }
    __syncthreads();

    const float npos = (float)n_pos_u;
    float part = 0.f;
#pragma unroll
    for (int r = 0; r < kSortItems; ++r) {
        const int li = wave * (kSortItems * kWave) + r * kWave + lane;
        if (li < count) {
            const uint32_t k = key[r];
            const uint32_t hot = k >> 31;
            const uint32_t d = (k >> dp.shift) & dp.mask;
            float dj = 0.f;
            if ((k & 0x7FFFFFFFu) != kIgnoredKey) {
                const uint32_t pos = out_base[d] + counts[wave][d] + rank[r];            // rank in the descending order
                const uint32_t cs = hot_base[d] + counts_hot[wave][d] + hrank[r];      // positives before it
                const float inter_prev = npos - (float)cs;                             // csrc/lovasz_softmax.cu:124-127
                const float inter = npos - (float)(cs + hot);
                const float j_now = 1.f - inter / (inter + (float)(pos + 1));
                const float j_prev = (pos == 0) ? 0.f : 1.f - inter_prev / (inter_prev + (float)pos);
                dj = j_now - j_prev;                                                   // csrc/lovasz_softmax.cu:141-147
                part += key_error(k) * dj;
            }
            if constexpr (Binned) {
                const uint32_t lp = region_start[val[r] >> region_bits] + slot[r];
                s_dj[lp] = dj;
                s_val[lp] = val[r];
            } else {
                jacc[row + val[r]] = dj;
            }
        }
    }
    part = group_reduce<64>(part, OpSum());
    if (lane == 0) wave_loss[wave] = part;
    __syncthreads();
    if (threadIdx.x == 0) {
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < kSortWaves; ++w) s += wave_loss[w];
        tile_loss[(int64_t)c * a.tiles + tile] = s;
    }
    if constexpr (Binned) {
        for (int i = threadIdx.x; i < count; i += kSortThreads) {
            const uint32_t v = s_val[i];
            const uint32_t region = v >> region_bits;
            const int64_t at = row + ((int64_t)region << region_bits) + region_base[region] + ((uint32_t)i - region_start[region]);
            jacc[at] = s_dj[i];
            idx_stage[at] = v & ((1u << region_bits) - 1u);
        }
    }
}

// One block per (region, class): the region's staged values (as many as its cursor counted) are
// permuted to pixel order inside LDS; pixels whose keys stayed out of the sort get their exact 0.
constexpr int kUnbinThreads = 1024;

template <int kRegionBits>
__global__ __launch_bounds__(kUnbinThreads) void lov_unbin(float *__restrict__ jacc, const SortArgs a,
                                                           const uint32_t *__restrict__ cursors, int regions, int P,
                                                           const float *__restrict__ tile_loss, float *__restrict__ losses,
                                                           int tiles) {
    typedef unsigned plh_u4 __attribute__((ext_vector_type(4)));
    constexpr int kRegion = 1 << kRegionBits;
    __shared__ __align__(16) float sorted[kRegion];
    const uint32_t *idx_stage = last_pass_rows(a, digit_plan(a.key_bits[blockIdx.y], kLastPass).passes).stage;
    const int64_t first = (int64_t)blockIdx.y * P + ((int64_t)blockIdx.x << kRegionBits);
    const int n = min(kRegion, P - (int)(blockIdx.x << kRegionBits));
    const int staged = min(n, (int)cursors[(int64_t)blockIdx.y * regions + blockIdx.x]);
    // 16-byte accesses where the region starts on a 16-byte boundary (rows of a multiple of 4 pixels)
    const bool vec = (first & 3) == 0;
    const int staged_v = vec ? (staged & ~3) : 0, n_v = vec ? (n & ~3) : 0;
    plh_f4 *sorted4 = reinterpret_cast<plh_f4 *>(sorted);
    for (int i = threadIdx.x; i < kRegion / 4; i += kUnbinThreads) sorted4[i] = plh_f4{0.f, 0.f, 0.f, 0.f};
    __syncthreads();
    for (int i = threadIdx.x * 4; i < staged_v; i += kUnbinThreads * 4) {
        const plh_u4 at = __builtin_nontemporal_load(reinterpret_cast<const plh_u4 *>(idx_stage + first + i));
        const plh_f4 v = __builtin_nontemporal_load(reinterpret_cast<const plh_f4 *>(jacc + first + i));
        sorted[at.x & (kRegion - 1)] = v.x;
        sorted[at.y & (kRegion - 1)] = v.y;
        sorted[at.z & (kRegion - 1)] = v.z;
        sorted[at.w & (kRegion - 1)] = v.w;
    }
    for (int i = staged_v + threadIdx.x; i < staged; i += kUnbinThreads)
        sorted[idx_stage[first + i] & (kRegion - 1)] = jacc[first + i];
    __syncthreads();
    // plain stores: the backward reads these values next, and what the caches keep of them helps it
    for (int i = threadIdx.x * 4; i < n_v; i += kUnbinThreads * 4)
        *reinterpret_cast<plh_f4 *>(jacc + first + i) = sorted4[i / 4];
    for (int i = n_v + threadIdx.x; i < n; i += kUnbinThreads) jacc[first + i] = sorted[i];

    // the first block of a class also adds up the class's per-tile shares of the loss, in a fixed order
    if (blockIdx.x != 0) return;
    __syncthreads();                                // `sorted` is free again
    const int c = blockIdx.y;
    float sum = 0.f;
    for (int i = threadIdx.x; i < tiles; i += kUnbinThreads) sum += tile_loss[(int64_t)c * tiles + i];
    sum = group_reduce<64>(sum, OpSum());
    if ((threadIdx.x & 63) == 0) sorted[threadIdx.x >> 6] = sum;
    __syncthreads();
    if (threadIdx.x == 0) {
        float total = 0.f;
        for (int w = 0; w < kUnbinThreads / 64; ++w) total += sorted[w];
        if (a.timed_out && *a.timed_out) total = __builtin_nanf("");        // look-back variant: a wait ran out
        losses[c] = total;
    }
}

__global__ __launch_bounds__(256) void lov_zero_f32(float *p, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) p[i] = 0.f;
}

__global__ __launch_bounds__(256) void lov_reduce_loss(const float *__restrict__ tile_loss, float *__restrict__ losses,
                                                       int tiles) {
    __shared__ float wave_sum[4];
    const int c = blockIdx.x;
    float s = 0.f;
    for (int i = threadIdx.x; i < tiles; i += 256) s += tile_loss[(int64_t)c * tiles + i];
    s = group_reduce<64>(s, OpSum());
    if ((threadIdx.x & 63) == 0) wave_sum[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) losses[c] = (wave_sum[0] + wave_sum[1]) + (wave_sum[2] + wave_sum[3]);
}

// ------------------------------------------------------------ backward ----

template <class T, int CP, int V>
__global__ __launch_bounds__(kRegsBlock) void lov_bwd_regs(const float *__restrict__ gout, const T *__restrict__ x,
                                                          const int64_t *__restrict__ lab, const float *__restrict__ jacc,
                                                          T *__restrict__ grad, int64_t P, int64_t m_size, int C,
                                                          int64_t ignore, unsigned xcd_run) {
    const int64_t pix = (tile_of_block(xcd_run) * kRegsBlock + threadIdx.x) * V;
    if (pix >= P) return;
    const int64_t n = pix / m_size;
    const int64_t base = pix + n * (int64_t)(C - 1) * m_size;
    float v[CP][V], d[CP][V];
#pragma unroll
    for (int j = 0; j < CP; ++j)
        if (chan_ok<CP>(j, C)) {
            load_vec<V>(x + base + (int64_t)j * m_size, v[j]);
            load_vec<V>(jacc + (int64_t)j * P + pix, d[j]);
        }
    int64_t lb[V];
    load_labels<V>(lab + pix, lb);
#pragma unroll
    for (int k = 0; k < V; ++k) {
        float mx = v[0][k];
#pragma unroll
        for (int j = 1; j < CP; ++j)
            if (chan_ok<CP>(j, C)) mx = fmaxf(mx, v[j][k]);
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (chan_ok<CP>(j, C)) {
                v[j][k] = expf(v[j][k] - mx);
                s += v[j][k];
            }
        float dot = 0.f;
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (chan_ok<CP>(j, C)) {
                v[j][k] = v[j][k] / s;
                const float dj = d[j][k] * gout[j];
                d[j][k] = (lb[k] == j) ? -dj : dj;
                dot += v[j][k] * d[j][k];
            }
        const bool ign = (lb[k] == ignore);
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (chan_ok<CP>(j, C)) v[j][k] = ign ? 0.f : v[j][k] * (d[j][k] - dot);
    }
#pragma unroll
    for (int j = 0; j < CP; ++j)
        if (chan_ok<CP>(j, C)) store_vec<V>(grad + base + (int64_t)j * m_size, v[j]);
}

template <class T>
__global__ __launch_bounds__(256) void lov_bwd_lane(const float *__restrict__ gout, const T *__restrict__ x,
                                                    const int64_t *__restrict__ lab, const float *__restrict__ jacc,
                                                    T *__restrict__ grad, int64_t P, int64_t m_size, int C,
                                                    int64_t ignore) {
    for (int64_t pix = (int64_t)blockIdx.x * 256 + threadIdx.x; pix < P; pix += (int64_t)gridDim.x * 256) {
        const int64_t n = pix / m_size;
        const int64_t base = pix + n * (int64_t)(C - 1) * m_size;
        const T *xs = x + base;
        const int64_t lb = lab[pix];
        float mx = -INFINITY;
#pragma unroll 8
        for (int j = 0; j < C; ++j) mx = fmaxf(mx, load_one(xs + (int64_t)j * m_size));
        float s = 0.f;
#pragma unroll 8
        for (int j = 0; j < C; ++j) s += expf(load_one(xs + (int64_t)j * m_size) - mx);
        float dot = 0.f;
#pragma unroll 8
        for (int j = 0; j < C; ++j) {
            const float p = expf(load_one(xs + (int64_t)j * m_size) - mx) / s;
            const float dj = jacc[(int64_t)j * P + pix] * gout[j];
            dot += p * ((lb == j) ? -dj : dj);
        }
        const bool ign = (lb == ignore);
#pragma unroll 8
        for (int j = 0; j < C; ++j) {
            const float p = expf(load_one(xs + (int64_t)j * m_size) - mx) / s;
            const float dj = jacc[(int64_t)j * P + pix] * gout[j];
            store_one(grad + (base + (int64_t)j * m_size), ign ? 0.f : p * (((lb == j) ? -dj : dj) - dot));
        }
    }
}

// ------------------------------------------------------------ host side ----

struct LovaszPlan {
    int64_t P, E;
    int tiles, tiles_pad;
    int regions;            // pixel regions per class row (0 = direct scatter)
    int region_bits;        // log2 of the pixels per region
    int64_t off_keys_a, off_keys_c, off_vals_a, off_vals_b, off_hist, off_hot, off_digit_total, off_hot_total,
        off_tile_loss, off_cursors, off_class, off_block_max, bytes;
    // look-back variant: tickets + time-out word + descriptors (cleared per call), totals, per-block tables
    bool look_back;
    int hist_blocks;
    int64_t off_lb_clear, lb_clear_bytes, off_lb_totals, off_lb_partial;
};

static int64_t round_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

static int make_plan(int64_t n_size, int64_t dimsize, int64_t m_size, LovaszPlan &pl, bool look_back = false) {
    if (n_size < 0 || dimsize < 0 || m_size < 0) return PLH_ERR_BAD_SIZE;
    if (dimsize >= 512) return PLH_ERR_TOO_MANY_CLASSES;
    const double numel = (double)n_size * (double)dimsize * (double)m_size;
    if (numel >= 2147483648.0) return PLH_ERR_BAD_SIZE;
    pl.P = n_size * m_size;
    pl.E = pl.P * dimsize;
    pl.tiles = (int)ceil_div(pl.P, kSortTile);
    pl.tiles_pad = (int)round_up(pl.tiles, kSortWaves);
    int64_t off = 0;
    pl.off_keys_a = off;      off += round_up(4 * pl.E, 256);
    pl.off_keys_c = off;      off += round_up(4 * pl.E, 256);
    pl.off_vals_a = off;      off += round_up(4 * pl.E, 256);
    pl.off_vals_b = off;      off += round_up(4 * pl.E, 256);
    pl.off_hist = off;        off += round_up(4 * dimsize * kRadix * pl.tiles_pad, 256);
    pl.off_hot = off;         off += round_up(4 * dimsize * kRadix * pl.tiles_pad, 256);
    pl.off_digit_total = off; off += round_up(4 * dimsize * kRadix, 256);
    pl.off_hot_total = off;   off += round_up(4 * dimsize * kRadix, 256);
    pl.off_tile_loss = off;   off += round_up(4 * dimsize * pl.tiles, 256);
    // the smallest region size that keeps a row within 256 regions (runs of >= 16 values per tile and region)
    pl.region_bits = kMinRegionBits;
    while (pl.region_bits < kMaxRegionBits && ceil_div(pl.P, (int64_t)1 << pl.region_bits) > 256) ++pl.region_bits;
    const int64_t regions = ceil_div(pl.P, (int64_t)1 << pl.region_bits);
    pl.regions = (regions <= kMaxRegions) ? (int)regions : 0;
    pl.off_cursors = off;     off += round_up(4 * dimsize * kMaxRegions, 256);
    pl.off_class = off;       off += round_up(4 * dimsize * 4, 256);      // pos_max[C], kept[C], all_min[C], key_bits[C]
    pl.off_block_max = off;   off += round_up(4 * dimsize * ceil_div(pl.P, 256), 256);   // [key blocks][C]
    // the look-back descriptors carry a count in 30 bits next to their 2 state bits
    if (look_back && pl.P >= ((int64_t)1 << 30)) return PLH_ERR_BAD_SIZE;
    pl.look_back = look_back && pl.regions > 0;
    pl.hist_blocks = (int)ceil_div(pl.tiles, 2);
    if (pl.look_back) {
        // [4 passes][C] tickets + 1 word, 3 x [C][tiles][kRadix] u32 descriptors, [C][tiles][kRadix] u64 ones
        pl.lb_clear_bytes = round_up(4 * (4 * dimsize + 1), 256) + (int64_t)(3 * 4 + 8) * dimsize * pl.tiles * kRadix;
        pl.off_lb_clear = off;    off += round_up(pl.lb_clear_bytes, 256);
        pl.off_lb_totals = off;   off += round_up(4 * (int64_t)kHistTables * dimsize * kRadix, 256);
        pl.off_lb_partial = off;  off += round_up(4 * (int64_t)dimsize * pl.hist_blocks * kHistTables * kRadix, 256);
    }
    pl.bytes = off;
    return PLH_OK;
}

}  // namespace plh

using namespace plh;

extern "C" int64_t plh_lovasz_workspace_bytes(int64_t n_size, int64_t dimsize, int64_t m_size) {
    LovaszPlan pl;
    const int rc = make_plan(n_size, dimsize, m_size, pl);
    return rc == PLH_OK ? pl.bytes : (int64_t)rc;
}

extern "C" int64_t plh_lovasz_lookback_workspace_bytes(int64_t n_size, int64_t dimsize, int64_t m_size) {
    LovaszPlan pl;
    const int rc = make_plan(n_size, dimsize, m_size, pl, true);
    return rc == PLH_OK ? pl.bytes : (int64_t)rc;
}

static int lovasz_forward(const void *logits, int32_t dtype, const int64_t *labels, float *losses, float *jacc,
                          void *workspace, int64_t workspace_bytes, int64_t n_size, int64_t dimsize, int64_t m_size,
                          int64_t ignore_index, void *stream, bool look_back) {
    if (!dtype_ok(dtype)) return PLH_ERR_BAD_DTYPE;
    LovaszPlan pl;
    int rc = make_plan(n_size, dimsize, m_size, pl, look_back);
    if (rc != PLH_OK) return rc;
    if (pl.E == 0) return PLH_OK;
    if (!logits || !labels || !losses || !jacc) return PLH_ERR_NULL_POINTER;
    if (misaligned(logits, dtype_size(dtype)) || misaligned(losses, 4) || misaligned(jacc, 4) || misaligned(labels, 8))
        return PLH_ERR_MISALIGNED;
    if (!workspace || misaligned(workspace, 256) || workspace_bytes < pl.bytes) return PLH_ERR_WORKSPACE;

    hipStream_t st = (hipStream_t)stream;
    char *ws = static_cast<char *>(workspace);
    uint32_t *keys_0 = reinterpret_cast<uint32_t *>(jacc);          // the keys as built, in pixel order; jacc is free until the last pass
    uint32_t *keys_a = reinterpret_cast<uint32_t *>(ws + pl.off_keys_a);
    uint32_t *keys_c = reinterpret_cast<uint32_t *>(ws + pl.off_keys_c);
    uint32_t *vals_a = reinterpret_cast<uint32_t *>(ws + pl.off_vals_a);
    uint32_t *vals_b = reinterpret_cast<uint32_t *>(ws + pl.off_vals_b);
    uint32_t *hist = reinterpret_cast<uint32_t *>(ws + pl.off_hist);
    uint32_t *hot = reinterpret_cast<uint32_t *>(ws + pl.off_hot);
    uint32_t *digit_total = reinterpret_cast<uint32_t *>(ws + pl.off_digit_total);
    uint32_t *hot_total = reinterpret_cast<uint32_t *>(ws + pl.off_hot_total);
    float *tile_loss = reinterpret_cast<float *>(ws + pl.off_tile_loss);
    uint32_t *pos_max = reinterpret_cast<uint32_t *>(ws + pl.off_class);
    uint32_t *kept = pos_max + dimsize;
    uint32_t *all_min = pos_max + 2 * dimsize;
    uint32_t *key_bits = pos_max + 3 * dimsize;
    const int C = (int)dimsize;

    uint32_t *block_table = reinterpret_cast<uint32_t *>(ws + pl.off_block_max);
    unsigned key_blocks = 0;

    // 1. keys (into keys_0 = jacc: rows of [C][P] u32; a row start stays 8-/16-byte aligned when P % V == 0)
    dispatch_dtype(dtype, [&](auto tag) {
        using T = decltype(tag);
        const T *x = static_cast<const T *>(logits);
        constexpr int VT = ElemTraits<T>::kVec;
        const Shape shape = pick_shape(dimsize, m_size, VT, sizeof(T), x, nullptr, labels, keys_0, nullptr);
        if (shape == Shape::RegsVec || shape == Shape::RegsOne) {
            const bool vec = (shape == Shape::RegsVec);
            const unsigned grid = vec ? regs_grid<VT>(pl.P) : regs_grid<1>(pl.P);
            const unsigned run = xcd_run_for(sizeof(T), m_size);
            key_blocks = grid;
            switch ((C + 3) / 4) {
#define PLH_CASE(K)                                                                                                 \
    case K:                                                                                                         \
        if (vec) hipLaunchKernelGGL((lov_keys_regs<T, 4 * K, VT>), dim3(grid), dim3(kRegsBlock), 0, st, x, labels,  \
                                    keys_0, block_table, pl.P, m_size, C, ignore_index, run);                       \
        else hipLaunchKernelGGL((lov_keys_regs<T, 4 * K, 1>), dim3(grid), dim3(kRegsBlock), 0, st, x, labels,       \
                                keys_0, block_table, pl.P, m_size, C, ignore_index, run);                           \
        break;
                PLH_CASE(1) PLH_CASE(2) PLH_CASE(3) PLH_CASE(4) PLH_CASE(5) PLH_CASE(6) PLH_CASE(7) PLH_CASE(8)
#undef PLH_CASE
            }
        } else {
            key_blocks = group_grid(pl.P, 256);
            hipLaunchKernelGGL(lov_keys_lane<T>, dim3(key_blocks), dim3(256), 0, st, x, labels, keys_0, block_table,
                               pl.P, m_size, C, ignore_index);
        }
    });
    hipLaunchKernelGGL(lov_class_max, dim3((unsigned)C), dim3(256), 0, st, block_table, (int)key_blocks, C, pos_max,
                       reinterpret_cast<uint32_t *>(ws + pl.off_cursors), pl.regions);
    hipLaunchKernelGGL(lov_absent_min, dim3(kAbsentBlocks, (unsigned)C), dim3(256), 0, st, keys_0, pos_max, all_min,
                       (int)pl.P);

    // 2. up to three stable scatter passes: (keys_0, -) -> (keys_a, vals_a) -> (keys_c, vals_b) -> (keys_a, vals_a);
    //    how many a class takes follows from the width of its keys (DigitPlan), the blocks of a pass
    //    that a class does not take return at once. The first pass drops the keys whose Jaccard
    //    difference is known to be 0 (keep_key) and counts what is left per class; the later passes
    //    work on those counts and their surplus blocks return at once.
    const dim3 tile_grid((unsigned)pl.tiles, (unsigned)C);
    // a histogram block counts two tiles; lov_row_scan reads the live tiles in whole groups of kSortWaves
    const dim3 hist_grid((unsigned)round_up(ceil_div(pl.tiles, 2), kSortWaves / 2), (unsigned)C);
    SortArgs a;
    a.desc = nullptr;
    a.desc_wide = nullptr;
    a.tickets = nullptr;
    a.timed_out = nullptr;
    a.keys_alt = nullptr;
    a.vals_alt = nullptr;
    a.tile_hist = hist;
    a.digit_total = digit_total;
    a.tile_hot = hot;
    a.hot_total = hot_total;
    a.key_bits = key_bits;
    a.P = (int)pl.P;
    a.tiles = pl.tiles;
    a.tiles_pad = pl.tiles_pad;
    uint32_t *lb_words = pl.look_back ? reinterpret_cast<uint32_t *>(ws + pl.off_lb_clear) : nullptr;
    uint32_t *lb_desc = pl.look_back ? reinterpret_cast<uint32_t *>(ws + pl.off_lb_clear + round_up(4 * (4 * C + 1), 256)) : nullptr;
    uint32_t *lb_totals = pl.look_back ? reinterpret_cast<uint32_t *>(ws + pl.off_lb_totals) : nullptr;
    if (pl.look_back) {
        // tickets, time-out word and descriptors start at zero; digit totals of every pass from one sweep over the keys
        hipLaunchKernelGGL(lov_zero_f32, dim3(4096), dim3(256), 0, st, reinterpret_cast<float *>(lb_words),
                           pl.lb_clear_bytes / 4);
        uint32_t *partial = reinterpret_cast<uint32_t *>(ws + pl.off_lb_partial);
        a.keys_in = keys_0;
        a.pos_max = pos_max;
        a.all_min = all_min;
        hipLaunchKernelGGL(lov_hist_all, dim3((unsigned)pl.hist_blocks, (unsigned)C), dim3(kSortThreads), 0, st, a, partial,
                           pl.hist_blocks);
        hipLaunchKernelGGL(lov_hist_reduce, dim3(kHistTables, (unsigned)C), dim3(kRadix), 0, st, partial, pl.hist_blocks, C,
                           lb_totals);
        a.timed_out = lb_words + 4 * C;
    }
    for (int pass = 0; pass < 3; ++pass) {
        a.keys_in = pass == 0 ? keys_0 : (pass == 1 ? keys_a : keys_c);
        a.vals_in = pass == 0 ? nullptr : (pass == 1 ? vals_a : vals_b);
        a.keys_out = pass == 1 ? keys_c : keys_a;
        a.vals_out = pass == 1 ? vals_b : vals_a;
        a.pass = pass;
        a.pos_max = (pass == 0) ? pos_max : nullptr;
        a.all_min = (pass == 0) ? all_min : nullptr;
        a.kept_in = (pass == 0) ? nullptr : kept;
        a.kept_out = (pass == 0) ? kept : nullptr;
        if (pl.look_back) {
            a.digit_total = lb_totals + (int64_t)pass * C * kRadix;
            a.desc = lb_desc + (int64_t)pass * C * pl.tiles * kRadix;
            a.tickets = lb_words + pass * C;
            hipLaunchKernelGGL(lov_scatter<true>, tile_grid, dim3(kSortThreads), 0, st, a);
            continue;
        }
        hipLaunchKernelGGL(lov_tile_hist<false>, hist_grid, dim3(kSortThreads), 0, st, a);
        hipLaunchKernelGGL(lov_row_scan, dim3(kRadix, (unsigned)C, 1), dim3(256), 0, st, hist, digit_total, hot,
                           hot_total, pl.tiles_pad, key_bits, pass, a.kept_in, (int)pl.P);
        hipLaunchKernelGGL(lov_scatter<false>, tile_grid, dim3(kSortThreads), 0, st, a);
    }

    // 3. last pass (the top digit of the class; bit 31 is never part of a digit) fused with the Jaccard
    //    step: reads the sorted-so-far rows and scatters the Jaccard differences into jacc
    a.keys_in = keys_a;
    a.vals_in = vals_a;
    a.keys_alt = keys_c;
    a.vals_alt = vals_b;
    a.keys_out = nullptr;
    a.vals_out = nullptr;
    a.pass = kLastPass;
    a.pos_max = nullptr;
    a.all_min = nullptr;
    a.kept_in = kept;
    a.kept_out = nullptr;
    if (pl.look_back) {
        a.digit_total = lb_totals + (int64_t)3 * C * kRadix;
        a.hot_total = lb_totals + (int64_t)4 * C * kRadix;
        a.desc_wide = reinterpret_cast<unsigned long long *>(lb_desc + (int64_t)3 * C * pl.tiles * kRadix);
        a.tickets = lb_words + 3 * C;
    } else {
        hipLaunchKernelGGL(lov_tile_hist<true>, hist_grid, dim3(kSortThreads), 0, st, a);
        hipLaunchKernelGGL(lov_row_scan, dim3(kRadix, (unsigned)C, 2), dim3(256), 0, st, hist, digit_total, hot, hot_total,
                           pl.tiles_pad, key_bits, kLastPass, kept, (int)pl.P);
    }
    if (pl.regions > 0) {
        uint32_t *cursors = reinterpret_cast<uint32_t *>(ws + pl.off_cursors);      // zeroed by lov_class_max
        // the value buffer that a class's last pass does not read receives the pixel offsets that go with
        // the staged values
        if (pl.look_back)
            hipLaunchKernelGGL((lov_final<true, true>), tile_grid, dim3(kSortThreads), 0, st, a, jacc, tile_loss, cursors,
                               pl.regions, pl.region_bits);
        else
            hipLaunchKernelGGL((lov_final<true, false>), tile_grid, dim3(kSortThreads), 0, st, a, jacc, tile_loss, cursors,
                               pl.regions, pl.region_bits);
        const dim3 unbin_grid((unsigned)pl.regions, (unsigned)C);
        switch (pl.region_bits) {
#define PLH_UNBIN(B)                                                                                                  \
    case B:                                                                                                           \
        hipLaunchKernelGGL(lov_unbin<B>, unbin_grid, dim3(kUnbinThreads), 0, st, jacc, a, cursors, pl.regions,        \
                           (int)pl.P, tile_loss, losses, pl.tiles);                                                   \
        break;
            PLH_UNBIN(13) PLH_UNBIN(14) PLH_UNBIN(15)
#undef PLH_UNBIN
        }
    } else {
        // direct scatter: the pixels whose keys stayed out of the sort are not written, so clear first
        // (jacc stopped being a key buffer when the first pass read it)
        hipLaunchKernelGGL(lov_zero_f32, dim3(4096), dim3(256), 0, st, jacc, pl.E);
        hipLaunchKernelGGL((lov_final<false, false>), tile_grid, dim3(kSortThreads), 0, st, a, jacc, tile_loss, nullptr, 0, 0);
        hipLaunchKernelGGL(lov_reduce_loss, dim3((unsigned)C), dim3(256), 0, st, tile_loss, losses, pl.tiles);
    }
    return check_launch();
}

extern "C" int plh_lovasz_forward(const void *logits, int32_t dtype, const int64_t *labels, float *losses, float *jacc,
                                  void *workspace, int64_t workspace_bytes,
                                  int64_t n_size, int64_t dimsize, int64_t m_size,
                                  int64_t ignore_index, void *stream) {
    return lovasz_forward(logits, dtype, labels, losses, jacc, workspace, workspace_bytes, n_size, dimsize, m_size,
                          ignore_index, stream, false);
}

extern "C" int plh_lovasz_forward_lookback(const void *logits, int32_t dtype, const int64_t *labels, float *losses,
                                           float *jacc, void *workspace, int64_t workspace_bytes,
                                           int64_t n_size, int64_t dimsize, int64_t m_size,
                                           int64_t ignore_index, void *stream) {
    return lovasz_forward(logits, dtype, labels, losses, jacc, workspace, workspace_bytes, n_size, dimsize, m_size,
                          ignore_index, stream, true);
}

extern "C" int plh_lovasz_backward(const float *grad_output, const void *logits, int32_t dtype, const int64_t *labels,
                                   const float *jacc, void *grad_logits,
                                   int64_t n_size, int64_t dimsize, int64_t m_size,
                                   int64_t ignore_index, void *stream) {
    if (!dtype_ok(dtype)) return PLH_ERR_BAD_DTYPE;
    LovaszPlan pl;
    const int rc = make_plan(n_size, dimsize, m_size, pl);
    if (rc != PLH_OK) return rc;
    if (pl.E == 0) return PLH_OK;
    if (!grad_output || !logits || !labels || !jacc || !grad_logits) return PLH_ERR_NULL_POINTER;
    if (misaligned(grad_output, 4) || misaligned(logits, dtype_size(dtype)) || misaligned(jacc, 4) ||
        misaligned(grad_logits, dtype_size(dtype)) || misaligned(labels, 8))
        return PLH_ERR_MISALIGNED;
    hipStream_t st = (hipStream_t)stream;
    const int C = (int)dimsize;
    dispatch_dtype(dtype, [&](auto tag) {
        using T = decltype(tag);
        const T *x = static_cast<const T *>(logits);
        T *g = static_cast<T *>(grad_logits);
        constexpr int VT = ElemTraits<T>::kVec;
        const Shape shape = pick_shape(dimsize, m_size, VT, sizeof(T), x, g, labels, jacc, nullptr);
        if (shape == Shape::RegsVec || shape == Shape::RegsOne) {
            const bool vec = (shape == Shape::RegsVec);
            const unsigned grid = vec ? regs_grid<VT>(pl.P) : regs_grid<1>(pl.P);
            const unsigned run = xcd_run_for(sizeof(T), m_size);
            switch ((C + 3) / 4) {
#define PLH_CASE(K)                                                                                                  \
    case K:                                                                                                          \
        if (vec) hipLaunchKernelGGL((lov_bwd_regs<T, 4 * K, VT>), dim3(grid), dim3(kRegsBlock), 0, st, grad_output,  \
                                    x, labels, jacc, g, pl.P, m_size, C, ignore_index, run);                         \
        else hipLaunchKernelGGL((lov_bwd_regs<T, 4 * K, 1>), dim3(grid), dim3(kRegsBlock), 0, st, grad_output, x,    \
                                labels, jacc, g, pl.P, m_size, C, ignore_index, run);                                \
        break;
                PLH_CASE(1) PLH_CASE(2) PLH_CASE(3) PLH_CASE(4) PLH_CASE(5) PLH_CASE(6) PLH_CASE(7) PLH_CASE(8)
#undef PLH_CASE
            }
        } else {
            hipLaunchKernelGGL(lov_bwd_lane<T>, dim3(group_grid(pl.P, 256)), dim3(256), 0, st, grad_output, x, labels,
                               jacc, g, pl.P, m_size, C, ignore_index);
        }
    });
    return check_launch();
}
