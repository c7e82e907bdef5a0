// One-hot / label-smoothed target encoding for gfx950 (csrc/one_hot_kernel.cu:194-335):
//   out[n, j, m] = 0 at an ignored pixel, else (j == label ? 1 - smooth : smooth / C).
// A pure write stream of 4*C*P bytes behind an 8*P byte read (labels are re-read per channel plane,
// from cache). The reference first reduces the labels
// to their maximum and minimum and copies both to the host (:301-304, a device synchronisation) to
// refuse labels outside [0, C). Here the encoding kernel raises two flags on the side while it has
// the labels in registers anyway; whether and when to read them back is the caller's choice. A
// label outside [0, C) never addresses memory: it just matches no channel.
#include "plh_common.hpp"

namespace plh {

__global__ void onehot_zero_flags(int32_t *flags) {
    if (threadIdx.x < 2) flags[threadIdx.x] = 0;
}

__device__ __forceinline__ void flag_range(int64_t lb, int64_t ignore, int C, int32_t *flags) {
    if (!flags || lb == ignore) return;
    if (lb >= (int64_t)C) flags[0] = 1;          // every writer stores the same value
    if (lb < 0) flags[1] = 1;
}

// C <= 32: lanes along pixels, V pixels per thread, one 4*V-byte store per channel.
template <int CP, int V, bool Uniform>
__global__ __launch_bounds__(kRegsBlock) void onehot_regs(const int64_t *__restrict__ lab, float *__restrict__ out,
                                                         int32_t *__restrict__ flags, int64_t P, int64_t m_size, int C,
                                                         int64_t ignore, float lb_pos, float lb_neg, unsigned xcd_run) {
    const PixelRef<V, Uniform> at(P, m_size, C, xcd_run);
    if (!at.live) return;
    int64_t lb[V];
    load_labels<V>(lab + at.pix, lb);
    int tgt[V];
    float neg[V];
#pragma unroll
    for (int k = 0; k < V; ++k) {
        flag_range(lb[k], ignore, C, flags);
        bool ign;
        tgt[k] = narrow_label(lb[k], ignore, C, ign);
        neg[k] = ign ? 0.f : lb_neg;
    }
    typename Pack<float, V>::Raw raw[CP];
#pragma unroll
    for (int j = 0; j < CP; ++j)
        if (chan_ok<CP>(j, C)) {
            float v[V];
#pragma unroll
            for (int k = 0; k < V; ++k) v[k] = (tgt[k] == j) ? lb_pos : neg[k];
            raw[j] = Pack<float, V>::put(v);
        }
    at.store_slice(out, C, m_size, raw);
}

// One block per 1024 consecutive elements of one channel plane (planes of 256 pixels or more, of any length and
// alignment): the output is written plane after plane like
// a plain fill, with stores that do not allocate in the caches (7.1 TB/s against 5.9 TB/s with ordinary stores
// at (8,19,1024,1024)); the labels are re-read per channel, from cache. Planes of more than kOnehotChunk pixels
// go chunk by chunk (blockIdx.y = channel, blockIdx.z = image * chunks + chunk), so that the labels a channel pass
// re-reads are the 8 MiB (1 MiB per XCD) that the pass before it left in the second-level caches: whole planes of
// 2048 x 2048 pixels ran at 3.4 TB/s.
constexpr int64_t kOnehotChunk = (int64_t)1 << 20;
template <bool Lines>      // Lines: every output plane starts on a 128-byte line and holds whole groups of four
__global__ __launch_bounds__(kRegsBlock) void onehot_plane(const int64_t *__restrict__ lab, float *__restrict__ out,
                                                          int32_t *__restrict__ flags, int64_t m_size, int C,
                                                          int chunks, int64_t chunk, int64_t ignore, float lb_pos,
                                                          float lb_neg) {
    const int j = blockIdx.y;
    const int n = chunks == 1 ? (int)blockIdx.z : (int)blockIdx.z / chunks, q = (int)blockIdx.z - n * chunks;
    // Planes of any length and alignment: the plane's first `head` elements (up to the first 128-byte line of the
    // output) are written one by one by the plane's first block; from there on a lane's four pixels are 16 bytes
    // on a 16-byte boundary and a wavefront's store is eight whole lines. The labels of those pixels start on
    // 8-byte boundaries only (the hardware takes 16-byte loads from there, the type says so). The last lane of
    // a plane may hold fewer than four pixels and goes pixel by pixel.
    const int64_t *lplane = lab + (int64_t)n * m_size;
    float *oplane = out + ((int64_t)n * C + j) * m_size;
    int64_t head = 0;
    if constexpr (!Lines) {
        const int64_t to_line = (int64_t)((128u - (unsigned)(reinterpret_cast<uintptr_t>(oplane) & 127u)) & 127u) / 4;
        head = to_line < m_size ? to_line : m_size;
    }
    auto encode = [&](int64_t label) { return (label == ignore) ? 0.f : ((label == j) ? lb_pos : lb_neg); };
    int64_t seen[5] = {ignore, ignore, ignore, ignore, ignore};      // this lane's labels, for the range check below
    if constexpr (!Lines) {
        if (q == 0 && blockIdx.x == 0 && (int64_t)threadIdx.x < head) {
            seen[4] = lplane[threadIdx.x];
            oplane[threadIdx.x] = encode(seen[4]);
        }
    }
    const int64_t m = head + (int64_t)q * chunk + ((int64_t)blockIdx.x * kRegsBlock + threadIdx.x) * 4;
    if constexpr (Lines) {
        if (m >= m_size) return;
    }
    if (Lines || m + 4 <= m_size) {
        const plh_l2_a8 a = *reinterpret_cast<const plh_l2_a8 *>(lplane + m);
        const plh_l2_a8 b = *reinterpret_cast<const plh_l2_a8 *>(lplane + m + 2);
        seen[0] = a.x; seen[1] = a.y; seen[2] = b.x; seen[3] = b.y;
        const plh_f4 v = {encode(a.x), encode(a.y), encode(b.x), encode(b.y)};
        __builtin_nontemporal_store(v, reinterpret_cast<plh_f4 *>(oplane + m));
    } else {
#pragma unroll
        for (int k = 0; k < 3; ++k)
            if (m + k < m_size) {
                seen[k] = lplane[m + k];
                oplane[m + k] = encode(seen[k]);
            }
    }
    if (flags != nullptr && j == 0) {            // block-uniform: the blocks of one channel check the range
        bool above = false, below = false;
#pragma unroll
        for (int k = 0; k < 5; ++k) {
            above |= seen[k] != ignore && seen[k] >= (int64_t)C;
            below |= seen[k] != ignore && seen[k] < 0;
        }
        if (above) flags[0] = 1;                 // every writer stores the same value
        if (below) flags[1] = 1;
    }
}

// Any C: one thread per V consecutive output elements of one channel row; labels are re-read per
// channel, through cache.
template <int V>
__global__ __launch_bounds__(256) void onehot_rows(const int64_t *__restrict__ lab, float *__restrict__ out,
                                                   int32_t *__restrict__ flags, int64_t n_size, int64_t C,
                                                   int64_t m_size, int64_t ignore, float lb_pos, float lb_neg) {
    const int64_t per_row = m_size / V;                      // V divides m_size
    const int64_t total = n_size * C * per_row;
    for (int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x; t < total; t += (int64_t)gridDim.x * 256) {
        const int64_t row = t / per_row, m = (t - row * per_row) * V;
        const int64_t n = row / C, j = row - n * C;
        float v[V];
#pragma unroll
        for (int k = 0; k < V; ++k) {
            const int64_t lb = lab[n * m_size + m + k];
            if (j == 0) flag_range(lb, ignore, (int)C, flags);
            v[k] = (lb == ignore) ? 0.f : ((lb == j) ? lb_pos : lb_neg);
        }
        store_vec<V>(out + row * m_size + m, v);
    }
}

}  // namespace plh

using namespace plh;

extern "C" int plh_onehot(const int64_t *labels, float *one_hot, int32_t *range_flags,
                          int64_t n_size, int64_t dimsize, int64_t m_size,
                          int64_t ignore_index, float smooth, void *stream) {
    const int rc = check_slice_args(one_hot, labels, one_hot, n_size, dimsize, m_size, 4, 4);
    if (rc != PLH_OK) return rc;
    if (range_flags && misaligned(range_flags, 4)) return PLH_ERR_MISALIGNED;
    hipStream_t st = (hipStream_t)stream;
    if (range_flags) hipLaunchKernelGGL(onehot_zero_flags, dim3(1), dim3(64), 0, st, range_flags);
    if (n_size * dimsize * m_size == 0) return range_flags ? check_launch() : PLH_OK;
    const int64_t P = n_size * m_size;
    const int C = (int)dimsize;
    const float lb_pos = 1.f - smooth;                       // csrc/one_hot_kernel.cu:305
    const float lb_neg = smooth / (float)dimsize;            // csrc/one_hot_kernel.cu:306
    const Shape shape = pick_shape(dimsize, m_size, 2, 4, one_hot, nullptr, labels, nullptr, nullptr);
    // Writing plane after plane like a plain fill is the fastest order measured (against all channels of a
    // pixel tile at once, i.e. C streams 4*m_size bytes apart: 5.3-5.8 TB/s with the same stores).
    const int64_t chunks = ceil_div(m_size, kOnehotChunk);
    if (m_size >= 256 && n_size * chunks < 65536 && dimsize < 65536) {
        // equal chunks of a whole number of 8 tiles: workgroups go round the 8 XCDs in launch order, so with a
        // multiple of 8 blocks per plane and chunk (the surplus ones return at once) a tile of pixels meets the same
        // XCD, and its labels that XCD's L2, in every channel pass. Planes of 977 or 258 tiles ran at 35-42 % of peak
        // (every channel pass fetched the labels from memory again) where planes of 1024 tiles ran at 90 %.
        const int64_t chunk = ceil_div(ceil_div(m_size, chunks), 8192) * 8192;
        const dim3 grid((unsigned)(chunk / 1024), (unsigned)dimsize, (unsigned)(n_size * chunks));
        if (m_size % 32 == 0 && !misaligned(one_hot, 128))
            hipLaunchKernelGGL(onehot_plane<true>, grid, dim3(kRegsBlock), 0, st, labels, one_hot, range_flags, m_size, C,
                               (int)chunks, chunk, ignore_index, lb_pos, lb_neg);
        else
            hipLaunchKernelGGL(onehot_plane<false>, grid, dim3(kRegsBlock), 0, st, labels, one_hot, range_flags, m_size, C,
                               (int)chunks, chunk, ignore_index, lb_pos, lb_neg);
        return check_launch();
    }
    if (shape == Shape::RegsVec || shape == Shape::RegsOne) {
        // row lengths that are not a multiple of 4: 2 pixels or 1 pixel per thread, general addressing
        const bool vec = (shape == Shape::RegsVec);
        const unsigned grid = vec ? regs_grid<2>(P) : regs_grid<1>(P);
        const unsigned run = xcd_run_for(4, m_size);
        switch ((C + 3) / 4) {
#define PLH_CASE(K)                                                                                                   \
    case K:                                                                                                           \
        if (vec) hipLaunchKernelGGL((onehot_regs<4 * K, 2, false>), dim3(grid), dim3(kRegsBlock), 0, st, labels,      \
                                    one_hot, range_flags, P, m_size, C, ignore_index, lb_pos, lb_neg, run);           \
        else hipLaunchKernelGGL((onehot_regs<4 * K, 1, false>), dim3(grid), dim3(kRegsBlock), 0, st, labels, one_hot, \
                                range_flags, P, m_size, C, ignore_index, lb_pos, lb_neg, run);                        \
        break;
            PLH_CASE(1) PLH_CASE(2) PLH_CASE(3) PLH_CASE(4) PLH_CASE(5) PLH_CASE(6) PLH_CASE(7) PLH_CASE(8)
#undef PLH_CASE
        }
    } else {
        const bool vec4 = (m_size % 4 == 0) && !misaligned(one_hot, 16);
        const int64_t units = n_size * dimsize * (vec4 ? m_size / 4 : m_size);
        const unsigned grid = (unsigned)(ceil_div(units, 256) < 65536 ? ceil_div(units, 256) : 65536);
        if (vec4) hipLaunchKernelGGL(onehot_rows<4>, dim3(grid), dim3(256), 0, st, labels, one_hot, range_flags, n_size,
                                     dimsize, m_size, ignore_index, lb_pos, lb_neg);
        else hipLaunchKernelGGL(onehot_rows<1>, dim3(grid), dim3(256), 0, st, labels, one_hot, range_flags, n_size,
                                dimsize, m_size, ignore_index, lb_pos, lb_neg);
    }
    return check_launch();
}
