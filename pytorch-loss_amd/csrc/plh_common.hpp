// Shared device/host helpers for the gfx950 loss kernels.
//
// Execution shapes of the channel-dim reductions:
//   "regs"  : up to 32 channels. Lanes run along consecutive pixels, each thread owns V
//             pixels and keeps the whole channel slice in VGPRs. Each per-channel load of
//             a wavefront is one contiguous 64*V*4-byte run, logits are read from HBM
//             exactly once and no cross-lane traffic is needed. (N, C) inputs with C <= 32
//             take the same kernels; a wavefront moves its 64 rows through a private LDS tile.
//   "split" : 33..512 channels in NCHW. The regs shape with the slice of a pixel shared out
//             over the 8 wavefronts of a block; per-wavefront statistics meet in LDS.
//   "wrow"  : (N, C) rows of 33..2048 elements (4096 for 16-bit rows in 16-byte pieces) held in the
//             registers of the 64 (or 16) lanes that share a row; every sweep after the first runs on registers.
//   "row"   : (N, C) rows longer than that (every loss, the OHEM scores and the Taylor ops): a
//             block per row, 16-byte chunks, running statistics that are rescaled when the
//             maximum moves, a second sweep from cache where a gradient is written.
//   "group" : everything else. G = 64: a wavefront per row striding over its channels (layer norm
//             on long rows); G = 1: a lane per pixel for more than 512 channels in NCHW, channel
//             loop through the caches. Reductions inside a group use DPP/swizzle; nothing is
//             staged in LDS.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "../../include/pytorch_loss_hip.h"

namespace plh {

constexpr int kWave = 64;

// ---- argument checks shared by the entry points -----------------------------

inline bool misaligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) != 0; }

// Largest element count the kernels index (64-bit offsets are used throughout;
// the bound keeps every intermediate product well inside int64).
constexpr int64_t kMaxNumel = (int64_t)1 << 40;

inline int check_launch() {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? PLH_OK : (int)e;
}

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
__device__ __forceinline__ int64_t ceil_div_dev(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Checks for the (n_size, dimsize, m_size) entry points. `out` is the tensor written.
inline int check_slice_args(const void *logits, const void *labels, const void *out,
                            int64_t n_size, int64_t dimsize, int64_t m_size, size_t logits_elem = 4,
                            size_t out_elem = 4) {
    if (n_size < 0 || dimsize < 0 || m_size < 0) return PLH_ERR_BAD_SIZE;
    if (n_size > kMaxNumel || dimsize > kMaxNumel || m_size > kMaxNumel) return PLH_ERR_BAD_SIZE;
    if (dimsize > (int64_t)1 << 30) return PLH_ERR_BAD_SIZE;
    const double numel = (double)n_size * (double)dimsize * (double)m_size;
    if (numel > (double)kMaxNumel) return PLH_ERR_BAD_SIZE;
    if (numel == 0) return PLH_OK;
    if (!logits || !labels || !out) return PLH_ERR_NULL_POINTER;
    if (misaligned(logits, logits_elem) || misaligned(out, out_elem) || misaligned(labels, 8)) return PLH_ERR_MISALIGNED;
    return PLH_OK;
}

inline int check_gout(const void *gout, int64_t stride) {
    if (!gout) return PLH_OK;
    if (stride != 0 && stride != 1) return PLH_ERR_BAD_STRIDE;
    if (misaligned(gout, 4)) return PLH_ERR_MISALIGNED;
    return PLH_OK;
}

// Which execution shape serves a (dimsize, m_size) problem. The vector form of the regs shape
// moves V pixels per thread (2 for fp32 logits, 4 for 16-bit logits: 8 bytes per lane and channel
// either way); it needs m_size % V == 0 and every tensor aligned to its V-element access:
// `typed0/typed1` hold `elem`-byte elements (logits, gradient), `f32a/f32b` fp32 (losses, upstream
// gradient), labels int64. nullptr = tensor not used.
// Split: the regs shape with the channels of a pixel shared out over the 8 wavefronts of a block
// (see "the split launch shape" below); only for kernels that have that form (`with_split`).
// SplitDeep: the split shape with half the pixels per lane (4 bytes per lane and channel) and up to 64
// channel slots per wavefront, for 257..512 channels; only for kernels that have it (`with_deep`).
enum class Shape { RegsVec, RegsOne, Split, SplitImage, SplitDeep, Wave, Lane };

constexpr int kMaxRegsChannels = 32;
constexpr int kSplitWaves = 8;
constexpr int kMaxSplitChannels = kMaxRegsChannels * kSplitWaves;
constexpr int kMaxDeepSlots = 64;
constexpr int kMaxDeepChannels = kMaxDeepSlots * kSplitWaves;

inline Shape pick_shape(int64_t dimsize, int64_t m_size, int V, size_t elem, const void *typed0, const void *typed1,
                        const void *labels, const void *f32a, const void *f32b, bool with_split = false,
                        bool with_deep = false, bool with_image = false, int regs_image_max = 0) {
    auto fits = [&](int v) {
        return (m_size % v == 0) && !(typed0 && misaligned(typed0, v * elem)) &&
               !(typed1 && misaligned(typed1, v * elem)) && !(f32a && misaligned(f32a, v * 4)) &&
               !(f32b && misaligned(f32b, v * 4)) && !(labels && misaligned(labels, v > 1 ? 16 : 8));
    };
    bool vec = fits(V) && !(labels && misaligned(labels, 16));
    // Planes that do not start on 128-byte lines (1022 x 1022, 510 x 510) take the tiles-per-image forms as the
    // odd ones do, where the caller has them for this channel count: fp32 LSR fwd+bwd (8,19,1022,1022)
    // 0.433 -> 0.395 ms, (8,150,510,510) 0.947 -> 0.834 ms against 8-byte accesses whose runs straddle lines.
    if (with_image && m_size >= 4096 && (m_size * (int64_t)elem) % 128 != 0 &&
        (dimsize > kMaxRegsChannels || dimsize <= regs_image_max))
        vec = false;
    if (dimsize <= kMaxRegsChannels) return vec ? Shape::RegsVec : Shape::RegsOne;
    if (with_split && vec && dimsize <= kMaxSplitChannels && m_size >= 64) return Shape::Split;
    // planes that start on element boundaries only (odd lengths) and are long enough that the partly filled
    // last block of every image is a small share: the split shape in tiles per image
    if (with_image && !vec && dimsize <= kMaxSplitChannels && m_size >= 4096) return Shape::SplitImage;
    if (with_deep && dimsize > kMaxSplitChannels && dimsize <= kMaxDeepChannels && m_size >= 64 && fits(V / 2))
        return Shape::SplitDeep;
    return m_size == 1 ? Shape::Wave : Shape::Lane;
}

// Channel-loop unrolling of the group kernels: with one lane per pixel (G = 1) the loads of a loop are
// a channel plane apart, and unrolling keeps four of them in flight per lane.
template <int G> constexpr int kGroupUnroll = (G == 1) ? 4 : 1;

// Grid for the group kernels: they loop, so the grid is capped.
inline unsigned group_grid(int64_t pixels, int pixels_per_block) {
    const int64_t want = ceil_div(pixels, pixels_per_block);
    const int64_t cap = 256 * 64;   // 64 resident-or-queued blocks per CU
    return (unsigned)(want < cap ? (want > 0 ? want : 1) : cap);
}

// ---- element types -----------------------------------------------------------
// Logits and gradients may be fp32, fp16 or bf16 in memory; arithmetic is always fp32.
struct f16 { uint16_t bits; };
struct bf16 { uint16_t bits; };

template <class T> struct ElemTraits;
template <> struct ElemTraits<float> { static constexpr int kVec = 2; static constexpr int32_t kTag = PLH_DTYPE_F32; };
template <> struct ElemTraits<f16> { static constexpr int kVec = 4; static constexpr int32_t kTag = PLH_DTYPE_F16; };
template <> struct ElemTraits<bf16> { static constexpr int kVec = 4; static constexpr int32_t kTag = PLH_DTYPE_BF16; };

inline size_t dtype_size(int32_t dtype) { return dtype == PLH_DTYPE_F32 ? 4 : 2; }
inline bool dtype_ok(int32_t dtype) { return dtype == PLH_DTYPE_F32 || dtype == PLH_DTYPE_F16 || dtype == PLH_DTYPE_BF16; }

// Calls f(T{}) with the element type that `dtype` names.
template <class F>
inline int dispatch_dtype(int32_t dtype, F &&f) {
    switch (dtype) {
        case PLH_DTYPE_F32: f(float{}); return PLH_OK;
        case PLH_DTYPE_F16: f(f16{}); return PLH_OK;
        case PLH_DTYPE_BF16: f(bf16{}); return PLH_OK;
        default: return PLH_ERR_BAD_DTYPE;
    }
}

__device__ __forceinline__ float widen(uint16_t bits, f16) { return (float)__builtin_bit_cast(_Float16, bits); }
__device__ __forceinline__ float widen(uint16_t bits, bf16) { return __builtin_bit_cast(float, (uint32_t)bits << 16); }
__device__ __forceinline__ uint16_t narrow(float v, f16) { return __builtin_bit_cast(uint16_t, (_Float16)v); }
__device__ __forceinline__ uint16_t narrow(float v, bf16) {          // round to nearest even, NaN stays NaN
    const uint32_t u = __builtin_bit_cast(uint32_t, v);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

// ---- vector access -----------------------------------------------------------

// All tensors of this path are streamed exactly once, so loads and stores carry the
// non-temporal hint: lines are not kept in L2 / Infinity Cache at the expense of others.
typedef float plh_f2 __attribute__((ext_vector_type(2)));
typedef float plh_f4 __attribute__((ext_vector_type(4)));
typedef long long plh_l2 __attribute__((ext_vector_type(2)));

template <int V>
__device__ __forceinline__ void load_vec(const float *p, float (&out)[V]) {
    if constexpr (V == 1) {
        out[0] = __builtin_nontemporal_load(p);
    } else if constexpr (V == 2) {
        const plh_f2 t = __builtin_nontemporal_load(reinterpret_cast<const plh_f2 *>(p));
        out[0] = t.x; out[1] = t.y;
    } else {
        const plh_f4 t = __builtin_nontemporal_load(reinterpret_cast<const plh_f4 *>(p));
        out[0] = t.x; out[1] = t.y; out[2] = t.z; out[3] = t.w;
    }
}

template <int V>
__device__ __forceinline__ void store_vec(float *p, const float (&v)[V]) {
    if constexpr (V == 1) {
        __builtin_nontemporal_store(v[0], p);
    } else if constexpr (V == 2) {
        const plh_f2 t = {v[0], v[1]};
        __builtin_nontemporal_store(t, reinterpret_cast<plh_f2 *>(p));
    } else {
        const plh_f4 t = {v[0], v[1], v[2], v[3]};
        __builtin_nontemporal_store(t, reinterpret_cast<plh_f4 *>(p));
    }
}

// Same, with ordinary (cache-allocating) stores: for intermediates that the next kernel reads back
// and that are small enough for the last-level cache to keep.
template <int V>
__device__ __forceinline__ void store_vec_cached(float *p, const float (&v)[V]) {
    if constexpr (V == 1) {
        *p = v[0];
    } else if constexpr (V == 2) {
        *reinterpret_cast<plh_f2 *>(p) = plh_f2{v[0], v[1]};
    } else {
        *reinterpret_cast<plh_f4 *>(p) = plh_f4{v[0], v[1], v[2], v[3]};
    }
}

typedef unsigned short plh_h2 __attribute__((ext_vector_type(2)));
typedef unsigned short plh_h4 __attribute__((ext_vector_type(4)));

template <int V, class T>
__device__ __forceinline__ void load_vec(const T *p, float (&out)[V]) {      // T = f16 or bf16
    const unsigned short *q = reinterpret_cast<const unsigned short *>(p);
    if constexpr (V == 1) {
        out[0] = widen(__builtin_nontemporal_load(q), T{});
    } else if constexpr (V == 2) {
        const plh_h2 t = __builtin_nontemporal_load(reinterpret_cast<const plh_h2 *>(q));
        out[0] = widen(t.x, T{}); out[1] = widen(t.y, T{});
    } else {
        const plh_h4 t = __builtin_nontemporal_load(reinterpret_cast<const plh_h4 *>(q));
        out[0] = widen(t.x, T{}); out[1] = widen(t.y, T{}); out[2] = widen(t.z, T{}); out[3] = widen(t.w, T{});
    }
}

template <int V, class T>
__device__ __forceinline__ void store_vec(T *p, const float (&v)[V]) {       // T = f16 or bf16
    unsigned short *q = reinterpret_cast<unsigned short *>(p);
    if constexpr (V == 1) {
        __builtin_nontemporal_store(narrow(v[0], T{}), q);
    } else if constexpr (V == 2) {
        const plh_h2 t = {narrow(v[0], T{}), narrow(v[1], T{})};
        __builtin_nontemporal_store(t, reinterpret_cast<plh_h2 *>(q));
    } else {
        const plh_h4 t = {narrow(v[0], T{}), narrow(v[1], T{}), narrow(v[2], T{}), narrow(v[3], T{})};
        __builtin_nontemporal_store(t, reinterpret_cast<plh_h4 *>(q));
    }
}

// single elements, cached (the group kernels re-read what they have just touched)
__device__ __forceinline__ float load_one(const float *p) { return *p; }
__device__ __forceinline__ float load_one(const f16 *p) { return widen(p->bits, f16{}); }
__device__ __forceinline__ float load_one(const bf16 *p) { return widen(p->bits, bf16{}); }
__device__ __forceinline__ void store_one(float *p, float v) { *p = v; }
__device__ __forceinline__ void store_one(f16 *p, float v) { p->bits = narrow(v, f16{}); }
__device__ __forceinline__ void store_one(bf16 *p, float v) { p->bits = narrow(v, bf16{}); }

template <int V>
__device__ __forceinline__ void load_labels(const int64_t *p, int64_t (&out)[V]) {
    if constexpr (V == 1) {
        out[0] = __builtin_nontemporal_load(p);
    } else {
#pragma unroll
        for (int k = 0; k < V; k += 2) {
            const plh_l2 t = __builtin_nontemporal_load(reinterpret_cast<const plh_l2 *>(p + k));
            out[k] = t.x; out[k + 1] = t.y;
        }
    }
}

// ---- packed register form of a channel slice -------------------------------------
// The regs kernels keep what they loaded in the registers it arrived in (two dwords per channel
// for V = ElemTraits<T>::kVec pixels, one for V = 1) and widen to fp32 at the point of use, so a
// 16-bit slice costs half the registers of an fp32 one and the wavefront count per SIMD stays
// the same for every element type.
typedef unsigned plh_u2 __attribute__((ext_vector_type(2)));
typedef float plh_bf_src __attribute__((ext_vector_type(2)));
typedef __bf16 plh_bf2 __attribute__((ext_vector_type(2)));
typedef _Float16 plh_hf2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ unsigned f32_bits(float v) { return __builtin_bit_cast(unsigned, v); }
__device__ __forceinline__ float bits_f32(unsigned v) { return __builtin_bit_cast(float, v); }

template <class T, int V> struct Pack;
typedef unsigned plh_u2_a4 __attribute__((ext_vector_type(2), aligned(4)));
typedef float plh_f2_a4 __attribute__((ext_vector_type(2), aligned(4)));
typedef long long plh_l2_a8 __attribute__((ext_vector_type(2), aligned(8)));

template <> struct Pack<float, 2> {
    typedef plh_u2 Raw;
    static __device__ __forceinline__ Raw load(const float *p) {
        return __builtin_nontemporal_load(reinterpret_cast<const plh_u2 *>(p));
    }
    static __device__ __forceinline__ void store(float *p, Raw r) {
        __builtin_nontemporal_store(r, reinterpret_cast<plh_u2 *>(p));
    }
    // the same 8 bytes from any element boundary (tiles per image on channel planes of odd length)
    static __device__ __forceinline__ Raw load_unaligned(const float *p) {
        const plh_u2_a4 t = __builtin_nontemporal_load(reinterpret_cast<const plh_u2_a4 *>(p));
        return Raw{t.x, t.y};
    }
    static __device__ __forceinline__ void store_unaligned(float *p, Raw r) {
        __builtin_nontemporal_store(plh_u2_a4{r.x, r.y}, reinterpret_cast<plh_u2_a4 *>(p));
    }
    static __device__ __forceinline__ void store_unaligned_cached(float *p, Raw r) {
        *reinterpret_cast<plh_u2_a4 *>(p) = plh_u2_a4{r.x, r.y};
    }
    static __device__ __forceinline__ float get(Raw r, int k) { return bits_f32(k == 0 ? r.x : r.y); }
    static __device__ __forceinline__ Raw put(const float (&g)[2]) { return Raw{f32_bits(g[0]), f32_bits(g[1])}; }
    // In-place update: pixels [k, k + kStep) of a slice element are replaced by results. A kernel that
    // is done with the inputs of those pixels writes its outputs over them and needs no second array.
    static constexpr int kStep = 1;
    static __device__ __forceinline__ void set(Raw &r, int k, const float (&g)[1]) {
        if (k == 0) r.x = f32_bits(g[0]);
        else r.y = f32_bits(g[0]);
    }
    // AND-mask that clears pixel k of a packed gradient when keep[k] is 0 (keep[k] is 0 or ~0)
    static __device__ __forceinline__ Raw mask(const unsigned (&keep)[2]) { return Raw{keep[0], keep[1]}; }
};
// Four fp32 pixels per lane, for the per-image form of the regs shape (channel planes of odd length:
// a lane's 16 bytes start on a 4-byte boundary; the hardware takes such accesses, the types say so).
typedef unsigned plh_u4w __attribute__((ext_vector_type(4)));
typedef unsigned plh_u4w_a4 __attribute__((ext_vector_type(4), aligned(4)));
typedef unsigned plh_u4_a2 __attribute__((ext_vector_type(4), aligned(2)));
typedef float plh_f4_a4 __attribute__((ext_vector_type(4), aligned(4)));
template <> struct Pack<float, 4> {
    typedef plh_u4w Raw;
    static __device__ __forceinline__ Raw load(const float *p) {
        const plh_u4w_a4 t = __builtin_nontemporal_load(reinterpret_cast<const plh_u4w_a4 *>(p));
        return Raw{t.x, t.y, t.z, t.w};
    }
    static __device__ __forceinline__ void store(float *p, Raw r) {
        __builtin_nontemporal_store(plh_u4w_a4{r.x, r.y, r.z, r.w}, reinterpret_cast<plh_u4w_a4 *>(p));
    }
    static __device__ __forceinline__ Raw load_unaligned(const float *p) { return load(p); }
    static __device__ __forceinline__ void store_unaligned(float *p, Raw r) { store(p, r); }
    static __device__ __forceinline__ void store_unaligned_cached(float *p, Raw r) {
        *reinterpret_cast<plh_u4w_a4 *>(p) = plh_u4w_a4{r.x, r.y, r.z, r.w};
    }
    static __device__ __forceinline__ float get(Raw r, int k) { return bits_f32(k == 0 ? r.x : (k == 1 ? r.y : (k == 2 ? r.z : r.w))); }
    static __device__ __forceinline__ Raw put(const float (&g)[4]) {
        return Raw{f32_bits(g[0]), f32_bits(g[1]), f32_bits(g[2]), f32_bits(g[3])};
    }
    static constexpr int kStep = 1;
    static __device__ __forceinline__ void set(Raw &r, int k, const float (&g)[1]) {
        if (k == 0) r.x = f32_bits(g[0]);
        else if (k == 1) r.y = f32_bits(g[0]);
        else if (k == 2) r.z = f32_bits(g[0]);
        else r.w = f32_bits(g[0]);
    }
    static __device__ __forceinline__ Raw mask(const unsigned (&keep)[4]) { return Raw{keep[0], keep[1], keep[2], keep[3]}; }
};
template <> struct Pack<float, 1> {
    typedef unsigned Raw;
    static __device__ __forceinline__ Raw load(const float *p) {
        return __builtin_nontemporal_load(reinterpret_cast<const unsigned *>(p));
    }
    static __device__ __forceinline__ void store(float *p, Raw r) {
        __builtin_nontemporal_store(r, reinterpret_cast<unsigned *>(p));
    }
    static __device__ __forceinline__ float get(Raw r, int) { return bits_f32(r); }
    static __device__ __forceinline__ Raw put(const float (&g)[1]) { return f32_bits(g[0]); }
    static constexpr int kStep = 1;
    static __device__ __forceinline__ void set(Raw &r, int, const float (&g)[1]) { r = f32_bits(g[0]); }
    static __device__ __forceinline__ Raw mask(const unsigned (&keep)[1]) { return keep[0]; }
};

// fp32 -> 16-bit pairs, round to nearest even. bf16 uses the hardware v_cvt_pk_bf16_f32 of gfx950.
__device__ __forceinline__ unsigned narrow2(float a, float b, bf16) {
    return __builtin_bit_cast(unsigned, __builtin_convertvector(plh_bf_src{a, b}, plh_bf2));
}
__device__ __forceinline__ unsigned narrow2(float a, float b, f16) {
    return __builtin_bit_cast(unsigned, __builtin_convertvector(plh_bf_src{a, b}, plh_hf2));
}
__device__ __forceinline__ float widen_lo(unsigned d, bf16) { return bits_f32(d << 16); }
__device__ __forceinline__ float widen_hi(unsigned d, bf16) { return bits_f32(d & 0xFFFF0000u); }
__device__ __forceinline__ float widen_lo(unsigned d, f16) { return (float)__builtin_bit_cast(_Float16, (uint16_t)d); }
__device__ __forceinline__ float widen_hi(unsigned d, f16) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(d >> 16));
}

typedef unsigned plh_u2_a2 __attribute__((ext_vector_type(2), aligned(2)));
typedef unsigned plh_u1_a2 __attribute__((aligned(2)));
template <class T> struct Pack<T, 4> {          // T = f16 or bf16
    typedef plh_u2 Raw;
    static __device__ __forceinline__ Raw load(const T *p) {
        return __builtin_nontemporal_load(reinterpret_cast<const plh_u2 *>(p));
    }
    static __device__ __forceinline__ void store(T *p, Raw r) {
        __builtin_nontemporal_store(r, reinterpret_cast<plh_u2 *>(p));
    }
    // the same 8 bytes from any element boundary (the per-image form on channel planes of odd length)
    static __device__ __forceinline__ Raw load_unaligned(const T *p) {
        const plh_u2_a2 t = __builtin_nontemporal_load(reinterpret_cast<const plh_u2_a2 *>(p));
        return Raw{t.x, t.y};
    }
    static __device__ __forceinline__ void store_unaligned(T *p, Raw r) {
        __builtin_nontemporal_store(plh_u2_a2{r.x, r.y}, reinterpret_cast<plh_u2_a2 *>(p));
    }
    static __device__ __forceinline__ void store_unaligned_cached(T *p, Raw r) {
        *reinterpret_cast<plh_u2_a2 *>(p) = plh_u2_a2{r.x, r.y};
    }
    static __device__ __forceinline__ float get(Raw r, int k) {
        const unsigned d = k < 2 ? r.x : r.y;
        return (k & 1) ? widen_hi(d, T{}) : widen_lo(d, T{});
    }
    static __device__ __forceinline__ Raw put(const float (&g)[4]) {
        return Raw{narrow2(g[0], g[1], T{}), narrow2(g[2], g[3], T{})};
    }
    static constexpr int kStep = 2;              // a dword holds two pixels
    static __device__ __forceinline__ void set(Raw &r, int k, const float (&g)[2]) {
        if (k == 0) r.x = narrow2(g[0], g[1], T{});
        else r.y = narrow2(g[0], g[1], T{});
    }
    static __device__ __forceinline__ Raw mask(const unsigned (&keep)[4]) {
        return Raw{(keep[0] & 0xFFFFu) | (keep[1] & 0xFFFF0000u), (keep[2] & 0xFFFFu) | (keep[3] & 0xFFFF0000u)};
    }
};
template <class T> struct Pack<T, 2> {          // T = f16 or bf16: one dword, two pixels
    typedef unsigned Raw;
    static __device__ __forceinline__ Raw load(const T *p) {
        return __builtin_nontemporal_load(reinterpret_cast<const unsigned *>(p));
    }
    static __device__ __forceinline__ void store(T *p, Raw r) {
        __builtin_nontemporal_store(r, reinterpret_cast<unsigned *>(p));
    }
    // the same 4 bytes from any element boundary (the per-image form on channel planes of odd length)
    static __device__ __forceinline__ Raw load_unaligned(const T *p) {
        return __builtin_nontemporal_load(reinterpret_cast<const plh_u1_a2 *>(p));
    }
    static __device__ __forceinline__ void store_unaligned(T *p, Raw r) {
        __builtin_nontemporal_store((plh_u1_a2)r, reinterpret_cast<plh_u1_a2 *>(p));
    }
    static __device__ __forceinline__ float get(Raw r, int k) { return (k & 1) ? widen_hi(r, T{}) : widen_lo(r, T{}); }
    static __device__ __forceinline__ Raw put(const float (&g)[2]) { return narrow2(g[0], g[1], T{}); }
    static constexpr int kStep = 2;
    static __device__ __forceinline__ void set(Raw &r, int, const float (&g)[2]) { r = narrow2(g[0], g[1], T{}); }
    static __device__ __forceinline__ Raw mask(const unsigned (&keep)[2]) {
        return (keep[0] & 0xFFFFu) | (keep[1] & 0xFFFF0000u);
    }
};
template <class T> struct Pack<T, 1> {          // T = f16 or bf16
    typedef unsigned Raw;
    static __device__ __forceinline__ Raw load(const T *p) {
        return __builtin_nontemporal_load(reinterpret_cast<const unsigned short *>(p));
    }
    static __device__ __forceinline__ void store(T *p, Raw r) {
        __builtin_nontemporal_store((unsigned short)r, reinterpret_cast<unsigned short *>(p));
    }
    static __device__ __forceinline__ float get(Raw r, int) { return widen_lo(r, T{}); }
    static __device__ __forceinline__ Raw put(const float (&g)[1]) { return narrow2(g[0], 0.f, T{}) & 0xFFFFu; }
    static constexpr int kStep = 1;
    static __device__ __forceinline__ void set(Raw &r, int, const float (&g)[1]) { r = narrow2(g[0], 0.f, T{}) & 0xFFFFu; }
    static __device__ __forceinline__ Raw mask(const unsigned (&keep)[1]) { return keep[0]; }
};

// Makes a packed slice element opaque to the optimiser: what is computed from it afterwards is not
// merged with what was computed from it before (used between two sweeps over a register-resident
// slice, where keeping every first-sweep intermediate alive would cost far more registers than
// the second evaluation costs instructions).
__device__ __forceinline__ void forget_origin(unsigned &r) { asm volatile("" : "+v"(r)); }
__device__ __forceinline__ void forget_origin(plh_u2 &r) { asm volatile("" : "+v"(r.x), "+v"(r.y)); }
__device__ __forceinline__ void forget_origin(plh_u4w &r) { asm volatile("" : "+v"(r.x), "+v"(r.y), "+v"(r.z), "+v"(r.w)); }

// A regs kernel is instantiated for CP = channels rounded up to a multiple of 4, and launched only
// for CP-3 <= C <= CP: the first CP-3 channel slots always exist, the last three are checked.
template <int CP>
__device__ __forceinline__ bool chan_ok(int j, int C) { return j < CP - 3 || j < C; }

// max(a, b, c) in one instruction. Like fmaxf it returns the largest non-NaN operand; a NaN logit
// still reaches the result through the exponential sum.
__device__ __forceinline__ float max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// Widens pixel k of a packed slice into xv[] and returns the maximum over its channels.
template <class T, int V, int CP>
__device__ __forceinline__ float widen_and_max(const typename Pack<T, V>::Raw (&raw)[CP], int k, int C, float (&xv)[CP]) {
#pragma unroll
    for (int j = 0; j < CP; ++j)
        if (chan_ok<CP>(j, C)) xv[j] = Pack<T, V>::get(raw[j], k);
    float mx = xv[0];
#pragma unroll
    for (int j = 1; j + 1 < CP - 3; j += 2) mx = max3(mx, xv[j], xv[j + 1]);
#pragma unroll
    for (int j = CP - 3; j < CP; ++j)
        if (j > 0 && j < C) mx = max3(mx, xv[j], xv[j]);
    return mx;
}

constexpr float kLog2e = 1.44269504088896340736f;
constexpr float kLn2 = 0.69314718055994530942f;

// Upstream gradient of the fused entry points: value = gout[...] * scale / divide_by[0].
struct Upstream {
    const float *gout;          // nullptr = 1
    int64_t stride;             // 0 = one scalar, 1 = per loss element
    const int64_t *divide_by;   // nullptr = 1; device-resident count (e.g. the valid pixels of a 'mean')
    float scale;                // host-side factor
    const uint8_t *keep;        // nullptr = every pixel; else one byte per pixel, 0 = the pixel takes no part (its
                                // upstream gradient is 0): how the hard-example losses hand their selection on
};

// `have` = how many of the V pixels from i on exist (the per-image form's last lane of an image has fewer).
template <int V>
__device__ __forceinline__ void load_upstream(const Upstream &up, int64_t i, float (&out)[V], int have = V) {
    if (up.gout != nullptr && up.stride != 0) {
        load_vec<V>(up.gout + i, out);
        return;
    }
    float g = up.gout ? *up.gout * up.scale : up.scale;
    if (up.divide_by) g = g / (float)(*up.divide_by);
#pragma unroll
    for (int k = 0; k < V; ++k) out[k] = g;
    if (up.keep) {                  // uniform
#pragma unroll
        for (int k = 0; k < V; ++k)
            if (k < have && up.keep[i + k] == 0) out[k] = 0.f;
    }
}

// ---- two-stage deterministic reduction of the losses ------------------------------
// Stage 1: every block of a forward kernel writes one partial sum and one partial count.
// Stage 2: a single block adds them in a fixed order (double accumulation) and writes the
// sum or the mean. No floating-point atomics anywhere, so results are run-to-run identical.
struct Partials {
    float *sum;
    int *cnt;
};

enum FinishMode { kFinishSum = 0, kFinishMeanOverCount = 1, kFinishMeanOverFixed = 2 };

constexpr int64_t kMinPartialSlots = 16384;   // the looping kernels cap their grid at this many blocks

inline int64_t partial_slots(int64_t units) {
    // the smallest tile any reducing kernel gives a block: 64 pixels (deep split shape, fp32)
    const int64_t blocks = ceil_div(units > 0 ? units : 1, 64);
    return blocks > kMinPartialSlots ? blocks : kMinPartialSlots;
}

inline int carve_partials(void *workspace, int64_t workspace_bytes, int64_t units, const void *loss_out,
                          const void *n_valid_out, Partials &part) {
    if (!loss_out) return PLH_ERR_NULL_POINTER;
    if (misaligned(loss_out, 4) || misaligned(n_valid_out, 8)) return PLH_ERR_MISALIGNED;
    const int64_t slots = partial_slots(units);
    if (!workspace || misaligned(workspace, 16) || workspace_bytes < 8 * slots) return PLH_ERR_WORKSPACE;
    part.sum = static_cast<float *>(workspace);
    part.cnt = reinterpret_cast<int *>(static_cast<char *>(workspace) + 4 * slots);
    return PLH_OK;
}

// One 1024-thread block adds `blocks` partial sums (and counts) in a fixed order and writes the sum or the mean.
__device__ inline void finish_block(const float *__restrict__ sums, const int *__restrict__ cnts, unsigned blocks,
                                    float *__restrict__ loss_out, int64_t *__restrict__ count_out, int mode,
                                    int64_t fixed_count) {
    __shared__ double s_sum[1024];
    __shared__ long long s_cnt[1024];
    double acc = 0.0;
    long long cnt = 0;
    // eight partials per trip, loaded before the first is added: the trip count is small and each
    // trip would otherwise wait out a full memory round trip (the order of the additions stays fixed)
    unsigned i = threadIdx.x;
    for (; i + 7 * 1024 < blocks; i += 8 * 1024) {
        float v[8];
        int n[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            v[u] = sums[i + u * 1024];
            n[u] = cnts ? cnts[i + u * 1024] : 0;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            acc += (double)v[u];
            cnt += n[u];
        }
    }
    for (; i < blocks; i += 1024) {
        acc += (double)sums[i];
        if (cnts) cnt += cnts[i];
    }
    s_sum[threadIdx.x] = acc;
    s_cnt[threadIdx.x] = cnt;
    __syncthreads();
    for (int half = 512; half > 0; half >>= 1) {
        if ((int)threadIdx.x < half) {
            s_sum[threadIdx.x] += s_sum[threadIdx.x + half];
            s_cnt[threadIdx.x] += s_cnt[threadIdx.x + half];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        const float total = (float)s_sum[0];
        float out = total;
        // same arithmetic as `losses.sum() / n_valid` in fp32 (0/0 = NaN when nothing is valid)
        if (mode == kFinishMeanOverCount) out = total / (float)s_cnt[0];
        if (mode == kFinishMeanOverFixed) out = total / (float)fixed_count;
        *loss_out = out;
        if (count_out) *count_out = (int64_t)s_cnt[0];
    }
}

// Defined in reduce.hip.
void finish_partials(const Partials &part, unsigned blocks, float *loss_out, int64_t *count_out, FinishMode mode,
                     int64_t fixed_count, hipStream_t stream);

// Per block the number of labels other than `ignore`, as partials for finish_partials (the sums are zeros); returns the
// number of blocks. For a pass that needs the mean's divisor before it runs. Defined in reduce.hip.
unsigned count_valid_partials(const int64_t *labels, int64_t P, int64_t ignore, const Partials &part, hipStream_t stream);

// The number of labels other than `ignore`, added to *total (which an earlier launch on the stream has zeroed) by at
// most 256 atomics. Defined in reduce.hip.
void count_valid_total(const int64_t *labels, int64_t P, int64_t ignore, unsigned long long *total, hipStream_t stream);

// What the score pass of an OHEM loss forward (ohem.hip: the cross-entropy score kernel; the large-margin forward kernel
// that also writes scores) leaves besides scores and losses, for the case that the threshold
// rule decides the selection (at least n_min pixels score within the threshold, so "beyond the n_min lowest" holds
// for every pixel above it): the byte mask and the per-block sums of that rule, and per block the number of pixels
// whose score, capped at 1 like the selection's keys, lies within the threshold. The first histogram kernel adds those
// numbers up; when they reach n_min it raises kEarlyFlag in the selection's state and every later kernel of the
// selection returns at once (the finish then adds up these sums instead of the relabelling pass's).
struct OhemEarly {
    uint8_t *kept;      // [P]; nullptr: nothing of this is produced
    float *sum;         // [blocks of the score kernel]
    int *cnt;           // [blocks]
    int *below;         // [blocks]
    float thresh;
};

// One byte per pixel for this thread's V pixels (nv of them exist).
template <int V>
__device__ __forceinline__ void store_kept(uint8_t *kept, int64_t pix, int nv, const bool (&kp)[V]) {
    typedef unsigned short u16_a1 __attribute__((aligned(1)));
    typedef unsigned u32_a1 __attribute__((aligned(1)));
    if (nv == V && V == 2) {
        *reinterpret_cast<u16_a1 *>(kept + pix) = (unsigned short)((unsigned)kp[0] | ((unsigned)kp[V - 1] << 8));
    } else if (nv == V && V == 4) {
        *reinterpret_cast<u32_a1 *>(kept + pix) =
            (unsigned)kp[0] | ((unsigned)kp[1 % V] << 8) | ((unsigned)kp[2 % V] << 16) | ((unsigned)kp[3 % V] << 24);
    } else {
#pragma unroll
        for (int k = 0; k < V; ++k)
            if (k < nv) kept[pix + k] = kp[k] ? 1 : 0;
    }
}

// Defined in lmargin.hip: plh_lmargin_forward that also writes each pixel's softmax probability at
// its label (1 where there is no target) into `scores`.
int lmargin_forward_with_scores(const void *logits, int32_t dtype, const int64_t *labels, float *losses, float *scores,
                                int64_t n_size, int64_t dimsize, int64_t m_size, int64_t ignore_index, float lam,
                                hipStream_t stream, float no_target_score = 1.f, const OhemEarly *early = nullptr,
                                unsigned *early_blocks = nullptr);

// ---- the "regs" launch shape ---------------------------------------------------
// 256 threads per block, V pixels per thread; block b of the grid owns the pixel tile
// tile_of_block(run). Hardware hands consecutive workgroup ids to the 8 XCDs round-robin; the
// tile order is permuted so that each XCD walks runs of `run` consecutive tiles: every XCD
// (own L2, own slice of the fabric) then streams contiguous address ranges per tensor instead
// of every eighth tile of all of them. The run length is chosen on the host (xcd_run_for).
constexpr int kRegsBlock = 256;
constexpr int kXcds = 8;

// Run length (in tiles) of the permutation; see xcd_run_for() for how the host picks it.
__device__ __forceinline__ int64_t tile_of_block(unsigned run) {
    const unsigned b = blockIdx.x;
    const unsigned span = kXcds * run;
    const unsigned sup = b / span, in = b % span;
    if ((sup + 1) * span <= gridDim.x) return (int64_t)sup * span + (in % kXcds) * run + in / kXcds;
    return b;   // ragged tail of the grid keeps its natural order
}

// Defined in api.hip.
unsigned xcd_run_for(size_t elem_bytes, int64_t m_size);

// Raw buffer descriptor over [p, p + 4 GiB): no stride, no swizzle, 32-bit data format.
constexpr int kBufferNT = 2;      // non-temporal hint of buffer loads / stores
__device__ __forceinline__ __amdgpu_buffer_rsrc_t tile_rsrc(const void *p) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, -1, 0x00020000);
}

template <int V>
inline unsigned regs_grid(int64_t pixels) { return (unsigned)ceil_div(ceil_div(pixels, V), kRegsBlock); }

// Where a thread of a regs-shape kernel works. `base` is the element offset of (image n, channel 0,
// first pixel); channel j of the same pixels sits at base + j*m_size. Two forms:
//   Uniform  - m_size is a multiple of the tile (kRegsBlock*V pixels), so a tile never straddles two
//              images and the grid has no ragged end: the image index and the channel base are
//              block-uniform (one scalar division per block, scalar base + 32-bit lane offset
//              addressing) and no bounds check is needed. Power-of-two image sizes take this form.
//   general  - any m_size: per-thread 64-bit index arithmetic and a bounds check.
//   rows     - the general form with one pixel per thread when m_size == 1, i.e. (N, C) inputs (flattened
//              channels-last segmentation logits, classification): a lane's channels are contiguous and
//              neighbouring lanes sit C elements apart, so direct loads would touch 64 cache lines per
//              instruction. Instead a wavefront copies its 64 rows (one contiguous run of 64*C elements)
//              through LDS with consecutive lanes on consecutive addresses, and every lane then picks its
//              row out of LDS; stores go the same way back. The LDS index is skewed by one word per 32
//              (e + e/32), which keeps the row reads of 64 lanes off a common bank for every C.
__device__ __forceinline__ int rows_skew(int e) { return e + (e >> 5); }

typedef unsigned plh_u4 __attribute__((ext_vector_type(4)));

// 16 bytes of consecutive elements starting at element e (a multiple of 4 or 8, so the skew is the same
// for all of them) into / out of a skewed tile.
template <class Word>
__device__ __forceinline__ void rows_scatter16(Word *tile, int e, plh_u4 v) {
    Word *at = tile + rows_skew(e);
    const unsigned d[4] = {v.x, v.y, v.z, v.w};
    if constexpr (sizeof(Word) == 4) {
#pragma unroll
        for (int i = 0; i < 4; ++i) at[i] = d[i];
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            at[2 * i] = (Word)(d[i] & 0xFFFFu);
            at[2 * i + 1] = (Word)(d[i] >> 16);
        }
    }
}
template <class Word>
__device__ __forceinline__ plh_u4 rows_gather16(const Word *tile, int e) {
    const Word *at = tile + rows_skew(e);
    unsigned d[4];
    if constexpr (sizeof(Word) == 4) {
#pragma unroll
        for (int i = 0; i < 4; ++i) d[i] = at[i];
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) d[i] = (unsigned)at[2 * i] | ((unsigned)at[2 * i + 1] << 16);
    }
    return plh_u4{d[0], d[1], d[2], d[3]};
}

//   per image - (Form == kPerImage) tiles that never straddle two images whatever m_size is: the grid is
//              (images) x (tiles per image), a lane takes V consecutive pixels of ONE image and the last
//              lane of an image may hold fewer (`nv`); its accesses then go pixel by pixel, and the pixels
//              it does not have read as ignored. Channel planes of odd length (513 x 513, 769 x 769 crops)
//              start on element boundaries only, which would leave one pixel per lane and runs of 256 (fp32)
//              or 128 bytes (16-bit) that share their first and last cache line with a neighbour; V = 4 with
//              16-byte (fp32) or 8-byte (16-bit) accesses on element boundaries makes the runs 1 KiB and
//              512 bytes (the hardware takes such accesses; the vector types of Pack<T, 4> say so).
constexpr int kGeneral = 0, kUniform = 1, kPerImage = 2;

// Grid of the per-image form.
template <int V>
inline unsigned image_grid(int64_t n_size, int64_t m_size) {
    return (unsigned)(n_size * ceil_div(m_size, (int64_t)kRegsBlock * V));
}

// Where the host picks it over one pixel per lane: planes long enough that the partly filled last
// block of every image is a small share, and slices that four pixels per lane still keep in registers:
// 96 dwords for all the slices a kernel holds (a 16-bit slice takes half the registers of an fp32 one).
template <class T, int Slices = 1>
constexpr int kImageFormMaxChannels = (96 / (Slices * (int)sizeof(T)) < kMaxRegsChannels) ? 96 / (Slices * (int)sizeof(T)) : kMaxRegsChannels;
template <class T, int Slices = 1>
inline bool image_form_pays(int C, int64_t m_size) { return C <= kImageFormMaxChannels<T, Slices> && m_size >= 4096; }

template <int V, int Form>
struct PixelRef {
    static constexpr bool Uniform = (Form == kUniform);
    int64_t pix;        // first pixel of this thread (index into labels / losses)
    int64_t base;       // block-uniform part of the channel-0 offset (Uniform) or the whole of it
    unsigned lane_off;  // 32-bit per-thread part (Uniform), else 0
    bool live;
    int nv;             // per-image form: pixels this lane has (0..V); V in the other forms
    int64_t wave_first; // rows form: the first row of this wavefront, and how many of its 64 rows exist
    int rows_here;

    __device__ __forceinline__ PixelRef(int64_t P, int64_t m_size, int C, unsigned xcd_run) {
        nv = V;
        if constexpr (Form == kPerImage) {
            const int64_t tiles = ceil_div_dev(m_size, (int64_t)kRegsBlock * V);
            const int64_t b = tile_of_block(xcd_run);
            const int64_t n = b / tiles;                        // block-uniform
            const int64_t local = ((b - n * tiles) * kRegsBlock + threadIdx.x) * V;
            const int64_t left = m_size - local;
            nv = left >= V ? V : (left > 0 ? (int)left : 0);
            live = nv > 0;
            const int64_t safe = live ? local : 0;
            pix = n * m_size + safe;
            base = n * (int64_t)C * m_size + safe;
            lane_off = 0;
        } else if constexpr (Uniform) {
            const int64_t start = tile_of_block(xcd_run) * (kRegsBlock * V);
            const int64_t n = start / m_size;
            lane_off = threadIdx.x * V;
            base = start + n * (int64_t)(C - 1) * m_size;
            pix = start + lane_off;
            live = true;
        } else {
            const int64_t tile = tile_of_block(xcd_run);
            const int64_t want = (tile * kRegsBlock + threadIdx.x) * V;
            live = want < P;
            pix = live ? want : 0;
            const int64_t n = pix / m_size;
            base = pix + n * (int64_t)(C - 1) * m_size;
            lane_off = 0;
            if constexpr (V == 1) {
                wave_first = tile * kRegsBlock + (threadIdx.x & ~63u);
                const int64_t left = P - wave_first;
                rows_here = left < 0 ? 0 : (left > 64 ? 64 : (int)left);
            }
        }
    }
    // (N, C) input with more than one channel: the rows form
    static __device__ __forceinline__ bool rows_form(int C, int64_t m_size) { return V == 1 && Form == kGeneral && m_size == 1 && C > 1; }

    // Labels, per-pixel fp32 outputs and the upstream gradient of this thread's pixels. In the per-image
    // form a lane with fewer than V pixels goes pixel by pixel and reads `ignore` for those it lacks.
    __device__ __forceinline__ void labels(const int64_t *lab, int64_t ignore, int64_t (&lb)[V]) const {
        if constexpr (Form == kPerImage) {
            if (nv == V) {
#pragma unroll
                for (int k = 0; k < V; k += 2) {
                    const plh_l2_a8 t = __builtin_nontemporal_load(reinterpret_cast<const plh_l2_a8 *>(lab + pix + k));
                    lb[k] = t.x; lb[k + 1] = t.y;
                }
            } else {
#pragma unroll
                for (int k = 0; k < V; ++k) lb[k] = k < nv ? lab[pix + k] : ignore;
            }
        } else {
            load_labels<V>(lab + pix, lb);
        }
    }
    __device__ __forceinline__ void store_f32(float *out, const float (&v)[V]) const {
        if constexpr (Form == kPerImage) {
            if (nv == V) {
                __builtin_nontemporal_store(plh_f4_a4{v[0], v[1], v[2], v[3]}, reinterpret_cast<plh_f4_a4 *>(out + pix));
            } else {
#pragma unroll
                for (int k = 0; k < V; ++k)
                    if (k < nv) out[pix + k] = v[k];
            }
        } else {
            store_vec<V>(out + pix, v);
        }
    }
    // the same through the cache (an output that a later kernel of the same call reads)
    __device__ __forceinline__ void store_f32_cached(float *out, const float (&v)[V]) const {
        if constexpr (Form == kPerImage) {
            if (nv == V) {
                *reinterpret_cast<plh_f4_a4 *>(out + pix) = plh_f4_a4{v[0], v[1], v[2], v[3]};
            } else {
#pragma unroll
                for (int k = 0; k < V; ++k)
                    if (k < nv) out[pix + k] = v[k];
            }
        } else {
            store_vec_cached<V>(out + pix, v);
        }
    }
    __device__ __forceinline__ void upstream(const Upstream &up, float (&go)[V]) const {
        if constexpr (Form == kPerImage) {
            if (up.gout != nullptr && up.stride != 0) {
                if (nv == V) {
                    const plh_f4_a4 t = __builtin_nontemporal_load(reinterpret_cast<const plh_f4_a4 *>(up.gout + pix));
                    go[0] = t.x; go[1] = t.y; go[2] = t.z; go[3] = t.w;
                } else {
#pragma unroll
                    for (int k = 0; k < V; ++k) go[k] = k < nv ? up.gout[pix + k] : 0.f;
                }
                return;
            }
        }
        load_upstream<V>(up, pix, go, nv);
    }

    // A wavefront's tile holds 64 rows of the kernel's channel count, skewed: 5.3 KB for 20 fp32 channels rather than
    // the 8.5 KB of 32, so that LDS does not hold the blocks per CU below what the registers allow.
    template <class T, int CP>
    static __device__ __forceinline__ typename std::conditional<sizeof(T) == 4, unsigned, unsigned short>::type *rows_tile() {
        typedef typename std::conditional<sizeof(T) == 4, unsigned, unsigned short>::type Word;
        constexpr int kChan = CP < kMaxRegsChannels ? CP : kMaxRegsChannels;
        __shared__ __attribute__((aligned(16))) Word tile[kRegsBlock / 64][64 * kChan + 64 * kChan / 32 + 8];
        return tile[threadIdx.x >> 6];
    }
    template <class T, int CP>
    __device__ __forceinline__ void rows_load(const T *t, int C, unsigned (&raw)[CP]) const {
        typedef typename std::conditional<sizeof(T) == 4, unsigned, unsigned short>::type Word;
        Word *tile = rows_tile<T, CP>();
        const int lane = threadIdx.x & 63;
        const Word *src = reinterpret_cast<const Word *>(t) + wave_first * C;
        const int n = rows_here * C;
        // Rows of odd length need no skew (a stride of C words between the lanes' reads is conflict-free by itself):
        // the tile is then a plain copy of the 64 rows, written 16 bytes per lane and step as it arrives and read
        // with one instruction per element (a base per lane, the channel as the instruction's offset) - about a
        // third of the skewed form's instructions.
        const bool plain = (C & 1) && rows_here == 64 && (reinterpret_cast<uintptr_t>(t) & 15) == 0;   // wave-uniform
        if (plain) {
            constexpr int kPer = 16 / (int)sizeof(Word);
            const plh_u4 *src4 = reinterpret_cast<const plh_u4 *>(src);
            plh_u4 *tile4 = reinterpret_cast<plh_u4 *>(tile);
            const int groups = n / kPer;                    // 64*C elements are a whole number of 16-byte groups
            for (int g = lane; g < groups; g += 128) {
                const bool two = g + 64 < groups;
                const plh_u4 a = src4[g];
                const plh_u4 b = two ? src4[g + 64] : a;
                tile4[g] = a;
                if (two) tile4[g + 64] = b;
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            const Word *mine = tile + lane * C;
#pragma unroll
            for (int j = 0; j < CP; ++j)
                if (chan_ok<CP>(j, C)) raw[j] = mine[j];
            __builtin_amdgcn_wave_barrier();        // the tile is free again only when every lane has its row
            return;
        }
        if (rows_here == 64 && (reinterpret_cast<uintptr_t>(t) & 15) == 0) {
            // a full wavefront: 64*C elements from a 16-byte boundary on, moved 16 bytes per lane and step
            constexpr int kPer = 16 / (int)sizeof(Word);
            const plh_u4 *src4 = reinterpret_cast<const plh_u4 *>(src);
            const int groups = n / kPer;
            for (int g = lane; g < groups; g += 128) {
                const bool two = g + 64 < groups;
                const plh_u4 a = src4[g];
                const plh_u4 b = two ? src4[g + 64] : a;
                rows_scatter16<Word>(tile, g * kPer, a);
                if (two) rows_scatter16<Word>(tile, (g + 64) * kPer, b);
            }
        } else if (lane < rows_here) {
            // the lanes that are still here are the first rows_here of the wavefront (kernels may have let the others go)
            for (int e = lane; e < n; e += rows_here) tile[rows_skew(e)] = src[e];
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (chan_ok<CP>(j, C)) raw[j] = tile[rows_skew(lane * C + j)];
        __builtin_amdgcn_wave_barrier();        // the tile is free again only when every lane has its row
    }
    template <class T, int CP>
    __device__ __forceinline__ void rows_store(T *t, int C, const unsigned (&raw)[CP]) const {
        typedef typename std::conditional<sizeof(T) == 4, unsigned, unsigned short>::type Word;
        Word *tile = rows_tile<T, CP>();
        const int lane = threadIdx.x & 63;
        const bool plain = (C & 1) && rows_here == 64 && (reinterpret_cast<uintptr_t>(t) & 15) == 0;   // as in rows_load
        if (plain) {
            Word *mine = tile + lane * C;
#pragma unroll
            for (int j = 0; j < CP; ++j)
                if (chan_ok<CP>(j, C)) mine[j] = (Word)raw[j];
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            constexpr int kPer = 16 / (int)sizeof(Word);
            plh_u4 *dst4 = reinterpret_cast<plh_u4 *>(reinterpret_cast<Word *>(t) + wave_first * C);
            const plh_u4 *tile4 = reinterpret_cast<const plh_u4 *>(tile);
            const int groups = rows_here * C / kPer;
            for (int g = lane; g < groups; g += 64) __builtin_nontemporal_store(tile4[g], dst4 + g);
            __builtin_amdgcn_wave_barrier();
            return;
        }
#pragma unroll
        for (int j = 0; j < CP; ++j)
            if (chan_ok<CP>(j, C)) tile[rows_skew(lane * C + j)] = (Word)raw[j];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        Word *dst = reinterpret_cast<Word *>(t) + wave_first * C;
        const int n = rows_here * C;
        if (rows_here == 64 && (reinterpret_cast<uintptr_t>(t) & 15) == 0) {
            constexpr int kPer = 16 / (int)sizeof(Word);
            plh_u4 *dst4 = reinterpret_cast<plh_u4 *>(dst);
            const int groups = n / kPer;
            for (int g = lane; g < groups; g += 64)
                __builtin_nontemporal_store(rows_gather16<Word>(tile, g * kPer), dst4 + g);
        } else if (lane < rows_here) {
            for (int e = lane; e < n; e += rows_here) dst[e] = tile[rows_skew(e)];
        }
        __builtin_amdgcn_wave_barrier();
    }
    // address of channel j for this thread's pixels
    template <class T>
    __device__ __forceinline__ T *chan(T *t, int j, int64_t m_size) const {
        return (t + (base + (int64_t)j * m_size)) + lane_off;
    }

    // The channel slice of this thread's pixels, as loaded. The Uniform form addresses through a
    // buffer descriptor that starts at the tile (scalar registers), a per-lane byte offset that is
    // the same for every channel and a scalar channel offset: no vector ALU work per load or store.
    template <class T, int CP>
    __device__ __forceinline__ void load_slice(const T *t, int C, int64_t m_size,
                                               typename Pack<T, V>::Raw (&raw)[CP]) const {
        if constexpr (Uniform) {
            static_assert(V * sizeof(T) == 8, "uniform tiles move 8 bytes per lane and channel");
            const __amdgpu_buffer_rsrc_t rsrc = tile_rsrc(t + base);
            const unsigned row = (unsigned)m_size * (unsigned)sizeof(T);
#pragma unroll
            for (int j = 0; j < CP; ++j)
                if (chan_ok<CP>(j, C))
                    raw[j] = __builtin_amdgcn_raw_buffer_load_b64(rsrc, lane_off * (unsigned)sizeof(T), j * row, kBufferNT);
        } else {
            if constexpr (V == 1) {
                if (rows_form(C, m_size)) {         // kernel-uniform
                    rows_load<T, CP>(t, C, raw);
                    return;
                }
            }
            if constexpr (Form == kPerImage) {
                if (nv < V) {                       // the last lane of an image (or a lane beyond it: zeros)
#pragma unroll
                    for (int j = 0; j < CP; ++j)
                        if (chan_ok<CP>(j, C)) {
                            float one[V];
#pragma unroll
                            for (int k = 0; k < V; ++k) one[k] = k < nv ? load_one(chan(t, j, m_size) + k) : 0.f;
                            raw[j] = Pack<T, V>::put(one);
                        }
                    return;
                }
            }
#pragma unroll
            for (int j = 0; j < CP; ++j)
                if (chan_ok<CP>(j, C)) {
                    if constexpr (Form == kPerImage) raw[j] = Pack<T, V>::load_unaligned(chan(t, j, m_size));
                    else raw[j] = Pack<T, V>::load(chan(t, j, m_size));
                }
        }
    }
    template <class T, int CP>
    __device__ __forceinline__ void store_slice(T *t, int C, int64_t m_size,
                                                const typename Pack<T, V>::Raw (&raw)[CP]) const {
        if constexpr (Uniform) {
            const __amdgpu_buffer_rsrc_t rsrc = tile_rsrc(t + base);
            const unsigned row = (unsigned)m_size * (unsigned)sizeof(T);
#pragma unroll
            for (int j = 0; j < CP; ++j)
                if (chan_ok<CP>(j, C))
                    __builtin_amdgcn_raw_buffer_store_b64(raw[j], rsrc, lane_off * (unsigned)sizeof(T), j * row, kBufferNT);
        } else {
            if constexpr (V == 1) {
                if (rows_form(C, m_size)) {         // kernel-uniform
                    rows_store<T, CP>(t, C, raw);
                    return;
                }
            }
            if constexpr (Form == kPerImage) {
                if (nv < V) {
#pragma unroll
                    for (int j = 0; j < CP; ++j)
                        if (chan_ok<CP>(j, C)) {
#pragma unroll
                            for (int k = 0; k < V; ++k)
                                if (k < nv) store_one(chan(t, j, m_size) + k, Pack<T, V>::get(raw[j], k));
                        }
                    return;
                }
            }
#pragma unroll
            for (int j = 0; j < CP; ++j)
                if (chan_ok<CP>(j, C)) {
                    if constexpr (Form == kPerImage) Pack<T, V>::store_unaligned(chan(t, j, m_size), raw[j]);
                    else Pack<T, V>::store(chan(t, j, m_size), raw[j]);
                }
        }
    }
};

// Uniform tiles: m_size is a multiple of the tile, and the byte offset of the last channel slot
// inside one image (what the scalar channel offset of the buffer form has to hold) fits 31 bits.
inline bool tiles_are_uniform(int64_t m_size, int V, size_t elem) {
    return m_size % ((int64_t)kRegsBlock * V) == 0 && V * elem == 8 &&
           m_size * (int64_t)elem * kMaxRegsChannels < ((int64_t)1 << 31);
}

// ---- the "split" launch shape ---------------------------------------------------
// Channel dimensions of 33..256 in NCHW: the slice of a pixel no longer fits one thread's registers,
// so the 8 wavefronts of a 512-thread block share it. Lanes still run along the pixels (V per lane,
// 8 bytes per lane and channel), wavefront w keeps channels [w*KW, (w+1)*KW) in registers, and the
// per-wavefront softmax statistics of a pixel meet in LDS. Logits are read once, and every
// per-channel access of a wavefront is one contiguous run of 512 bytes, as in the regs shape.
constexpr int kSplitBlock = kWave * kSplitWaves;

template <int V>
inline unsigned split_grid(int64_t pixels) { return (unsigned)ceil_div(pixels, (int64_t)kWave * V); }

// Slots per wavefront for C channels: C/8 rounded up to a multiple of 4 (the kernels are instantiated
// for 8, 12, ..., 32 slots). Measured at 40 channels, fp32 LSR fwd+bwd at (8,40,512,512): 8 slots (5
// wavefronts hold channels) 0.193 ms, 5 slots (all 8 wavefronts) 0.221 ms, 12 / 16 / 20 slots 0.207 /
// 0.213 / 0.225 ms: neither fewer idle slots nor fewer wavefronts in the exchange through LDS pays.
#define PLH_SPLIT_SLOT_CASES \
    PLH_CASE(8) PLH_CASE(12) PLH_CASE(16) PLH_CASE(20) PLH_CASE(24) PLH_CASE(28) PLH_CASE(32)
inline int split_slots(int64_t dimsize) {
    const int per = (int)ceil_div(dimsize, kSplitWaves);
    const int kw = (per + 3) / 4 * 4;
    return kw < 8 ? 8 : kw;
}
// fp32 slices of 16 or 20 slots per wavefront (97..160 channels) take four pixels per lane in the tiles-per-image
// form of the LSR kernels: 1 KiB runs, 80 registers of slice. Measured fwd+bwd on (8,150,513,513): 0.951 -> 0.824 ms;
// with 8 slots (40 and 60 channels) it changed nothing or lost (0.282 -> 0.303 ms on (8,40,481,641)).
inline bool split_image_wide(int64_t dimsize) { return split_slots(dimsize) == 16 || split_slots(dimsize) == 20; }
// The deep form (257..512 channels): 40, 48, 56 or 64 slots per wavefront.
#define PLH_SPLIT_DEEP_CASES PLH_CASE(40) PLH_CASE(48) PLH_CASE(56) PLH_CASE(64)
inline int split_slots_deep(int64_t dimsize) {
    const int per = (int)ceil_div(dimsize, kSplitWaves);
    const int kw = (per + 7) / 8 * 8;
    return kw < 40 ? 40 : kw;
}

// `PerImage`: tiles that never straddle two images (grid = images x tiles per image, split_image_grid), for channel
// planes that start on element boundaries only (odd lengths: 513 x 513 crops with 150 classes): a lane's V pixels
// are moved with accesses of the same width from element boundaries, the last lane of an image may hold fewer
// (`nv`) and then goes pixel by pixel; the pixels it lacks read as ignored and are never stored.
template <int V>
inline unsigned split_image_grid(int64_t n_size, int64_t m_size) {
    return (unsigned)(n_size * ceil_div(m_size, (int64_t)kWave * V));
}

template <class T, int V, int KW, bool PerImage = false>
struct SplitSlice {
    int64_t pix;      // first of this lane's V pixels (0 for a lane beyond the end: it still loads, never stores)
    int64_t base;     // element offset of (image, channel 0, pix)
    int first;        // first channel of this wavefront
    int here;         // channels of this wavefront that exist (0..KW), wave-uniform
    int nv;           // pixels this lane has (V, or fewer in the last lane of an image)
    bool live;

    __device__ __forceinline__ SplitSlice(int64_t P, int64_t m_size, int C, unsigned xcd_run) {
        if constexpr (PerImage) {
            const int64_t tiles = ceil_div_dev(m_size, (int64_t)kWave * V);
            const int64_t b = tile_of_block(xcd_run);
            const int64_t n = b / tiles;                        // block-uniform
            const int64_t local = ((b - n * tiles) * kWave + (threadIdx.x & 63)) * V;
            const int64_t left = m_size - local;
            nv = left >= V ? V : (left > 0 ? (int)left : 0);
            live = nv > 0;
            const int64_t safe = live ? local : 0;
            pix = n * m_size + safe;
            base = n * (int64_t)C * m_size + safe;
        } else {
            const int64_t want = (tile_of_block(xcd_run) * kWave + (threadIdx.x & 63)) * V;
            live = want < P;
            nv = V;
            pix = live ? want : 0;
            const int64_t n = pix / m_size;
            base = pix + n * (int64_t)(C - 1) * m_size;
        }
        first = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)) * KW;
        const int left = C - first;
        here = left < 0 ? 0 : (left > KW ? KW : left);
    }
    // Slot i holds channel min(first + i, C - 1): a slot beyond the last channel repeats it, so that no
    // load sits behind a branch; what is computed from such a slot is masked by the caller (i < here).
    __device__ __forceinline__ void load(const T *t, int C, int64_t m_size, typename Pack<T, V>::Raw (&raw)[KW]) const {
        if constexpr (PerImage) {
            if (nv < V) {                           // the last lane of an image (or a lane beyond it: zeros)
#pragma unroll
                for (int i = 0; i < KW; ++i) {
                    const int j = (first + i < C) ? first + i : C - 1;
                    float one[V];
#pragma unroll
                    for (int k = 0; k < V; ++k) one[k] = k < nv ? load_one(t + (base + (int64_t)j * m_size) + k) : 0.f;
                    raw[i] = Pack<T, V>::put(one);
                }
                return;
            }
        }
#pragma unroll
        for (int i = 0; i < KW; ++i) {
            const int j = (first + i < C) ? first + i : C - 1;
            if constexpr (PerImage) raw[i] = Pack<T, V>::load_unaligned(t + (base + (int64_t)j * m_size));
            else raw[i] = Pack<T, V>::load(t + (base + (int64_t)j * m_size));
        }
    }
    __device__ __forceinline__ void store(T *t, int64_t m_size, const typename Pack<T, V>::Raw (&raw)[KW]) const {
        if constexpr (PerImage) {
            if (nv < V) {
#pragma unroll
                for (int i = 0; i < KW; ++i)
                    if (i < here) {
#pragma unroll
                        for (int k = 0; k < V; ++k)
                            if (k < nv) store_one(t + (base + (int64_t)(first + i) * m_size) + k, Pack<T, V>::get(raw[i], k));
                    }
                return;
            }
        }
#pragma unroll
        for (int i = 0; i < KW; ++i)
            if (i < here) {
                // through the cache: a run's first and last line are completed there by the neighbouring tiles'
                // blocks (non-temporal stores cost 3-15 % here: LSR fp32 (8,60,513,513) 0.369 against 0.339 ms)
                if constexpr (PerImage) Pack<T, V>::store_unaligned_cached(t + (base + (int64_t)(first + i) * m_size), raw[i]);
                else Pack<T, V>::store(t + (base + (int64_t)(first + i) * m_size), raw[i]);
            }
    }
    // Labels, per-pixel fp32 outputs and the upstream gradient of this lane's pixels.
    __device__ __forceinline__ void labels(const int64_t *lab, int64_t ignore, int64_t (&lb)[V]) const {
        if constexpr (PerImage) {
            if (nv == V) {
#pragma unroll
                for (int k = 0; k < V; k += 2) {
                    const plh_l2_a8 t = __builtin_nontemporal_load(reinterpret_cast<const plh_l2_a8 *>(lab + pix + k));
                    lb[k] = t.x; lb[k + 1] = t.y;
                }
            } else {
#pragma unroll
                for (int k = 0; k < V; ++k) lb[k] = k < nv ? lab[pix + k] : ignore;
            }
        } else {
            load_labels<V>(lab + pix, lb);
        }
    }
    template <bool Cached = false>
    __device__ __forceinline__ void store_f32(float *out, const float (&v)[V]) const {
        if constexpr (PerImage) {
            if (nv == V) {
#pragma unroll
                for (int k = 0; k < V; k += 2) {
                    if constexpr (Cached) *reinterpret_cast<plh_f2_a4 *>(out + pix + k) = plh_f2_a4{v[k], v[k + 1]};
                    else __builtin_nontemporal_store(plh_f2_a4{v[k], v[k + 1]}, reinterpret_cast<plh_f2_a4 *>(out + pix + k));
                }
            } else {
#pragma unroll
                for (int k = 0; k < V; ++k)
                    if (k < nv) out[pix + k] = v[k];
            }
        } else {
            if constexpr (Cached) store_vec_cached<V>(out + pix, v);
            else store_vec<V>(out + pix, v);
        }
    }
    __device__ __forceinline__ void upstream(const Upstream &up, float (&go)[V]) const {
        if constexpr (PerImage) {
            if (up.gout != nullptr && up.stride != 0) {
#pragma unroll
                for (int k = 0; k < V; ++k) go[k] = k < nv ? up.gout[pix + k] : 0.f;
                return;
            }
        }
        load_upstream<V>(up, pix, go, nv);
    }
};

// Channels that wavefront w of a split block holds.
__device__ __forceinline__ int split_count(int w, int KW, int C) {
    const int left = C - w * KW;
    return left < 0 ? 0 : (left > KW ? KW : left);
}

__device__ __forceinline__ float fast_log(float x) { return __builtin_amdgcn_logf(x) * 0.69314718055994530942f; }

// exp(x) for x <= 0 through the hardware exp2: 2 instructions instead of ~10. Relative
// error stays below 1e-6 for the arguments a max-subtracted softmax produces.
__device__ __forceinline__ float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896340736f); }

// Labels arrive as int64; inside a kernel only "which channel, if any" matters. Narrowing once
// per pixel turns the per-channel 64-bit compares into 32-bit ones. -1 = no target channel
// (ignored pixel, or a label outside [0, C), which the reference leaves undefined).
__device__ __forceinline__ int narrow_label(int64_t lb, int64_t ignore, int C, bool &ignored) {
    ignored = (lb == ignore);
    int tgt = (!ignored && lb >= 0 && lb < (int64_t)C) ? (int)lb : -1;
    asm("" : "+v"(tgt));      // opaque from here on: keeps the per-channel compares 32 bits wide
    return tgt;
}

// log(1 + e) for e in [0, 1]: alternating series below 1/32 (relative error < 2e-7), hardware
// log2 above (absolute error ~6e-8 on a value >= 0.03). Replaces log1pf (~25 instructions).
__device__ __forceinline__ float fast_log1p_unit(float e) {
    const float series = e * (1.f + e * (-0.5f + e * (0.33333334f + e * (-0.25f + e * 0.2f))));
    const float direct = __builtin_amdgcn_logf(1.f + e) * 0.69314718055994530942f;
    return (e < 0.03125f) ? series : direct;
}

// ---- wave64 reductions ---------------------------------------------------------
// Intra-row steps (16 lanes) are DPP moves folded into the VALU op, the 16<->16
// step is a ds_swizzle, the 32<->32 step a ds_bpermute. Every lane ends with the
// full result.

template <int Ctrl>
__device__ __forceinline__ float dpp_move(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
        0, __builtin_bit_cast(int, v), Ctrl, 0xF, 0xF, true));
}

__device__ __forceinline__ float swizzle_xor16(float v) {
    // bit-mode swizzle: and_mask 0x1F, or_mask 0, xor_mask 0x10
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));
}

__device__ __forceinline__ float bpermute_xor32(float v) {
    const int lane = __lane_id();
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(((lane ^ 32) << 2), __builtin_bit_cast(int, v)));
}

struct OpSum { __device__ __forceinline__ float operator()(float a, float b) const { return a + b; } };
struct OpMax { __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); } };

// Reduce over groups of G consecutive lanes (G = 1, 16, 32 or 64).
template <int G, class Op>
__device__ __forceinline__ float group_reduce(float v, Op op) {
    if constexpr (G >= 16) {
        v = op(v, dpp_move<0xB1>(v));    // quad_perm [1,0,3,2]
        v = op(v, dpp_move<0x4E>(v));    // quad_perm [2,3,0,1]
        v = op(v, dpp_move<0x141>(v));   // row_half_mirror
        v = op(v, dpp_move<0x140>(v));   // row_mirror
    }
    if constexpr (G >= 32) v = op(v, swizzle_xor16(v));
    if constexpr (G >= 64) v = op(v, bpermute_xor32(v));
    return v;
}

// Block-wide sum for 256-thread blocks (4 waves) through LDS, fixed order; every thread gets
// the result. All 256 threads must call it.
__device__ __forceinline__ float block_sum_256(float v, float *lds4) {
    v = group_reduce<64>(v, OpSum());
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) lds4[wave] = v;
    __syncthreads();
    const float r = (lds4[0] + lds4[1]) + (lds4[2] + lds4[3]);
    __syncthreads();
    return r;
}

// The forwards of the split shape end with one wavefront's worth of work per pixel of a lane (combine the 8
// wavefronts' statistics, a logarithm or two). Wavefront k of a block does that for pixel k of every lane, so the
// tail of a block is one pixel long instead of V (16-bit elements, V = 4: LSR forward (8,150,512,512) 0.164 -> 0.138 ms).
// PLH_SPLIT_MY_LABEL picks the label of that pixel (in the kernel's own body: handed to a function by reference, the
// array of labels ends up in scratch memory); split_block_partials forms the block's sum and count from the V
// finishing wavefronts (all of them call it, the others have left the kernel).
#define PLH_SPLIT_MY_LABEL(my_lb, lb, wave, V)                                   \
    int64_t my_lb = lb[0];                                                       \
    _Pragma("unroll") for (int k_ = 1; k_ < V; ++k_) my_lb = ((wave) == k_) ? lb[k_] : my_lb;
template <int V>
__device__ __forceinline__ void split_block_partials(float out, bool counted, int wave, int lane, Partials part) {
    __shared__ float fin[2][8];
    const float bs = group_reduce<64>(out, OpSum());
    const float bc = group_reduce<64>(counted ? 1.f : 0.f, OpSum());
    if (lane == 0) {
        fin[0][wave] = bs;
        fin[1][wave] = bc;
    }
    __syncthreads();                                // the V wavefronts that are still here
    if (threadIdx.x == 0) {
        float ts = fin[0][0], tc = fin[1][0];
#pragma unroll
        for (int k = 1; k < V; ++k) {
            ts += fin[0][k];
            tc += fin[1][k];
        }
        part.sum[blockIdx.x] = ts;
        part.cnt[blockIdx.x] = (int)tc;             // at most 256 per block: exact in fp32
    }
}

__device__ __forceinline__ float block_max_256(float v, float *lds4) {
    v = group_reduce<64>(v, OpMax());
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) lds4[wave] = v;
    __syncthreads();
    const float r = fmaxf(fmaxf(lds4[0], lds4[1]), fmaxf(lds4[2], lds4[3]));
    __syncthreads();
    return r;
}

// ---- 16-byte chunks of a contiguous row (4 fp32 or 8 16-bit elements) -------------------
template <class T> struct RowChunk;
template <> struct RowChunk<float> {
    static constexpr int kLen = 4;
    static __device__ __forceinline__ void load(const float *p, float (&v)[4]) {
        const plh_f4 t = *reinterpret_cast<const plh_f4 *>(p);
        v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    }
    static __device__ __forceinline__ void store(float *p, const float (&v)[4]) {
        __builtin_nontemporal_store(plh_f4{v[0], v[1], v[2], v[3]}, reinterpret_cast<plh_f4 *>(p));
    }
    static __device__ __forceinline__ void store_cached(float *p, const float (&v)[4]) {
        *reinterpret_cast<plh_f4 *>(p) = plh_f4{v[0], v[1], v[2], v[3]};
    }
};
template <class T> struct RowChunk {             // T = f16 or bf16
    static constexpr int kLen = 8;
    static __device__ __forceinline__ void load(const T *p, float (&v)[8]) {
        const plh_u4 t = *reinterpret_cast<const plh_u4 *>(p);
        const unsigned d[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = widen_lo(d[i], T{});
            v[2 * i + 1] = widen_hi(d[i], T{});
        }
    }
    static __device__ __forceinline__ void store(T *p, const float (&v)[8]) {
        const plh_u4 t = {narrow2(v[0], v[1], T{}), narrow2(v[2], v[3], T{}), narrow2(v[4], v[5], T{}),
                          narrow2(v[6], v[7], T{})};
        __builtin_nontemporal_store(t, reinterpret_cast<plh_u4 *>(p));
    }
    static __device__ __forceinline__ void store_cached(T *p, const float (&v)[8]) {
        *reinterpret_cast<plh_u4 *>(p) = plh_u4{narrow2(v[0], v[1], T{}), narrow2(v[2], v[3], T{}),
                                                 narrow2(v[4], v[5], T{}), narrow2(v[6], v[7], T{})};
    }
};

// ---- pieces of a contiguous row: L elements of 2 .. 16 bytes together, at an address aligned to their size ----
template <class T, int L> struct RowPiece {
    static_assert(L * sizeof(T) <= 16 && (L & (L - 1)) == 0, "pieces of 1, 2, 4 or 8 elements, 16 bytes at most");
    static __device__ __forceinline__ void load(const T *p, float (&v)[L]) {
        if constexpr (L == RowChunk<T>::kLen) {
            RowChunk<T>::load(p, v);
        } else if constexpr (L == 1) {
            v[0] = load_one(p);
        } else if constexpr (sizeof(T) == 4) {                   // two fp32
            const plh_f2 t = *reinterpret_cast<const plh_f2 *>(p);
            v[0] = t.x; v[1] = t.y;
        } else if constexpr (L == 2) {                           // two 16-bit elements: one dword
            const unsigned d = *reinterpret_cast<const unsigned *>(p);
            v[0] = widen_lo(d, T{}); v[1] = widen_hi(d, T{});
        } else {                                                 // four 16-bit elements
            const plh_u2 t = *reinterpret_cast<const plh_u2 *>(p);
            v[0] = widen_lo(t.x, T{}); v[1] = widen_hi(t.x, T{});
            v[2] = widen_lo(t.y, T{}); v[3] = widen_hi(t.y, T{});
        }
    }
    static __device__ __forceinline__ void store(T *p, const float (&v)[L]) {
        if constexpr (L == RowChunk<T>::kLen) {
            RowChunk<T>::store(p, v);
        } else if constexpr (L == 1) {
            store_one(p, v[0]);
        } else if constexpr (sizeof(T) == 4) {       // short pieces go through the cache: a wavefront's stores
            *reinterpret_cast<plh_f2 *>(p) = plh_f2{v[0], v[1]};         // of one step cover parts of lines, which
        } else if constexpr (L == 2) {                                   // the next steps complete there
            *reinterpret_cast<unsigned *>(p) = narrow2(v[0], v[1], T{});
        } else {
            *reinterpret_cast<plh_u2 *>(p) = plh_u2{narrow2(v[0], v[1], T{}), narrow2(v[2], v[3], T{})};
        }
    }
    // Cached: 16-byte pieces through the cache as well -- for short rows that end inside a line,
    // four to a wavefront: (1 M, 200) LSR backward fp32 0.370 -> 0.315 ms, bf16 0.201 -> 0.154 ms; with a wavefront
    // per row it made no difference. A compile-time choice: with both kinds of store in one kernel behind a
    // wave-uniform branch the aligned rows lost 10-15 %.
    template <bool Cached>
    static __device__ __forceinline__ void store(T *p, const float (&v)[L]) {
        if constexpr (L == RowChunk<T>::kLen && Cached) RowChunk<T>::store_cached(p, v);
        else store(p, v);
    }
};

// ---- a wavefront holds rows of an (N, C) input in registers --------------------------------
// G lanes share a row (G = 64: one row per wavefront; G = 16: four short rows per wavefront, so that a
// wavefront still has a few KB in flight), NI steps of G lanes, a piece of L elements per lane and step
// (16 bytes where the rows allow it; rows whose length in bytes is only a multiple of 8, 4 or 2 move in
// pieces of that size): a row is read once and every load of it is in flight before the first one is used.
template <class T, int NI, int L_, int G = 64>
struct WaveRow {
    static constexpr int L = L_;
    float v[NI][L];
    // `sub` = lane within the row's group; elements beyond the row read as -inf (and are never stored)
    __device__ __forceinline__ void load(const T *xs, int C, int sub) {
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int e0 = (sub + G * i) * L;
            const bool ok = e0 < C;                   // a row holds a whole number of pieces
            RowPiece<T, L>::load(xs + (ok ? e0 : 0), v[i]);
#pragma unroll
            for (int l = 0; l < L; ++l) v[i][l] = ok ? v[i][l] : -INFINITY;
        }
    }
    __device__ __forceinline__ float max() const {
        float m = -INFINITY;
#pragma unroll
        for (int i = 0; i < NI; ++i)
#pragma unroll
            for (int l = 0; l < L; ++l) m = fmaxf(m, v[i][l]);
        return group_reduce<G>(m, OpMax());
    }
};

// The rows a wavefront works on in one round of a kernel's loop: 64 / G of them, consecutive; a group
// past the last row repeats the last row and stores nothing.
template <int G>
struct WaveRowAt {
    static constexpr int kRowsPerWave = 64 / G;
    static constexpr int kRowsPerBlock = 4 * kRowsPerWave;          // 256-thread blocks
    int sub, grp;               // lane within its row's group, group within the wavefront
    int64_t start, stride;      // wave-uniform: first row of the wavefront's first round, rows per round of the grid
    __device__ __forceinline__ WaveRowAt() {
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
        sub = lane % G;
        grp = lane / G;
        start = ((int64_t)blockIdx.x * 4 + wave) * kRowsPerWave;
        stride = (int64_t)gridDim.x * kRowsPerBlock;
    }
};

// Results of a wavefront's short rows written as one run. With 16 lanes per row and pieces shorter than 16 bytes a
// step's stores are four separate segments of 32..128 bytes; the four rows of a round are contiguous in memory, so
// they are gathered in LDS (as stored: T) and leave as 16-byte pieces of one run of 4*C elements, whose lines are
// whole except the run's first and last.
template <class T, int L, int G, int NI>
struct WaveRowSpan {
    static constexpr bool kUse = (G == 16 && L < RowChunk<T>::kLen);
    static constexpr int kRows = 64 / G;
    static constexpr int kRowSlots = G * NI * L;         // the longest row this instance holds (a multiple of 16 elements)
    static __device__ __forceinline__ T *tile() {
        __shared__ __attribute__((aligned(16))) T buf[4][kUse ? kRows * kRowSlots : 8];
        return buf[threadIdx.x >> 6];
    }
    // the piece of step i of lane (grp, sub) into the tile
    static __device__ __forceinline__ void stage(T *tile, int C, int grp, int e0, const float (&g)[L]) {
        T *at = tile + grp * C + e0;
        if constexpr (sizeof(T) == 4) {
#pragma unroll
            for (int l = 0; l < L; ++l) reinterpret_cast<float *>(at)[l] = g[l];
        } else if constexpr (L == 1) {
            store_one(at, g[0]);
        } else {
#pragma unroll
            for (int l = 0; l < L; l += 2) *reinterpret_cast<unsigned *>(at + l) = narrow2(g[l], g[l + 1], T{});
        }
    }
    // the rows of the round (`rows` of them, from `dst` on) out of the tile; all 64 lanes call it
    static __device__ __forceinline__ void flush(const T *tile, T *dst, int rows, int C) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        constexpr int kPer = 16 / (int)sizeof(T);
        typedef typename std::conditional<sizeof(T) == 4, plh_u4w_a4, plh_u4_a2>::type Piece;   // 16 bytes from an element boundary
        const int lane = threadIdx.x & 63, n = rows * C;
        const plh_u4 *tile4 = reinterpret_cast<const plh_u4 *>(tile);
        for (int c = lane; c < n / kPer; c += 64) {
            const plh_u4 v = tile4[c];
            __builtin_nontemporal_store(Piece{v.x, v.y, v.z, v.w}, reinterpret_cast<Piece *>(dst + c * kPer));
        }
        const int done = n / kPer * kPer;
        if (lane < n - done) dst[done + lane] = tile[done + lane];
        __builtin_amdgcn_wave_barrier();        // the tile is free again only when every lane has read its pieces
    }
};

// Lanes per row, piece length and steps for a row of C elements. Rows of up to 256 elements get 16 lanes,
// longer ones a whole wavefront. The piece is the largest of 16, 8, 4, 2 bytes that divides the row's bytes
// and that every tensor involved is aligned to. Instantiated steps -- 16 lanes: 4, 8, 16 single elements,
// 2, 4, 8 pieces of two, 2, 4 of four, 2 of eight; 64 lanes: 8, 16, 32 single elements, 4, 8, 16 pieces of
// two, 2, 4, 8 of four or eight. Rows of 257..512 elements also get 16 lanes (32 slots per lane: 4 steps of eight,
// 8 of four, 16 of two or 32 single elements; a whole wavefront per row takes a power-of-two number of steps, and for
// 528 bytes it left the bf16 LSR backward at 39 % of peak).
constexpr int kWaveRowCap = 2048;       // 32 steps of 64 lanes, one element each
constexpr int kWaveRowShort = 256;

// Geometry of the backwards that walk every channel plane in its own cache lines (lsr_bwd_planes, taylor_ce_bwd_planes):
// a lane moves 16 bytes (4 fp32 or 8 16-bit elements), a line holds kLine elements, a block's tile is 256 lanes' worth
// of pixels and the stage holds one line's worth of pixels before it. PlanePixel: what is staged per pixel.
template <class T> struct PlaneGeom {
    static constexpr int kPer = 16 / (int)sizeof(T), kLine = 128 / (int)sizeof(T), kTile = 256 * kPer, kHalo = kLine;
};
struct PlanePixel {
    float lse;          // LSR: the pixel's log-sum-exp; Taylor cross entropy: the upstream gradient over the pixel's S
    int lab;            // the label, -1 for a pixel that takes no part, C for one without a target channel
};

// Which (N, C) rows of LSR and Taylor cross entropy take the backward that is elementwise over the flattened tensor, from
// one value per row that the forward leaves, instead of the one that holds the row in registers and recomputes. The
// elementwise backward runs at 75-79 % of the HBM peak on fp32 rows of any length (1 GiB of logits; 80-90 % on 256 MiB),
// the recomputing one at 55-72 % (70-88 %), best on rows of a multiple of 32 classes from 96 to 768, which stay with it.
// 16-bit rows: the elementwise backward pays up to 96 classes (bf16 (1048576,64) 0.085 -> 0.043 ms) and beyond
// `long_16bit` classes (1024 for both: LSR bf16 (244032,1100) 0.264 -> 0.196 ms, Taylor (209715,1280) 0.205 -> 0.173), and
// only on rows of whole 16-byte chunks among the short ones; between, the recomputing kernels are as fast or faster
// (bf16 (1048576,256) 0.187 / 0.191).
inline bool row_backward_is_elementwise(size_t elem_bytes, int64_t dimsize, int64_t long_16bit) {
    if (dimsize <= 32) return false;            // the register-resident kernels' rows
    if (elem_bytes == 4) return !(dimsize % 32 == 0 && dimsize >= 96 && dimsize <= 768);
    return dimsize > long_16bit || (dimsize % 8 == 0 && dimsize <= 96);
}
// 16-bit rows that move in 16-byte pieces go up to 4096 elements (8 steps of 64 lanes, 8 elements each: the
// same 64 registers as an fp32 row of 2048); a block per row spends most of such a short row's time in its
// barriers (bf16 LSR forward at (65536, 4096): 45 % of peak).
// 16-byte chunks per thread of the elementwise backwards over flattened rows (lsr_bwd_flat_lse, lm_bwd_flat_saved)
constexpr int kFlatChunks = 2;

template <class T>
inline int wrow_cap(int piece) { return piece == 8 ? 2 * kWaveRowCap : kWaveRowCap; }


template <class T>
static int wrow_piece(const T *x, const T *second, int C, const T *third = nullptr) {
    int len = RowChunk<T>::kLen;
    while (len > 1 && (C % len != 0 || misaligned(x, len * sizeof(T)) || (second && misaligned(second, len * sizeof(T))) ||
                       (third && misaligned(third, len * sizeof(T)))))
        len /= 2;
    return len;
}
template <class T>
static int wrow_steps(int C, int piece, int lanes) {
    const int per = lanes * piece;
    const int need = (C + per - 1) / per;
    int steps = piece == 1 ? (lanes == 16 ? 4 : 8) : (piece == 2 && lanes == 64 ? 4 : 2);   // the smallest instantiated sizes
    while (steps < need) steps *= 2;
    // 129..160 elements in short pieces (150 classes, channels last) would fill 5 of 8 or 10 of 16 steps: they have
    // instances of their own
    if (lanes == 16 && piece == 2 && need == 5) return 5;
    if (lanes == 16 && piece == 1 && (need == 9 || need == 10)) return 10;
    return steps;
}
// Kernels that write a row of results have a second instance for short rows in 16-byte pieces whose ends fall inside
// 128-byte lines (RowPiece::store<true>): which (piece, lanes) have it, and which rows take it.
template <class T>
constexpr bool wrow_cached_form(int piece, int lanes) { return lanes == 16 && piece == RowChunk<T>::kLen; }
template <class T>
inline bool wrow_rows_end_inside_lines(int C) { return (C * (int)sizeof(T)) % 128 != 0; }
// LAUNCH(NI, L, G) launches the kernel instance; its grid is group_grid(rows, WaveRowAt<G>::kRowsPerBlock).
#define PLH_WROW_STEPS3(PIECE, LANES, C, A, B, D, LAUNCH)                                \
    switch (wrow_steps<T>(C, PIECE, LANES)) {                                            \
        case A: LAUNCH(A, PIECE, LANES); break;                                          \
        case B: LAUNCH(B, PIECE, LANES); break;                                          \
        default: LAUNCH(D, PIECE, LANES); break;                                         \
    }
// WIDE_SHORT (a constant expression): which rows of 257..512 elements in pieces shorter than 16 bytes take the 16-lane
// form too -- 2: all (the forwards), 1: not those of single elements (kernels that write a row: 32 staged steps per
// lane lose to the wavefront per row, bf16 (512 K, 301) large-margin backward 0.255 -> 0.363 ms), 0: none (the Taylor
// backwards: bf16 (512 K, 300) cross-entropy backward 0.255 -> 0.293 ms with it).
#define PLH_WROW_DISPATCH(PIECE, C, LAUNCH) PLH_WROW_DISPATCH_IF(PIECE, C, LAUNCH, 2)
#define PLH_WROW_DISPATCH_IF(PIECE, C, LAUNCH, WIDE_SHORT)                               \
    do {                                                                                 \
        const int wrow_len = (PIECE);                                                    \
        if ((C) > kWaveRowShort && (C) <= 2 * kWaveRowShort) {                           \
            if (wrow_len == RowChunk<T>::kLen) {                                         \
                if constexpr (RowChunk<T>::kLen == 8) LAUNCH(4, 8, 16);                  \
                else LAUNCH(8, 4, 16);                                                   \
                break;                                                                   \
            }                                                                            \
            if constexpr ((WIDE_SHORT) == 2) {                                           \
                if (wrow_len == 1) {                                                     \
                    LAUNCH(32, 1, 16);                                                   \
                    break;                                                               \
                }                                                                        \
            }                                                                            \
            if constexpr ((WIDE_SHORT) >= 1) {                                           \
                if (wrow_len == 2) {                                                     \
                    LAUNCH(16, 2, 16);                                                   \
                    break;                                                               \
                }                                                                        \
                if constexpr (RowChunk<T>::kLen == 8) {                                  \
                    if (wrow_len == 4) {                                                 \
                        LAUNCH(8, 4, 16);                                                \
                        break;                                                           \
                    }                                                                    \
                }                                                                        \
            }                                                                            \
        }                                                                                \
        if ((C) <= kWaveRowShort) {                                                      \
            if (wrow_len == 1) {                                                         \
                if (wrow_steps<T>(C, 1, 16) == 10) LAUNCH(10, 1, 16);                    \
                else { PLH_WROW_STEPS3(1, 16, C, 4, 8, 16, LAUNCH) }                     \
            } else if (wrow_len == 2) {                                                  \
                if (wrow_steps<T>(C, 2, 16) == 5) LAUNCH(5, 2, 16);                      \
                else { PLH_WROW_STEPS3(2, 16, C, 2, 4, 8, LAUNCH) }                      \
            }                                                                            \
            else if (wrow_len == 4) { PLH_WROW_STEPS3(4, 16, C, 2, 4, 4, LAUNCH) }       \
            else if constexpr (RowChunk<T>::kLen == 8) { LAUNCH(2, 8, 16); }             \
        } else {                                                                         \
            if (wrow_len == 1) { PLH_WROW_STEPS3(1, 64, C, 8, 16, 32, LAUNCH) }          \
            else if (wrow_len == 2) { PLH_WROW_STEPS3(2, 64, C, 4, 8, 16, LAUNCH) }      \
            else if (wrow_len == 4) { PLH_WROW_STEPS3(4, 64, C, 2, 4, 8, LAUNCH) }       \
            else if constexpr (RowChunk<T>::kLen == 8) { PLH_WROW_STEPS3(8, 64, C, 2, 4, 8, LAUNCH) } \
        }                                                                                \
    } while (0)

// ---- a block per row: rows longer than a wavefront's registers (a vocabulary) ------------------
// One block of 1024 (or, for shorter rows, 256) threads per row at a time, 16-byte loads, four of them in flight per lane, and running
// per-lane statistics that are rescaled when the maximum moves, so a sweep reads the row once.
constexpr int kRowBlock = 1024;      // long rows: few, large blocks, so that the rows in flight stay within the
                                     // last-level cache for the backward's second sweep
constexpr int kRowBlockShort = 256;  // rows of up to kRowShortMax elements: more rows in flight, four chunks per
constexpr int kRowShortMax = 24576;  // lane where there was one, a quarter of the wavefronts in every barrier.
                                     // Measured fp32 LSR fwd+bwd, 256 against 1024 threads: (16384, 4096) 0.153 / 0.223 ms,
                                     // (8192, 16384) 0.339 / 0.355, (4096, 21841) 0.230 / 0.228, (8192, 32000) 0.679 / 0.605
inline int row_threads_for(int C, int short_max = kRowShortMax) { return C <= short_max ? kRowBlockShort : kRowBlock; }
// The same limit for a forward sweep, by the bytes of a row (112 KiB): what decides is how long a block's loads are
// in flight against the reduction that follows them, and a 16-bit row of 32000 or 50257 elements is a short one.
// Measured bf16 forward, 256 against 1024 threads: LSR (8192, 32000) 0.106 / 0.142 ms, (4096, 50257) 0.085 / 0.091,
// (2048, 128256) 0.106 / 0.100; Taylor cross entropy (8192, 32000) 0.113 / 0.164 (its backward 0.263 / 0.420).
template <class T>
inline int row_threads_for_sweep(int C) { return (int64_t)C * (int64_t)sizeof(T) <= 112 * 1024 ? kRowBlockShort : kRowBlock; }
__device__ __forceinline__ int row_threads() { return (int)blockDim.x; }      // either of the two

struct RowStats { float m, s, sx; };

// Block-wide reductions over the block's threads; every thread gets the result. lds: kRowBlock / 64 floats.
template <class Op>
__device__ __forceinline__ float row_block_reduce(float v, float *lds, Op op) {
    v = group_reduce<64>(v, op);
    if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = v;
    __syncthreads();
    float r = lds[0];
    for (int w = 1; w < row_threads() / 64; ++w) r = op(r, lds[w]);
    __syncthreads();
    return r;
}

template <int L>
__device__ __forceinline__ void row_absorb(const float (&v)[L], RowStats &st) {
    float cm = v[0];
#pragma unroll
    for (int i = 1; i < L; ++i) cm = fmaxf(cm, v[i]);
    if (cm > st.m) {
        st.s *= fast_exp(st.m - cm);               // 0 * exp(-inf) on the first chunk
        st.m = cm;
    }
    // while everything seen so far is -inf (masked vocabulary entries) the terms are exp(-inf - 0) = 0,
    // not exp(-inf + inf) = NaN
    const float ref = (st.m == -INFINITY) ? 0.f : st.m;
#pragma unroll
    for (int i = 0; i < L; ++i) {
        st.s += fast_exp(v[i] - ref);
        st.sx += v[i];
    }
}

// How a row splits into 16-byte chunks: `head` leading elements up to the first 16-byte boundary,
// `chunks` chunks, then the rest. Rows of any length qualify as long as the tensor itself starts on a
// 16-byte boundary (`aligned`); otherwise the whole row is the head.
template <class T>
struct RowSplit {
    int head, chunks, tail_from;
    __device__ __forceinline__ RowSplit(const T *xs, int C, bool aligned) {
        constexpr int L = RowChunk<T>::kLen;
        const int mis = (int)((reinterpret_cast<uintptr_t>(xs) / sizeof(T)) % L);
        const int lead = (L - mis) % L;
        head = aligned ? (lead < C ? lead : C) : C;
        chunks = (C - head) / L;
        tail_from = head + chunks * L;
    }
};

template <class T>
__device__ __forceinline__ RowStats row_sweep(const T *xs, int C, bool aligned) {
    constexpr int L = RowChunk<T>::kLen;
    const RowSplit<T> sp(xs, C, aligned);
    RowStats st{-INFINITY, 0.f, 0.f};
    const T *body = xs + sp.head;
    int i = threadIdx.x;
    for (; i + 3 * row_threads() < sp.chunks; i += 4 * row_threads()) {
        float v[4][L];
#pragma unroll
        for (int u = 0; u < 4; ++u) RowChunk<T>::load(body + (int64_t)(i + u * row_threads()) * L, v[u]);
#pragma unroll
        for (int u = 0; u < 4; ++u) row_absorb<L>(v[u], st);
    }
    for (; i < sp.chunks; i += row_threads()) {
        float v[L];
        RowChunk<T>::load(body + (int64_t)i * L, v);
        row_absorb<L>(v, st);
    }
    // head and tail, element by element (the whole row when it cannot be moved in chunks)
    for (int j = threadIdx.x; j < sp.head; j += row_threads()) {
        const float v[1] = {load_one(xs + j)};
        row_absorb<1>(v, st);
    }
    for (int j = sp.tail_from + threadIdx.x; j < C; j += row_threads()) {
        const float v[1] = {load_one(xs + j)};
        row_absorb<1>(v, st);
    }
    return st;
}

// Calls fn(value, index) for this thread's share of a row: chunks of 16 bytes, four loads in flight,
// then the head and tail element by element.
template <class T, class Fn>
__device__ __forceinline__ void row_visit(const T *xs, int C, bool aligned, Fn fn) {
    constexpr int L = RowChunk<T>::kLen;
    const RowSplit<T> sp(xs, C, aligned);
    const T *body = xs + sp.head;
    int i = threadIdx.x;
    for (; i + 3 * row_threads() < sp.chunks; i += 4 * row_threads()) {
        float v[4][L];
#pragma unroll
        for (int u = 0; u < 4; ++u) RowChunk<T>::load(body + (int64_t)(i + u * row_threads()) * L, v[u]);
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int e = 0; e < L; ++e) fn(v[u][e], sp.head + (i + u * row_threads()) * L + e);
    }
    for (; i < sp.chunks; i += row_threads()) {
        float v[L];
        RowChunk<T>::load(body + (int64_t)i * L, v);
#pragma unroll
        for (int e = 0; e < L; ++e) fn(v[e], sp.head + i * L + e);
    }
    for (int j = threadIdx.x; j < sp.head; j += row_threads()) fn(load_one(xs + j), j);
    for (int j = sp.tail_from + threadIdx.x; j < C; j += row_threads()) fn(load_one(xs + j), j);
}

// Writes fn(value, index) over a row of `out` that sits at the same offset from a 16-byte boundary as `xs`.
template <class T, class Fn>
__device__ __forceinline__ void row_map(const T *xs, T *out, int C, bool aligned, Fn fn) {
    constexpr int L = RowChunk<T>::kLen;
    const RowSplit<T> sp(xs, C, aligned);
    for (int i = threadIdx.x; i < sp.chunks; i += row_threads()) {
        float v[L];
        RowChunk<T>::load(xs + sp.head + (int64_t)i * L, v);
#pragma unroll
        for (int e = 0; e < L; ++e) v[e] = fn(v[e], sp.head + i * L + e);
        RowChunk<T>::store(out + sp.head + (int64_t)i * L, v);
    }
    for (int j = threadIdx.x; j < sp.head; j += row_threads()) store_one(out + j, fn(load_one(xs + j), j));
    for (int j = sp.tail_from + threadIdx.x; j < C; j += row_threads()) store_one(out + j, fn(load_one(xs + j), j));
}

// Block-wide (M, S [, sum x]) from the per-lane running values.
__device__ __forceinline__ RowStats row_combine(RowStats st, float *lds, bool want_sx) {
    RowStats r;
    r.m = row_block_reduce(st.m, lds, OpMax());
    const float mine = (st.m == -INFINITY) ? 0.f : st.s * fast_exp(st.m - r.m);
    r.s = row_block_reduce(mine, lds, OpSum());
    r.sx = want_sx ? row_block_reduce(st.sx, lds, OpSum()) : 0.f;
    return r;
}

// Rows are moved in 16-byte chunks when the tensors start on 16-byte boundaries (a row of the gradient
// then sits at the same offset from a boundary as the row of logits it belongs to).
template <class T>
static int row_chunks_ok(const T *x, const T *grad, int C) {
    return (!misaligned(x, 16) && !(grad && misaligned(grad, 16))) ? 1 : 0;
}


}  // namespace plh
