// Soft dice loss for binary segmentation on gfx950 (csrc/soft_dice_kernel_v2.cu:54-407).
// Per row n of (batchsize, sample_size) logits x and float labels y, with q = sigmoid(x):
//   numer = 2 sum(q y) + smooth,  denor = sum(q^p + y) + smooth,  loss_n = 1 - numer / denor
// The label enters the denominator as it is, not raised to p (:86-91); the pure-torch V1/V2 classes use y^p
// (pytorch_loss/soft_dice_loss.py:35, :84), which is the same number for the binary labels the loss is meant for.
//   dloss_n/dx = p q^p (1 - q) numer / denor^2 - 2 y q (1 - q) / denor        (:236-247)
// Forward is a two-stage fixed-order reduction (per-block partial sums, then one block per row that
// adds them in double), so results do not depend on scheduling. It leaves (numer, denor) per row in
// `stats`; the backward is then a single elementwise pass (the reference reduces the row a second
// time in its backward, :343-377).
#include "plh_common.hpp"

namespace plh {

constexpr int kDiceBlock = 256;
constexpr int kDicePerThread = 4;
constexpr int kDiceTile = kDiceBlock * kDicePerThread;

__device__ __forceinline__ float dice_pow(float v, float p, int mode) {
    return mode == 1 ? v : (mode == 2 ? v * v : powf(v, p));
}
static int pow_mode(float p) { return p == 1.f ? 1 : (p == 2.f ? 2 : 0); }

__device__ __forceinline__ float sigmoid_fast(float x) {
    return __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-x * kLog2e));
}

// Vec: rows that start on 16-byte boundaries and hold a whole number of 4-element groups. Otherwise (rows of odd
// length: a 513 x 513 crop per sample) a group is still moved in one access, from an element boundary (the
// hardware takes such accesses, the types of Pack<T, 4> say so); only a row's last group goes element by element.
template <class T, bool Vec>
__device__ __forceinline__ void dice_load(const T *row, int64_t i, int64_t L, float (&v)[kDicePerThread]) {
    if constexpr (Vec) {
        load_vec<kDicePerThread>(row + i, v);
    } else {
        if (i + kDicePerThread <= L) {
            const typename Pack<T, 4>::Raw raw = Pack<T, 4>::load_unaligned(row + i);
#pragma unroll
            for (int k = 0; k < kDicePerThread; ++k) v[k] = Pack<T, 4>::get(raw, k);
        } else {
#pragma unroll
            for (int k = 0; k < kDicePerThread; ++k) v[k] = (i + k < L) ? load_one(row + i + k) : 0.f;
        }
    }
}

// blockIdx.y = row, blockIdx.x strides over the row's tiles; partial[(row * gridDim.x + block) * 2 + {0,1}].
// Two tiles per trip keep four 16-byte loads per lane in flight.
template <class T, bool Vec>
__global__ __launch_bounds__(kDiceBlock) void dice_partial(const T *__restrict__ x, const T *__restrict__ y,
                                                          float *__restrict__ partial, int64_t L, float p, int mode) {
    __shared__ float red[8];
    const T *xr = x + (int64_t)blockIdx.y * L, *yr = y + (int64_t)blockIdx.y * L;
    float a = 0.f, d = 0.f;
    const int64_t step = (int64_t)gridDim.x * kDiceTile;
    for (int64_t i = ((int64_t)blockIdx.x * kDiceBlock + threadIdx.x) * kDicePerThread; i < L; i += 2 * step) {
        float xv[2][kDicePerThread], yv[2][kDicePerThread];
        const bool second = i + step < L;
        dice_load<T, Vec>(xr, i, L, xv[0]);
        dice_load<T, Vec>(yr, i, L, yv[0]);
        if (second) {
            dice_load<T, Vec>(xr, i + step, L, xv[1]);
            dice_load<T, Vec>(yr, i + step, L, yv[1]);
        }
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            if (h == 1 && !second) break;
#pragma unroll
            for (int k = 0; k < kDicePerThread; ++k) {
                const bool in = Vec || (i + h * step + k < L);
                const float q = sigmoid_fast(xv[h][k]);
                a += in ? q * yv[h][k] : 0.f;
                d += in ? dice_pow(q, p, mode) + yv[h][k] : 0.f;
            }
        }
    }
    // both sums through one pass: DPP within the wave, then one LDS exchange between the four waves
    a = group_reduce<64>(a, OpSum());
    d = group_reduce<64>(d, OpSum());
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) {
        red[2 * wave] = a;
        red[2 * wave + 1] = d;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        float *out = partial + ((int64_t)blockIdx.y * gridDim.x + blockIdx.x) * 2;
        out[0] = (red[0] + red[2]) + (red[4] + red[6]);
        out[1] = (red[1] + red[3]) + (red[5] + red[7]);
    }
}

// One block per row: adds the row's partials in a fixed order.
__global__ __launch_bounds__(kDiceBlock) void dice_finish(const float *__restrict__ partial, int blocks, float smooth,
                                                         float *__restrict__ losses, float *__restrict__ stats) {
    __shared__ double sh[2][kDiceBlock];
    const float *row = partial + (int64_t)blockIdx.x * blocks * 2;
    double a = 0.0, d = 0.0;
    for (int b = threadIdx.x; b < blocks; b += kDiceBlock) {
        a += (double)row[2 * b];
        d += (double)row[2 * b + 1];
    }
    sh[0][threadIdx.x] = a;
    sh[1][threadIdx.x] = d;
    __syncthreads();
    for (int s = kDiceBlock / 2; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) {
            sh[0][threadIdx.x] += sh[0][threadIdx.x + s];
            sh[1][threadIdx.x] += sh[1][threadIdx.x + s];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        const float numer = (float)(2.0 * sh[0][0] + (double)smooth), denor = (float)(sh[1][0] + (double)smooth);
        stats[2 * blockIdx.x] = numer;
        stats[2 * blockIdx.x + 1] = denor;
        losses[blockIdx.x] = 1.f - numer / denor;
    }
}

template <class T, bool Vec>
__global__ __launch_bounds__(kDiceBlock) void dice_backward(const float *__restrict__ gout, const T *__restrict__ x,
                                                           const T *__restrict__ y, const float *__restrict__ stats,
                                                           T *__restrict__ gx, int64_t L, float p, int mode) {
    const int64_t off = (int64_t)blockIdx.y * L;
    const float numer = stats[2 * blockIdx.y], denor = stats[2 * blockIdx.y + 1], g = gout[blockIdx.y];
    const float c1 = g * p * numer / (denor * denor), c2 = g * 2.f / denor;
    auto grad_of = [&](float xv, float yv) {
        const float q = sigmoid_fast(xv);
        const float w = q * (1.f - q);
        // p q^p (1-q) numer/denor^2 - 2 y q (1-q)/denor, with q^p (1-q) = q^(p-1) * q(1-q)
        const float qp1 = mode == 1 ? 1.f : (mode == 2 ? q : powf(q, p - 1.f));
        return w * (c1 * qp1 - c2 * yv);
    };
    // Rows that start on element boundaries only: the elements up to the gradient row's first 128-byte line are
    // written one by one by the row's first block; from there on a wavefront's stores are whole lines.
    int64_t head = 0;
    if constexpr (!Vec) {
        const int64_t to_line = (int64_t)((128u - (unsigned)(reinterpret_cast<uintptr_t>(gx + off) & 127u)) & 127u) / (int64_t)sizeof(T);
        head = to_line < L ? to_line : L;
        if (blockIdx.x == 0 && (int64_t)threadIdx.x < head)
            store_one(gx + off + threadIdx.x, grad_of(load_one(x + off + threadIdx.x), load_one(y + off + threadIdx.x)));
    }
    for (int64_t i = head + ((int64_t)blockIdx.x * kDiceBlock + threadIdx.x) * kDicePerThread; i < L;
         i += (int64_t)gridDim.x * kDiceTile) {
        float xv[kDicePerThread], yv[kDicePerThread], r[kDicePerThread];
        dice_load<T, Vec>(x + off, i, L, xv);
        dice_load<T, Vec>(y + off, i, L, yv);
#pragma unroll
        for (int k = 0; k < kDicePerThread; ++k) r[k] = grad_of(xv[k], yv[k]);
        if constexpr (Vec) {
            store_vec<kDicePerThread>(gx + off + i, r);
        } else {
            if (i + kDicePerThread <= L) {
                Pack<T, 4>::store_unaligned(gx + off + i, Pack<T, 4>::put(r));
            } else {
#pragma unroll
                for (int k = 0; k < kDicePerThread; ++k)
                    if (i + k < L) store_one(gx + off + i + k, r[k]);
            }
        }
    }
}

static int64_t dice_blocks(int64_t batch, int64_t L) {
    const int64_t want = ceil_div(L > 0 ? L : 1, kDiceTile);
    // a reduction streams best from about four resident blocks per compute unit
    const int64_t cap = 1024 / (batch > 0 ? batch : 1);
    const int64_t lim = cap < 1 ? 1 : cap;
    return want < lim ? want : lim;
}

static int dice_check(const void *x, const void *y, const void *out, int64_t batch, int64_t L, size_t es) {
    if (batch < 0 || L < 0 || batch > 65535 || L > kMaxNumel) return PLH_ERR_BAD_SIZE;
    if ((double)batch * (double)L > (double)kMaxNumel) return PLH_ERR_BAD_SIZE;
    if (batch * L == 0) return PLH_OK;
    if (!x || !y || !out) return PLH_ERR_NULL_POINTER;
    if (misaligned(x, es) || misaligned(y, es)) return PLH_ERR_MISALIGNED;
    return PLH_OK;
}

}  // namespace plh

using namespace plh;

extern "C" int64_t plh_soft_dice_workspace_bytes(int64_t batchsize, int64_t sample_size) {
    if (batchsize < 0 || sample_size < 0 || batchsize > 65535) return PLH_ERR_BAD_SIZE;
    return (batchsize * dice_blocks(batchsize, sample_size) * 8 + 255) / 256 * 256;
}

extern "C" int plh_soft_dice_forward(const void *logits, int32_t dtype, const void *labels, float *losses, float *stats,
                                     void *workspace, int64_t workspace_bytes, int64_t batchsize, int64_t sample_size,
                                     float p, float smooth, void *stream) {
    if (!dtype_ok(dtype)) return PLH_ERR_BAD_DTYPE;
    const size_t es = dtype_size(dtype);
    int rc = dice_check(logits, labels, losses, batchsize, sample_size, es);
    if (rc != PLH_OK) return rc;
    if (batchsize == 0) return PLH_OK;
    if (!losses || !stats) return PLH_ERR_NULL_POINTER;
    if (misaligned(losses, 4) || misaligned(stats, 4)) return PLH_ERR_MISALIGNED;
    const int64_t blocks = dice_blocks(batchsize, sample_size);
    if (!workspace || misaligned(workspace, 256) || workspace_bytes < batchsize * blocks * 8) return PLH_ERR_WORKSPACE;
    hipStream_t st = (hipStream_t)stream;
    float *partial = static_cast<float *>(workspace);
    const int mode = pow_mode(p);
    const dim3 grid((unsigned)blocks, (unsigned)batchsize);
    dispatch_dtype(dtype, [&](auto tag) {
        using T = decltype(tag);
        const T *x = static_cast<const T *>(logits), *y = static_cast<const T *>(labels);
        const bool vec = sample_size % kDicePerThread == 0 && !misaligned(x, kDicePerThread * sizeof(T)) &&
                         !misaligned(y, kDicePerThread * sizeof(T));
        if (vec) hipLaunchKernelGGL((dice_partial<T, true>), grid, dim3(kDiceBlock), 0, st, x, y, partial, sample_size, p, mode);
        else hipLaunchKernelGGL((dice_partial<T, false>), grid, dim3(kDiceBlock), 0, st, x, y, partial, sample_size, p, mode);
    });
    hipLaunchKernelGGL(dice_finish, dim3((unsigned)batchsize), dim3(kDiceBlock), 0, st, partial, (int)blocks, smooth,
                       losses, stats);
    return check_launch();
}

extern "C" int plh_soft_dice_backward(const float *grad_output, const void *logits, int32_t dtype, const void *labels,
                                      const float *stats, void *grad_logits, int64_t batchsize, int64_t sample_size,
                                      float p, void *stream) {
    if (!dtype_ok(dtype)) return PLH_ERR_BAD_DTYPE;
    const size_t es = dtype_size(dtype);
    const int rc = dice_check(logits, labels, grad_logits, batchsize, sample_size, es);
    if (rc != PLH_OK) return rc;
    if (batchsize * sample_size == 0) return PLH_OK;
    if (!grad_output || !stats) return PLH_ERR_NULL_POINTER;
    if (misaligned(grad_output, 4) || misaligned(stats, 4) || misaligned(grad_logits, es)) return PLH_ERR_MISALIGNED;
    hipStream_t st = (hipStream_t)stream;
    const int mode = pow_mode(p);
    // elementwise: one tile per block streams best
    const dim3 grid((unsigned)ceil_div(sample_size, kDiceTile), (unsigned)batchsize);
    dispatch_dtype(dtype, [&](auto tag) {
        using T = decltype(tag);
        const T *x = static_cast<const T *>(logits), *y = static_cast<const T *>(labels);
        T *gx = static_cast<T *>(grad_logits);
        const bool vec = sample_size % kDicePerThread == 0 && !misaligned(x, kDicePerThread * sizeof(T)) &&
                         !misaligned(y, kDicePerThread * sizeof(T)) && !misaligned(gx, kDicePerThread * sizeof(T));
        if (vec) hipLaunchKernelGGL((dice_backward<T, true>), grid, dim3(kDiceBlock), 0, st, grad_output, x, y, stats, gx,
                                    sample_size, p, mode);
        else hipLaunchKernelGGL((dice_backward<T, false>), grid, dim3(kDiceBlock), 0, st, grad_output, x, y, stats, gx,
                                sample_size, p, mode);
    });
    return check_launch();
}
