// Second stage of the deterministic loss reduction: one block adds the per-block partials
// left behind by a forward kernel, in a fixed order, and writes the sum or the mean.
#include "plh_common.hpp"

namespace plh {

__global__ __launch_bounds__(1024) void finish_kernel(const float *__restrict__ sums, const int *__restrict__ cnts,
                                                      unsigned blocks, float *__restrict__ loss_out,
                                                      int64_t *__restrict__ count_out, int mode, int64_t fixed_count) {
    finish_block(sums, cnts, blocks, loss_out, count_out, mode, fixed_count);
}

void finish_partials(const Partials &part, unsigned blocks, float *loss_out, int64_t *count_out, FinishMode mode,
                     int64_t fixed_count, hipStream_t stream) {
    hipLaunchKernelGGL(finish_kernel, dim3(1), dim3(1024), 0, stream, part.sum, part.cnt, blocks, loss_out, count_out,
                       (int)mode, fixed_count);
}

// Per block the number of labels other than `ignore`: a loop over the labels in 16-byte pairs, four loads in flight per
// thread (`lab` on a 16-byte boundary; an odd last label goes to block 0).
__global__ __launch_bounds__(256) void count_valid_kernel(const int64_t *__restrict__ lab, int64_t P, int64_t ignore,
                                                          float *__restrict__ sums, int *__restrict__ cnts) {
    __shared__ float red[4];
    typedef long long pair_t __attribute__((ext_vector_type(2)));
    const pair_t *lab2 = reinterpret_cast<const pair_t *>(lab);
    const int64_t pairs = P / 2;
    const int64_t stride = (int64_t)gridDim.x * 256;
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    int n = 0;
    for (; i + 3 * stride < pairs; i += 4 * stride) {
        pair_t v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = __builtin_nontemporal_load(lab2 + i + u * stride);
#pragma unroll
        for (int u = 0; u < 4; ++u) n += (v[u].x != ignore ? 1 : 0) + (v[u].y != ignore ? 1 : 0);
    }
    for (; i < pairs; i += stride) {
        const pair_t v = lab2[i];
        n += (v.x != ignore ? 1 : 0) + (v.y != ignore ? 1 : 0);
    }
    if (blockIdx.x == 0 && threadIdx.x == 0 && (P & 1)) n += lab[P - 1] != ignore ? 1 : 0;
    // a block counts at most P / gridDim.x + 2048 labels, below 2^24 for every P the entry points take: the float sum
    // is exact
    const float total = block_sum_256((float)n, red);
    if (threadIdx.x == 0) {
        sums[blockIdx.x] = 0.f;
        cnts[blockIdx.x] = (int)total;
    }
}

// The same label by label, for a label tensor that starts on an 8-byte boundary only.
__global__ __launch_bounds__(256) void count_valid_kernel_unaligned(const int64_t *__restrict__ lab, int64_t P, int64_t ignore,
                                                                    float *__restrict__ sums, int *__restrict__ cnts) {
    __shared__ float red[4];
    const int64_t stride = (int64_t)gridDim.x * 256;
    int n = 0;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < P; i += stride) n += lab[i] != ignore ? 1 : 0;
    const float total = block_sum_256((float)n, red);
    if (threadIdx.x == 0) {
        sums[blockIdx.x] = 0.f;
        cnts[blockIdx.x] = (int)total;
    }
}

// The number of labels other than `ignore` added to *total (zeroed by an earlier launch on the stream): at most 256
// blocks, one 64-bit atomic each.
__global__ __launch_bounds__(256) void count_valid_total_kernel(const int64_t *__restrict__ lab, int64_t P, int64_t ignore,
                                                                unsigned long long *__restrict__ total) {
    __shared__ float red[4];
    const int64_t stride = (int64_t)gridDim.x * 256;
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    long long n = 0;
    for (; i + 3 * stride < P; i += 4 * stride) {
        int64_t v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = __builtin_nontemporal_load(lab + i + u * stride);
#pragma unroll
        for (int u = 0; u < 4; ++u) n += v[u] != ignore ? 1 : 0;
    }
    for (; i < P; i += stride) n += lab[i] != ignore ? 1 : 0;
    // per thread at most P / (256 * gridDim.x) + 4 < 2^16 labels for P < 2^31 and 256 blocks; the block's sum goes in
    // two exact float halves
    const float lo = block_sum_256((float)(n & 0xFF), red), hi = block_sum_256((float)(n >> 8), red);
    if (threadIdx.x == 0) atomicAdd(total, (unsigned long long)lo + ((unsigned long long)hi << 8));
}

void count_valid_total(const int64_t *labels, int64_t P, int64_t ignore, unsigned long long *total, hipStream_t stream) {
    int64_t blocks = ceil_div(P, (int64_t)4096);
    blocks = blocks < 1 ? 1 : (blocks > 256 ? 256 : blocks);
    hipLaunchKernelGGL(count_valid_total_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, labels, P, ignore, total);
}

unsigned count_valid_partials(const int64_t *labels, int64_t P, int64_t ignore, const Partials &part, hipStream_t stream) {
    // at least 4096 labels per block, at most 2048 blocks (8 per CU): P < 2^31 leaves a block 2^20 labels
    int64_t blocks = ceil_div(P, (int64_t)4096);
    blocks = blocks < 1 ? 1 : (blocks > 2048 ? 2048 : blocks);
    if (misaligned(labels, 16))
        hipLaunchKernelGGL(count_valid_kernel_unaligned, dim3((unsigned)blocks), dim3(256), 0, stream, labels, P, ignore,
                           part.sum, part.cnt);
    else
        hipLaunchKernelGGL(count_valid_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, labels, P, ignore, part.sum,
                           part.cnt);
    return (unsigned)blocks;
}

// data[i] *= *scalar, unless *scalar is exactly 1 (every block reads the scalar and returns).
template <class T>
__global__ __launch_bounds__(256) void scale_unless_one_kernel(T *__restrict__ data, int64_t numel,
                                                               const float *__restrict__ scalar) {
    const float g = *scalar;
    if (g == 1.f) return;
    constexpr int kPer = 16 / (int)sizeof(T);
    const int64_t stride = (int64_t)gridDim.x * 256;
    const int64_t vecs = numel / kPer;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < vecs; i += stride) {
        const plh_u4 w = __builtin_nontemporal_load(reinterpret_cast<const plh_u4 *>(data) + i);
        unsigned d[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            if constexpr (sizeof(T) == 4) {
                d[k] = f32_bits(bits_f32(d[k]) * g);
            } else {
                const uint16_t lo = narrow(widen((uint16_t)(d[k] & 0xFFFFu), T{}) * g, T{});
                const uint16_t hi = narrow(widen((uint16_t)(d[k] >> 16), T{}) * g, T{});
                d[k] = (unsigned)lo | ((unsigned)hi << 16);
            }
        }
        __builtin_nontemporal_store(plh_u4{d[0], d[1], d[2], d[3]}, reinterpret_cast<plh_u4 *>(data) + i);
    }
    if (blockIdx.x == 0) {
        for (int64_t i = vecs * kPer + threadIdx.x; i < numel; i += 256) store_one(data + i, load_one(data + i) * g);
    }
}

}  // namespace plh

extern "C" int plh_scale_unless_one(void *data, int32_t dtype, int64_t numel, const float *scalar, void *stream) {
    using namespace plh;
    if (!dtype_ok(dtype)) return PLH_ERR_BAD_DTYPE;
    if (numel < 0) return PLH_ERR_BAD_SIZE;
    if (numel == 0) return PLH_OK;
    if (!data || !scalar) return PLH_ERR_NULL_POINTER;
    // whole 16-byte words from the first element on
    if (misaligned(data, 16) || misaligned(scalar, 4)) return PLH_ERR_MISALIGNED;
    int64_t blocks = ceil_div(numel * (int64_t)dtype_size(dtype), (int64_t)(256 * 16 * 4));
    blocks = blocks < 1 ? 1 : (blocks > 16384 ? 16384 : blocks);
    dispatch_dtype(dtype, [&](auto tag) {
        using T = decltype(tag);
        hipLaunchKernelGGL(scale_unless_one_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                           static_cast<T *>(data), numel, scalar);
    });
    return check_launch();
}

extern "C" int64_t plh_reduce_workspace_bytes(int64_t units) {
    if (units < 0 || units > plh::kMaxNumel) return PLH_ERR_BAD_SIZE;
    return 8 * plh::partial_slots(units);
}
