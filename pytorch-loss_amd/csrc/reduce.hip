// Second stage of the deterministic loss reduction: one block adds the per-block partials
// left behind by a forward kernel, in a fixed order, and writes the sum or the mean.
#include "plh_common.hpp"

namespace plh {

__global__ __launch_bounds__(1024) void finish_kernel(const float *__restrict__ sums, const int *__restrict__ cnts,
                                                      unsigned blocks, float *__restrict__ loss_out,
                                                      int64_t *__restrict__ count_out, int mode, int64_t fixed_count) {
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

void finish_partials(const Partials &part, unsigned blocks, float *loss_out, int64_t *count_out, FinishMode mode,
                     int64_t fixed_count, hipStream_t stream) {
    hipLaunchKernelGGL(finish_kernel, dim3(1), dim3(1024), 0, stream, part.sum, part.cnt, blocks, loss_out, count_out,
                       (int)mode, fixed_count);
}

}  // namespace plh

extern "C" int64_t plh_reduce_workspace_bytes(int64_t units) {
    if (units < 0 || units > plh::kMaxNumel) return PLH_ERR_BAD_SIZE;
    return 8 * plh::partial_slots(units);
}
