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

}  // namespace plh

extern "C" int64_t plh_reduce_workspace_bytes(int64_t units) {
    if (units < 0 || units > plh::kMaxNumel) return PLH_ERR_BAD_SIZE;
    return 8 * plh::partial_slots(units);
}
