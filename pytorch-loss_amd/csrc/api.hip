// Library-level entry points: ABI version, error text, and the plain copy kernel
// used to calibrate byte counters and to measure achievable copy bandwidth.
#include "plh_common.hpp"

namespace plh {

__global__ __launch_bounds__(256) void stream_copy_vec4(const float4 *__restrict__ src, float4 *__restrict__ dst,
                                                        int64_t n4) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n4) dst[i] = src[i];
}

__global__ __launch_bounds__(256) void stream_copy_scalar(const float *__restrict__ src, float *__restrict__ dst,
                                                          int64_t first, int64_t numel) {
    const int64_t i = first + (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < numel) dst[i] = src[i];
}

// Run length of the XCD-aware tile permutation (tile_of_block). Measured on MI355X over six
// segmentation shapes, both element sizes and five kernels (LSR and large-margin forward and
// backward, OHEM scores): runs of 8..32 tiles are within 1 % of the best almost everywhere, runs of
// 64..288 lose 3..20 % on several shapes. The one systematic exception: fp32 logits whose channel
// plane is a multiple of 4 MiB (1024x1024, 2048x1024) run 3 % faster with runs of 1024 tiles, which
// costs 16-bit logits of the same shapes up to 13 %, hence the element-size condition.
unsigned xcd_run_for(size_t elem_bytes, int64_t m_size) {
    if (elem_bytes == 4 && m_size > 0 && (m_size * 4) % ((int64_t)4 << 20) == 0) return 1024u;
    return 32u;
}

}  // namespace plh

using namespace plh;

extern "C" int plh_abi_version(void) { return PLH_ABI_VERSION; }

extern "C" const char *plh_error_string(int code) {
    switch (code) {
        case PLH_OK: return "ok";
        case PLH_ERR_NULL_POINTER: return "a required pointer is NULL";
        case PLH_ERR_BAD_SIZE: return "negative or unsupported size";
        case PLH_ERR_BAD_STRIDE: return "grad_output_stride must be 0 (broadcast scalar) or 1 (per element)";
        case PLH_ERR_TOO_MANY_CLASSES: return "num of classes should be less than 512";
        case PLH_ERR_WORKSPACE: return "workspace is NULL, misaligned or smaller than the op's plh_*_workspace_bytes()";
        case PLH_ERR_MISALIGNED: return "a pointer is not aligned to its element size";
        case PLH_ERR_BAD_DTYPE: return "dtype must be PLH_DTYPE_F32, PLH_DTYPE_F16 or PLH_DTYPE_BF16";
        default: break;
    }
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "unknown error code";
}

extern "C" int plh_stream_copy(const float *src, float *dst, int64_t numel, void *stream) {
    if (numel < 0 || numel > kMaxNumel) return PLH_ERR_BAD_SIZE;
    if (numel == 0) return PLH_OK;
    if (!src || !dst) return PLH_ERR_NULL_POINTER;
    if (misaligned(src, 4) || misaligned(dst, 4)) return PLH_ERR_MISALIGNED;
    hipStream_t st = (hipStream_t)stream;
    int64_t done = 0;
    if (!misaligned(src, 16) && !misaligned(dst, 16) && numel >= 4) {
        const int64_t n4 = numel / 4;
        hipLaunchKernelGGL(stream_copy_vec4, dim3((unsigned)ceil_div(n4, 256)), dim3(256), 0, st,
                           reinterpret_cast<const float4 *>(src), reinterpret_cast<float4 *>(dst), n4);
        done = n4 * 4;
    }
    if (done < numel) {
        hipLaunchKernelGGL(stream_copy_scalar, dim3((unsigned)ceil_div(numel - done, 256)), dim3(256), 0, st,
                           src, dst, done, numel);
    }
    return check_launch();
}
