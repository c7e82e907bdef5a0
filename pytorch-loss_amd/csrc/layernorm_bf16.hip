// layer norm kernels for bf16 elements (see layernorm_kernels.hpp).
#include "layernorm_kernels.hpp"

namespace plh {
PLH_LN_INSTANTIATE(bf16)
}  // namespace plh
