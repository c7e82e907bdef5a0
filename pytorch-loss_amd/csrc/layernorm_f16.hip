// layer norm kernels for f16 elements (see layernorm_kernels.hpp).
#include "layernorm_kernels.hpp"

namespace plh {
PLH_LN_INSTANTIATE(f16)
}  // namespace plh
