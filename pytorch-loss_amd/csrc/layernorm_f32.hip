// layer norm kernels for float elements (see layernorm_kernels.hpp).
#include "layernorm_kernels.hpp"

namespace plh {
PLH_LN_INSTANTIATE(float)
}  // namespace plh
