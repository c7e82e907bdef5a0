// LSR kernels that leave loss partials and gradient in one pass, for bf16 logits (one translation unit per element
// type and direction).
#include "lsr_kernels.hpp"
namespace plh {
PLH_LSR_INSTANTIATE_BOTH(bf16)
}
