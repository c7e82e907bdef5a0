// LSR kernels for f16 logits (one translation unit per element type).
#include "lsr_kernels.hpp"
namespace plh {
PLH_LSR_INSTANTIATE(f16)
}
