// LSR backward kernels for f16 logits (one translation unit per element type and direction).
#include "lsr_kernels.hpp"
namespace plh {
PLH_LSR_INSTANTIATE_BWD(f16)
}
