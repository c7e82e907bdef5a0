// Large-margin kernels for f16 logits (one translation unit per element type).
#include "lmargin_kernels.hpp"
namespace plh {
PLH_LM_INSTANTIATE(f16)
}
