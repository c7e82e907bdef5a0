// Large-margin forward kernels for f16 logits (one translation unit per element type and direction).
#include "lmargin_kernels.hpp"
namespace plh {
PLH_LM_INSTANTIATE(f16, true, false)
}
