// Large-margin backward kernels for float logits (one translation unit per element type and direction).
#include "lmargin_kernels.hpp"
namespace plh {
PLH_LM_INSTANTIATE(float, false, true)
}
