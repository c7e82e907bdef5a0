// Large-margin kernels for float logits (one translation unit per element type).
#include "lmargin_kernels.hpp"
namespace plh {
PLH_LM_INSTANTIATE(float)
}
