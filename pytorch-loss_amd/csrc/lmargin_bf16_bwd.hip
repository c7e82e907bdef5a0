// Large-margin backward kernels for bf16 logits (one translation unit per element type and direction).
#include "lmargin_kernels.hpp"
namespace plh {
PLH_LM_INSTANTIATE(bf16, false, true)
}
