// Large-margin kernels for bf16 logits (one translation unit per element type).
#include "lmargin_kernels.hpp"
namespace plh {
PLH_LM_INSTANTIATE(bf16)
}
