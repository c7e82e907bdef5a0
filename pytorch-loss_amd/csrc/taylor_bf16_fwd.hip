// Taylor softmax forward kernels for bf16 elements (see taylor_kernels.hpp).
#include "taylor_kernels.hpp"
namespace plh {
PLH_TAYLOR_INSTANTIATE(bf16, kTaylorFwd)
}
