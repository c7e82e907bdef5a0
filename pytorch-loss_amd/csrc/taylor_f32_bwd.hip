// Taylor softmax backward kernels for float elements (see taylor_kernels.hpp).
#include "taylor_kernels.hpp"
namespace plh {
PLH_TAYLOR_INSTANTIATE(float, kTaylorBwd)
}
