// Taylor cross-entropy forward kernels for f16 elements (see taylor_kernels.hpp).
#include "taylor_kernels.hpp"
namespace plh {
PLH_TAYLOR_INSTANTIATE(f16, kTaylorCeFwd)
}
