// LDS-staged grid sampler kernels for _Float16 tensors, planes on the 16-byte grid.
#include "gs2d_lds_launch.hpp"

namespace opscv {

template hipError_t lds_launch_typed<_Float16, false>(const GridSamplerArgs&, const LdsPlan&, hipStream_t);

}  // namespace opscv
