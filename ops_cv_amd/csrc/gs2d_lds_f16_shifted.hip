// LDS-staged grid sampler kernels for _Float16 tensors, planes off the 16-byte grid (shifted layout).
#include "gs2d_lds_launch.hpp"

namespace opscv {

template hipError_t lds_launch_typed<_Float16, true>(const GridSamplerArgs&, const LdsPlan&, hipStream_t);

}  // namespace opscv
