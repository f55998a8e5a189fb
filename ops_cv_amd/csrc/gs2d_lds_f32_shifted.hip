// LDS-staged grid sampler kernels for float tensors, planes off the 16-byte grid (shifted layout).
#include "gs2d_lds_launch.hpp"

namespace opscv {

template hipError_t lds_launch_typed<float, true>(const GridSamplerArgs&, const LdsPlan&, hipStream_t);

}  // namespace opscv
