// LDS-staged grid sampler kernels for float tensors.
#include "gs2d_lds_launch.hpp"

namespace opscv {

template hipError_t lds_launch_typed<float>(const GridSamplerArgs&, const LdsPlan&, hipStream_t);

}  // namespace opscv
