// LDS-staged grid sampler kernels for __bf16 tensors.
#include "gs2d_lds_launch.hpp"

namespace opscv {

template hipError_t lds_launch_typed<__bf16>(const GridSamplerArgs&, const LdsPlan&, hipStream_t);

}  // namespace opscv
