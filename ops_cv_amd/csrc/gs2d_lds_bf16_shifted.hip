// LDS-staged grid sampler kernels for __bf16 tensors, planes off the 16-byte grid (shifted layout).
#include "gs2d_lds_launch.hpp"

namespace opscv {

template hipError_t lds_launch_typed<__bf16, true>(const GridSamplerArgs&, const LdsPlan&, hipStream_t);

}  // namespace opscv
