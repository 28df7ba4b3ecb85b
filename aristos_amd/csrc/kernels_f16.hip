// The kernels of the MoE layer forward for Element = f16_t (see kernels_impl.hpp).
#include "kernels_impl.hpp"

namespace kleos_amd {
KLEOS_INSTANTIATE_ELEMENT(f16_t)
}  // namespace kleos_amd
