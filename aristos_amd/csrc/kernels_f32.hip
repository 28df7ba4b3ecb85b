// The kernels of the MoE layer forward for Element = float (see kernels_impl.hpp).
#include "kernels_impl.hpp"

namespace kleos_amd {
KLEOS_INSTANTIATE_ELEMENT(float)
}  // namespace kleos_amd
