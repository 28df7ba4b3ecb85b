// The kernels of the MoE layer forward for Element = tf32_t (see kernels_impl.hpp).
#include "kernels_impl.hpp"

namespace kleos_amd {
KLEOS_INSTANTIATE_ELEMENT(tf32_t)
}  // namespace kleos_amd
