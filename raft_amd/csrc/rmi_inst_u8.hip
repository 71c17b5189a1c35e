// Kernel instantiations for uint8_t inputs.
#include "rmi_launch.hpp"

namespace rmi {
run_fn lookup_u8(const PolicyKey& k) { return lookup_for<uint8_t, false, false>(k); }
}  // namespace rmi
