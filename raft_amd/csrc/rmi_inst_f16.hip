// Kernel instantiations for f16_t inputs.
#include "rmi_launch.hpp"

namespace rmi {
run_fn lookup_f16(const PolicyKey& k) { return lookup_for<f16_t, true, false>(k); }
}  // namespace rmi
