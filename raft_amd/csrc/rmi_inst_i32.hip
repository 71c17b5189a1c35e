// Kernel instantiations for int32_t inputs.
#include "rmi_launch.hpp"

namespace rmi {
run_fn lookup_i32(const PolicyKey& k) { return lookup_for<int32_t, false, false>(k); }
}  // namespace rmi
