// Kernel instantiations for int8_t inputs.
#include "rmi_launch.hpp"

namespace rmi {
run_fn lookup_i8(const PolicyKey& k) { return lookup_for<int8_t, false, false>(k); }
}  // namespace rmi
