// Kernel instantiations for int64_t inputs.
#include "rmi_launch.hpp"

namespace rmi {
run_fn lookup_i64(const PolicyKey& k) { return lookup_for<int64_t, false, false>(k); }
}  // namespace rmi
