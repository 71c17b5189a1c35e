// Kernel instantiations for double inputs.
#include "rmi_launch.hpp"

namespace rmi {
run_fn lookup_f64(const PolicyKey& k) { return lookup_for<double, true, true>(k); }
}  // namespace rmi
