// Kernel instantiations for float inputs.
#include "rmi_launch.hpp"

namespace rmi {
run_fn lookup_f32(const PolicyKey& k) { return lookup_for<float, true, false>(k); }
}  // namespace rmi
