// Kernel instantiations for bf16_t inputs.
#include "rmi_launch.hpp"

namespace rmi {
run_fn lookup_bf16(const PolicyKey& k) { return lookup_for<bf16_t, true, false>(k); }
}  // namespace rmi
