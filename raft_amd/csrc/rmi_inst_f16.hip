// Kernel instantiations for f16_t inputs.
#include "rmi_launch.hpp"

namespace rmi {
run_fn lookup_f16(const PolicyKey& k) { return lookup_for<f16_t, true, false>(k); }
norm_fn lookup_norm_f16(int main_op, int red_op) { return lookup_norm_for<f16_t, false>(main_op, red_op); }
run_fn lookup_meanvar_f16() { return &run<PolMeanVar<f16_t>>; }
}  // namespace rmi
