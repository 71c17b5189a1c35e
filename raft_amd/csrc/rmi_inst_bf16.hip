// Kernel instantiations for bf16_t inputs.
#include "rmi_launch.hpp"

namespace rmi {
run_fn lookup_bf16(const PolicyKey& k) { return lookup_for<bf16_t, true, false>(k); }
norm_fn lookup_norm_bf16(int main_op, int red_op) { return lookup_norm_for<bf16_t, false>(main_op, red_op); }
run_fn lookup_meanvar_bf16() { return &run<PolMeanVar<bf16_t>>; }
}  // namespace rmi
