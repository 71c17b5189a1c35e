// Kernel instantiations for float inputs.
#include "rmi_launch.hpp"

namespace rmi {
run_fn lookup_f32(const PolicyKey& k) { return lookup_for<float, true, false>(k); }
norm_fn lookup_norm_f32(int main_op, int red_op) { return lookup_norm_for<float, false>(main_op, red_op); }
run_fn lookup_meanvar_f32() { return &run<PolMeanVar<float>>; }
}  // namespace rmi
