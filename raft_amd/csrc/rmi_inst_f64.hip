// Kernel instantiations for double inputs.
#include "rmi_launch.hpp"

namespace rmi {
run_fn lookup_f64(const PolicyKey& k) { return lookup_for<double, true, true>(k); }
norm_fn lookup_norm_f64(int main_op, int red_op) { return lookup_norm_for<double, true>(main_op, red_op); }
run_fn lookup_meanvar_f64() { return &run<PolMeanVar<double>>; }
}  // namespace rmi
