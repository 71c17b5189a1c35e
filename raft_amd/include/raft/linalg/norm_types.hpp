#pragma once
namespace raft::linalg {
// How a norm is computed (linalg/norm_types.hpp:13-23 in the reference).
enum NormType : unsigned short {
  L0PseudoNorm = 0,  // sum(x_i != 0 ? 1 : 0); not a norm
  L1Norm       = 1,  // sum(|x_i|)
  L2Norm       = 2,  // sum(x_i^2); the square root is the caller's final_op
  LinfNorm           // max(|x_i|)
};
}  // namespace raft::linalg
