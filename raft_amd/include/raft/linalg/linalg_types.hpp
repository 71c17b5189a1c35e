#pragma once
#include <raft/core/types.hpp>
namespace raft::linalg {
enum class FillMode { UPPER, LOWER };
enum class Operation { NON_TRANSPOSE, TRANSPOSE };
}  // namespace raft::linalg
