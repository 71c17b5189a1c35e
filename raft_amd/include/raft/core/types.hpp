#pragma once
namespace raft {
// Whether a reduction or broadcast runs along a matrix's rows (one result per
// row) or along its columns (one result per column).  core/types.hpp:17.
enum class Apply { ALONG_ROWS, ALONG_COLUMNS };
}  // namespace raft
