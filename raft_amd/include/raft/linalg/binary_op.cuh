// Elementwise binary operations (linalg/binary_op.cuh:34-85 in the reference), built on
// raft::linalg::map.  For translation units compiled by hipcc.
#pragma once

#include <raft/linalg/map.cuh>

namespace raft::linalg {

template <typename InType, typename Lambda, typename OutType = InType, typename IdxType = int,
          int TPB = 256>
void binaryOp(
  OutType* out, const InType* in1, const InType* in2, IdxType len, Lambda op, hipStream_t stream)
{
  return detail::map<false>(stream, out, len, op, in1, in2);
}

template <typename InType, typename Lambda, typename OutType,
          typename = std::enable_if_t<is_mdspan_v<InType> && is_mdspan_v<OutType>>>
void binary_op(raft::resources const& handle, InType in1, InType in2, OutType out, Lambda op)
{
  return map(handle, in1, in2, out, op);
}

}  // namespace raft::linalg
