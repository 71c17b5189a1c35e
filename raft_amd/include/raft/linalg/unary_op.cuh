// Elementwise unary operations (linalg/unary_op.cuh:33-120 in the reference), built on
// raft::linalg::map.  For translation units compiled by hipcc.
#pragma once

#include <raft/linalg/map.cuh>

namespace raft::linalg {

template <typename InType, typename Lambda, typename IdxType = int, typename OutType = InType,
          int TPB = 256>
void unaryOp(OutType* out, const InType* in, IdxType len, Lambda op, hipStream_t stream)
{
  return detail::map<false>(stream, out, len, op, in);
}

namespace detail {
// op(&result, offset) writes the element; the map wants it returned
template <typename OutType, typename Lambda>
struct write_only_adapter {
  Lambda op;
  template <typename IdxType>
  __device__ OutType operator()(IdxType offset)
  {
    OutType r;
    op(&r, offset);
    return r;
  }
};
}  // namespace detail

template <typename OutType, typename Lambda, typename IdxType = int, int TPB = 256>
void writeOnlyUnaryOp(OutType* out, IdxType len, Lambda op, hipStream_t stream)
{
  return detail::map<true>(stream, out, len, detail::write_only_adapter<OutType, Lambda>{op});
}

template <typename InType, typename Lambda, typename OutType,
          typename = std::enable_if_t<is_mdspan_v<InType> && is_mdspan_v<OutType>>>
void unary_op(raft::resources const& handle, InType in, OutType out, Lambda op)
{
  return map(handle, in, out, op);
}

template <typename OutType, typename Lambda, typename = std::enable_if_t<is_mdspan_v<OutType>>>
void write_only_unary_op(const raft::resources& handle, OutType out, Lambda op)
{
  return writeOnlyUnaryOp(out.data_handle(), out.size(), op, resource::get_cuda_stream(handle));
}

}  // namespace raft::linalg
