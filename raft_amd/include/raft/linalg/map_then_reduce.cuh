// Whole-array map followed by a reduction to one scalar
// (linalg/map_then_reduce.cuh:37-80, linalg/detail/map_then_reduce.cuh:47-95 in the
// reference).  Unlike the reference's atomic accumulation the result here is
// deterministic: partial results are folded in a fixed order.
#pragma once

#include <raft/core/operators.hpp>
#include <raft/linalg/detail/rmi_bridge.hpp>

namespace raft::linalg {
namespace detail {
template <typename InType, typename OutType, typename MapOp, typename ReduceLambda,
          typename... Args>
void map_reduce_call(const resources* res, OutType* out, size_t len, OutType neutral, MapOp map,
                     ReduceLambda op, hipStream_t stream, const InType* in, Args...)
{
  static_assert(sizeof...(Args) == 0,
                "map-then-reduce over several input arrays is not lowered to the reduction "
                "library; only map(in[i]) is");
  raft::detail::rmi::reduce(res, stream, out, in, std::int64_t(1), (std::int64_t)len, true, true,
                            neutral, false, map, op, raft::identity_op());
}
}  // namespace detail

template <typename InType, typename MapOp, typename IdxType = std::uint32_t, int TPB = 256,
          typename... Args, typename OutType = InType>
void mapThenSumReduce(OutType* out, IdxType len, MapOp map, hipStream_t stream, const InType* in,
                      Args... args)
{
  detail::map_reduce_call<InType, OutType>(nullptr, out, (size_t)len, (OutType)0, map,
                                           raft::add_op(), stream, in, args...);
}

template <typename InType, typename MapOp, typename ReduceLambda, typename IdxType = std::uint32_t,
          int TPB = 256, typename OutType = InType, typename... Args>
[[deprecated("Use function `mapReduce` from `raft/linalg/map_reduce.cuh")]] void mapThenReduce(
  OutType* out, size_t len, OutType neutral, MapOp map, ReduceLambda op, hipStream_t stream,
  const InType* in, Args... args)
{
  detail::map_reduce_call<InType, OutType>(nullptr, out, len, neutral, map, op, stream, in,
                                           args...);
}

}  // namespace raft::linalg
