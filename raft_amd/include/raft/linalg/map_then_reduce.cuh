// Whole-array map followed by a reduction to one scalar
// (linalg/map_then_reduce.cuh:37-80, linalg/detail/map_then_reduce.cuh:47-95 in the
// reference).  Unlike the reference's atomic accumulation the result here is
// deterministic: partial results are folded in a fixed order.
#pragma once

#include <raft/core/operators.hpp>
#include <raft/linalg/detail/rmi_bridge.hpp>

namespace raft::linalg {
namespace detail {
// The reference calls map(in[i]) (linalg/detail/map_then_reduce.cuh:58-61); the
// reduction's main_op is called with (value, index).  A map functor of the caller's
// own is wrapped so that it sees the value alone.
template <typename MapOp>
struct unary_map_adapter {
  MapOp map;
  template <typename T, typename I>
  constexpr RAFT_INLINE_FUNCTION auto operator()(const T& x, I) const
  {
    return map(x);
  }
};

template <typename InType, typename OutType, typename MapOp, typename ReduceLambda,
          typename... Args>
void map_reduce_call(const resources* res, OutType* out, size_t len, OutType neutral, MapOp map,
                     ReduceLambda op, hipStream_t stream, const InType* in, Args... args)
{
  if constexpr (sizeof...(Args) > 0) {
    // map(in[i], args[i]...) over several arrays: arbitrary device code by nature
#if defined(__HIPCC__)
    (void)res;
    raft::detail::rmi::generic::map_reduce_multi(stream, out, (std::int64_t)len, neutral, map, op,
                                                 in, args...);
#else
    static_assert(sizeof...(Args) == 0,
                  "map-then-reduce over several input arrays runs device code of the caller: "
                  "compile this translation unit with hipcc");
#endif
  } else if constexpr (raft::detail::rmi::main_tag<MapOp>::value >= 0) {
    raft::detail::rmi::reduce(res, stream, out, in, std::int64_t(1), (std::int64_t)len, true,
                              true, neutral, false, map, op, raft::identity_op());
  } else {
    raft::detail::rmi::reduce(res, stream, out, in, std::int64_t(1), (std::int64_t)len, true,
                              true, neutral, false, unary_map_adapter<MapOp>{map}, op,
                              raft::identity_op());
  }
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
