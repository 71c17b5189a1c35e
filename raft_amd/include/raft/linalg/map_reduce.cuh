// map_reduce: out = op-fold of map(in[i]) starting from `neutral`
// (linalg/map_reduce.cuh:37-103 in the reference).
#pragma once

#include <raft/core/device_mdspan.hpp>
#include <raft/core/resource/cuda_stream.hpp>
#include <raft/linalg/map_then_reduce.cuh>

namespace raft::linalg {

template <typename InType, typename MapOp, typename ReduceLambda, typename IdxType = std::uint32_t,
          int TPB = 256, typename OutType = InType, typename... Args>
void mapReduce(OutType* out, size_t len, OutType neutral, MapOp map, ReduceLambda op,
               hipStream_t stream, const InType* in, Args... args)
{
  detail::map_reduce_call<InType, OutType>(nullptr, out, len, neutral, map, op, stream, in,
                                           args...);
}

template <typename InValueType, typename MapOp, typename ReduceLambda, typename IndexType,
          typename OutValueType, typename ScalarIdxType, typename... Args>
void map_reduce(raft::resources const& handle,
                raft::device_vector_view<const InValueType, IndexType> in,
                raft::device_scalar_view<OutValueType, ScalarIdxType> out,
                OutValueType neutral,
                MapOp map,
                ReduceLambda op,
                Args... args)
{
  detail::map_reduce_call<InValueType, OutValueType>(&handle, out.data_handle(),
                                                     (size_t)in.extent(0), neutral, map, op,
                                                     resource::get_cuda_stream(handle),
                                                     in.data_handle(), args...);
}

}  // namespace raft::linalg
