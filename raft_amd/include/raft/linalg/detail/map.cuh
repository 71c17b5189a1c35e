// Elementwise map over zero or more equally sized arrays, optionally with the flat
// element offset as first argument (linalg/detail/map.cuh:27-225 in the reference).
// The functor is arbitrary device code, so the kernel is instantiated in the caller's
// translation unit: include from files compiled by hipcc.
//
// Each lane moves packs of R consecutive elements, R chosen so that the widest element
// type fills a 16-byte lane access (narrower types move proportionally less), four
// packs per lane in flight, a workgroup's packs interleaved so every access instruction
// covers one contiguous span of the wave.  gfx950 serves vector accesses at any
// element-aligned address, so no alignment prologue is needed (the reference peels up to
// R - 1 elements on the left and lowers R when the pointers' alignments disagree,
// :61-101,112-166); the last len % R elements are handled one by one.  `out` may alias
// an input: every pack is loaded before it is stored and no two lanes share an element.
#pragma once

#if !defined(__HIPCC__)
#error "raft/linalg/map.cuh instantiates device code: include it only from hipcc translation units"
#endif

#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

#include <raft/core/device_mdspan.hpp>
#include <raft/core/error.hpp>
#include <raft/core/resource/cuda_stream.hpp>
#include <raft/core/resources.hpp>

namespace raft {
namespace linalg::detail {

constexpr int kMapBlock  = 256;
constexpr int kMapUnroll = 4;

template <bool PassOffset, typename OutT, typename IdxT, typename Func, typename... InTs>
__device__ __forceinline__ auto map_apply(Func& f, const IdxT& offset, const InTs&... ins) -> OutT
{
  if constexpr (PassOffset) {
    return f(offset, ins...);
  } else {
    return f(ins...);
  }
}

template <typename T, int R>
struct map_pack {
  T v[R];
};

// Packs of 4, 8 or 16 bytes move as one non-temporal access (every element is read and
// written once); other sizes element by element.
template <int BYTES>
struct map_word {
  using type = void;
};
template <>
struct map_word<4> {
  using type = std::uint32_t;
};
template <>
struct map_word<8> {
  typedef std::uint32_t type __attribute__((ext_vector_type(2)));
};
template <>
struct map_word<16> {
  typedef std::uint32_t type __attribute__((ext_vector_type(4)));
};

template <typename T, int R, bool NT = true>
__device__ __forceinline__ map_pack<T, R> map_load(const T* p, std::int64_t off)
{
  map_pack<T, R> x;
  using W = typename map_word<(int)sizeof(map_pack<T, R>)>::type;
  if constexpr (!std::is_void_v<W> && std::is_trivially_copyable_v<T>) {
    typedef W W_unaligned __attribute__((aligned(1)));
    W w;
    if constexpr (NT) {
      w = __builtin_nontemporal_load(reinterpret_cast<const W_unaligned*>(p + off));
    } else {
      w = *reinterpret_cast<const W_unaligned*>(p + off);
    }
    __builtin_memcpy(&x, &w, sizeof(x));
  } else {
    __builtin_memcpy(&x, p + off, sizeof(x));
  }
  return x;
}

template <typename T, int R, bool NT = true>
__device__ __forceinline__ void map_store(T* p, std::int64_t off, const map_pack<T, R>& x)
{
  using W = typename map_word<(int)sizeof(map_pack<T, R>)>::type;
  if constexpr (!std::is_void_v<W> && std::is_trivially_copyable_v<T>) {
    typedef W W_unaligned __attribute__((aligned(1)));
    W w;
    __builtin_memcpy(&w, &x, sizeof(x));
    if constexpr (NT) {
      __builtin_nontemporal_store(w, reinterpret_cast<W_unaligned*>(p + off));
    } else {
      *reinterpret_cast<W_unaligned*>(p + off) = w;
    }
  } else {
    __builtin_memcpy(p + off, &x, sizeof(x));
  }
}

template <int R, bool PassOffset, typename IdxT>
struct map_cfg {};

// one pack per input array, held in registers between the loads and the stores
template <int R, typename... Ts>
struct map_pack_set {};
template <int R, typename T, typename... Ts>
struct map_pack_set<R, T, Ts...> {
  map_pack<T, R> head;
  map_pack_set<R, Ts...> tail;
};

template <int R>
__device__ __forceinline__ void map_load_set(map_pack_set<R>&, std::int64_t)
{
}
template <int R, typename T, typename... Ts>
__device__ __forceinline__ void map_load_set(map_pack_set<R, T, Ts...>& s, std::int64_t off,
                                             const T* p, const Ts*... ps)
{
  s.head = map_load<T, R>(p, off);
  map_load_set(s.tail, off, ps...);
}

// all packs unpacked into xs: apply f element by element and store the result pack
template <int R, bool PassOffset, typename IdxT, typename OutT, typename Func, typename... Done>
__device__ __forceinline__ void map_store_set(map_cfg<R, PassOffset, IdxT>, OutT* out,
                                              std::int64_t off, Func& f, const map_pack_set<R>&,
                                              const map_pack<Done, R>&... xs)
{
  map_pack<OutT, R> o;
#pragma unroll
  for (int j = 0; j < R; ++j)
    o.v[j] = map_apply<PassOffset, OutT, IdxT, Func, Done...>(f, static_cast<IdxT>(off + j),
                                                              xs.v[j]...);
  map_store<OutT, R>(out, off, o);
}
template <int R, bool PassOffset, typename IdxT, typename OutT, typename Func, typename T,
          typename... Rest, typename... Done>
__device__ __forceinline__ void map_store_set(map_cfg<R, PassOffset, IdxT> cfg, OutT* out,
                                              std::int64_t off, Func& f,
                                              const map_pack_set<R, T, Rest...>& s,
                                              const map_pack<Done, R>&... xs)
{
  map_store_set(cfg, out, off, f, s.tail, xs..., s.head);
}

template <int R, bool PassOffset, typename OutT, typename IdxT, typename Func, typename... InTs>
__global__ __launch_bounds__(kMapBlock) void map_kernel(OutT* out, std::int64_t len, Func f,
                                                        const InTs*... ins)
{
  const std::int64_t npack = len / R;
  const std::int64_t p0 =
    (std::int64_t)blockIdx.x * (kMapBlock * kMapUnroll) + (std::int64_t)threadIdx.x;
  map_pack_set<R, InTs...> held[kMapUnroll];
  if (npack > 0) {
    // unconditional loads (a pack past the end re-reads the last one): under a lane mask
    // the compiler waits for every load in turn
#pragma unroll
    for (int u = 0; u < kMapUnroll; ++u) {
      const std::int64_t p = p0 + (std::int64_t)u * kMapBlock;
      map_load_set(held[u], (p < npack ? p : npack - 1) * R, ins...);
    }
  }
#pragma unroll
  for (int u = 0; u < kMapUnroll; ++u) {
    const std::int64_t p = p0 + (std::int64_t)u * kMapBlock;
    if (p < npack) map_store_set(map_cfg<R, PassOffset, IdxT>{}, out, p * R, f, held[u]);
  }
  // the last len % R elements, one per lane of the first workgroup
  const std::int64_t i = npack * R + (std::int64_t)threadIdx.x;
  if (blockIdx.x == 0 && i < len)
    out[i] = map_apply<PassOffset, OutT, IdxT, Func, InTs...>(f, static_cast<IdxT>(i), ins[i]...);
}

template <typename T>
constexpr int map_ratio_of()
{
  // elements per 16-byte access, or 1 for types that do not tile 16 bytes
  if constexpr (std::is_trivially_copyable_v<T> && sizeof(T) <= 16 && (16 % sizeof(T)) == 0) {
    return 16 / (int)sizeof(T);
  } else {
    return 1;
  }
}

constexpr int map_min(int a) { return a; }
template <typename... I>
constexpr int map_min(int a, int b, I... rest)
{
  return map_min(a < b ? a : b, rest...);
}

template <bool PassOffset, typename OutT, typename IdxT, typename Func, typename... InTs>
void map(hipStream_t stream, OutT* out_ptr, IdxT len, Func f, const InTs*... in_ptrs)
{
  if (len <= 0) return;
  constexpr int R          = map_min(map_ratio_of<OutT>(), map_ratio_of<InTs>()...);
  const std::int64_t n     = (std::int64_t)len;
  const std::int64_t npack = n / R;
  std::int64_t blocks      = (npack + kMapBlock * kMapUnroll - 1) / (kMapBlock * kMapUnroll);
  if (blocks < 1) blocks = 1;
  RAFT_EXPECTS(blocks <= 0x7fffffffLL, "map: too many elements for one launch");
  hipLaunchKernelGGL((map_kernel<R, PassOffset, OutT, IdxT, Func, InTs...>),
                     dim3((unsigned)blocks), dim3(kMapBlock), 0, stream, out_ptr, n, f,
                     in_ptrs...);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess)
    throw raft::hip_error(std::string("HIP error encountered at: map_kernel: ") +
                          hipGetErrorString(e));
}

template <typename OutType, typename InType>
void map_check_shape(OutType out, InType in)
{
  RAFT_EXPECTS(in.is_exhaustive() && out.size() == in.size(),
               "All inputs must be contiguous and have the same size as the output");
}

template <bool PassOffset, typename OutType, typename Func, typename... InTypes>
void map(const raft::resources& res, OutType out, Func f, InTypes... ins)
{
  RAFT_EXPECTS(out.is_exhaustive(), "Output must be contiguous");
  (map_check_shape(out, ins), ...);
  map<PassOffset, typename OutType::value_type, typename OutType::index_type, Func,
      typename InTypes::value_type...>(resource::get_cuda_stream(res), out.data_handle(),
                                       static_cast<typename OutType::index_type>(out.size()), f,
                                       ins.data_handle()...);
}

}  // namespace linalg::detail
}  // namespace raft
