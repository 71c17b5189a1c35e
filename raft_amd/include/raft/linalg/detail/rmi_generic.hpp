// Reductions with ARBITRARY device functors, for translation units compiled by
// hipcc.  The closed functor vocabulary goes through the C ABI of the reduction
// library; anything else (device lambdas, caller-defined functor structs, output
// types the library does not know) cannot cross a C ABI and is instantiated here,
// in the caller's translation unit, the way the reference instantiates all of its
// kernels (linalg/detail/coalesced_reduction-inl.cuh, detail/strided_reduction.cuh).
//
// Semantics are the reference's: every participating lane starts from `init`
// (which therefore has to be reduce_op's neutral element), main_op receives the
// index along the reduced axis, and
//   dots[k] = final_op(inplace ? reduce_op(dots[k], acc) : acc).
// Unlike the reference there are no atomics: partial results of the strided and
// split plans are folded in a fixed order, so results are repeatable.
//
// The kernels are wave64 / gfx950 code: 16-byte lane loads for arithmetic element
// types, ds_bpermute butterflies on 32-bit words for accumulators of any trivially
// copyable type, LDS across waves.  They are simpler than the library's tuned
// kernels.  Accumulation happens in OutType with the caller's reduce_op, exactly as
// written, with one exception the reference makes too
// (coalesced_reduction-inl.cuh:255,421,568, strided_reduction.cuh:146): when reduce_op is
// raft::add_op and OutType is float or double, lanes, workgroups and partial results carry
// a wider sum (fp64 for float; a Kahan-Babuska-Neumaier pair for double) that is rounded
// to OutType once, before final_op.
#pragma once

#if !defined(__HIPCC__)
#error "rmi_generic.hpp holds device code: include it only from hipcc translation units"
#endif

#include <hip/hip_runtime.h>

#include <cstdint>
#include <map>
#include <mutex>
#include <string>
#include <type_traits>

#include <raft/core/error.hpp>
#include <raft/core/operators.hpp>
#include <raft/linalg/detail/map.cuh>
#include <raft/linalg/detail/rmi_scratch.hpp>

namespace raft::detail::rmi::generic {

constexpr int kWave  = 64;
constexpr int kBlock = 256;

template <typename T>
__device__ __forceinline__ T shfl_xor_any(const T& v, int mask)
{
  static_assert(std::is_trivially_copyable_v<T>, "accumulators must be trivially copyable");
  constexpr int NW = (sizeof(T) + 3) / 4;
  std::uint32_t w[NW] = {};
  __builtin_memcpy(w, &v, sizeof(T));
#pragma unroll
  for (int i = 0; i < NW; ++i)
    w[i] = (std::uint32_t)__shfl_xor((int)w[i], mask, kWave);
  T r;
  __builtin_memcpy(&r, w, sizeof(T));
  return r;
}

// all-reduce over groups of G lanes (G a power of two <= 64); reduce_op must be
// commutative for every lane to end with the same value, which the callers below
// do not rely on: only lane 0 of a group uses the result.
template <typename T, typename Red>
__device__ __forceinline__ T group_reduce(T acc, int G, Red& red)
{
  for (int m = G >> 1; m >= 1; m >>= 1)
    acc = red(acc, shfl_xor_any(acc, m));
  return acc;
}

// ---- wider accumulators for sums --------------------------------------------------------
// sum + running compensation (Kahan-Babuska-Neumaier); value = s + c
struct kbn_sum {
  double s, c;
  kbn_sum() = default;
  __host__ __device__ kbn_sum(double v) : s(v), c(0.0) {}
  __host__ __device__ explicit operator double() const { return s + c; }
};
struct wide_add {
  __host__ __device__ double operator()(double a, double b) const { return a + b; }
  __host__ __device__ kbn_sum operator()(const kbn_sum& a, const kbn_sum& b) const
  {
    kbn_sum r;
    r.s = a.s + b.s;
    // the low-order bits that the addition dropped, taken from the smaller operand
    const double lost = (a.s < 0 ? -a.s : a.s) >= (b.s < 0 ? -b.s : b.s) ? (a.s - r.s) + b.s
                                                                          : (b.s - r.s) + a.s;
    r.c = (a.c + b.c) + lost;
    return r;
  }
};
template <typename Out>
struct wide_sum {
  using type = Out;
};
template <>
struct wide_sum<float> {
  using type = double;
};
template <>
struct wide_sum<double> {
  using type = kbn_sum;
};
template <typename Out, typename Red>
constexpr bool sums_wide()
{
  return std::is_same_v<Red, raft::add_op> && (std::is_same_v<Out, float> || std::is_same_v<Out, double>);
}
// final_op behind the rounding of a wide sum to the caller's OutType
template <typename Out, typename Fin>
struct narrow_then {
  Fin fin;
  template <typename Acc>
  __host__ __device__ auto operator()(const Acc& a) const
  {
    return fin(static_cast<Out>(static_cast<double>(a)));
  }
};

// One 16-byte lane load (global_load_dwordx4) at any element-aligned address.  The input
// is streamed once, so the load is marked non-temporal, except where the cache lines of a
// load instruction are shared with the next one (rows of a lane-group kernel that do not
// fill 128-byte lines: 1M x 100 floats read 58 % of 8 TB/s with plain loads, 39 % without
// the lines being kept).
struct alignas(4) pack16 {
  std::uint32_t w[4];
};
template <bool NT = true>
__device__ __forceinline__ pack16 load_pack16(const void* p)
{
  typedef std::uint32_t u32x4 __attribute__((ext_vector_type(4)));
  typedef u32x4 u32x4_unaligned __attribute__((aligned(1)));
  u32x4 v;
  if constexpr (NT) {
    v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_unaligned*>(p));
  } else {
    v = *reinterpret_cast<const u32x4_unaligned*>(p);
  }
  pack16 r;
  r.w[0] = v[0], r.w[1] = v[1], r.w[2] = v[2], r.w[3] = v[3];
  return r;
}

// V elements at `p`: one non-temporal 16-byte lane load when V > 1, else one element
template <int V, typename In>
__device__ __forceinline__ void load_elems(const In* p, In (&x)[V])
{
  if constexpr (V > 1) {
    const pack16 raw = load_pack16(p);
    __builtin_memcpy(x, raw.w, 16);
  } else if constexpr (std::is_arithmetic_v<In>) {
    x[0] = __builtin_nontemporal_load(p);
  } else {
    x[0] = *p;
  }
}

// elements per 16-byte lane load, or 1 when the element type is not a power-of-two
// sized arithmetic type
template <typename In>
constexpr int vec_width()
{
  if constexpr (std::is_arithmetic_v<In> && (sizeof(In) == 1 || sizeof(In) == 2 ||
                                             sizeof(In) == 4 || sizeof(In) == 8)) {
    return 16 / (int)sizeof(In);
  } else {
    return 1;
  }
}

// acc = fold of main_op(row[j], j0 + j) over the D elements at `row`: whole 16-byte
// vectors first + k * stride (four lane loads in flight), then the tail elements.
// j0 is the position of row[0] along the reduced axis.
template <typename In, typename Out, typename Idx, bool NT = true, typename Main, typename Red>
__device__ __forceinline__ Out sweep_row(const In* row, Idx D, int first, int stride, Out acc,
                                         Main& main_op, Red& red, Idx j0 = 0)
{
  constexpr int V = vec_width<In>();
  if constexpr (V > 1) {
    constexpr int U = 4;
    using pack       = pack16;
    const Idx nvec   = D / V;
    const char* base = reinterpret_cast<const char*>(row);
    auto take = [&](const pack& raw, Idx v) {
      In x[V];
      __builtin_memcpy(x, raw.w, 16);
#pragma unroll
      for (int j = 0; j < V; ++j)
        acc = red(acc, static_cast<Out>(main_op(x[j], static_cast<Idx>(j0 + v * V + j))));
    };
    Idx v = first;
    for (; v + (Idx)(U - 1) * stride < nvec; v += (Idx)U * stride) {
      pack raw[U];
#pragma unroll
      for (int u = 0; u < U; ++u)
        raw[u] = load_pack16<NT>(base + (std::size_t)(v + (Idx)u * stride) * 16);
#pragma unroll
      for (int u = 0; u < U; ++u)
        take(raw[u], v + (Idx)u * stride);
    }
    for (; v < nvec; v += stride) {
      take(load_pack16<NT>(base + (std::size_t)v * 16), v);
    }
    for (Idx j = nvec * V + first; j < D; j += stride)
      acc = red(acc, static_cast<Out>(main_op(row[j], static_cast<Idx>(j0 + j))));
  } else {
    for (Idx j = first; j < D; j += stride)
      acc = red(acc, static_cast<Out>(main_op(row[j], static_cast<Idx>(j0 + j))));
  }
  return acc;
}

// G lanes of a wave per row (rows are contiguous, D elements each)
template <typename In, typename Out, typename Idx, typename Main, typename Red, typename Fin,
          typename Dst>
__global__ __launch_bounds__(kBlock) void rows_group_kernel(Dst* dots, const In* data, Idx D,
                                                            Idx N, Out init, bool inplace,
                                                            Main main_op, Red red, Fin fin,
                                                            int G, int logG, bool nt)
{
  const int lane         = threadIdx.x & (kWave - 1);
  const std::int64_t wid = (std::int64_t)blockIdx.x * (kBlock / kWave) + (threadIdx.x >> 6);
  const int c            = lane & (G - 1);
  const std::int64_t row = wid * (kWave >> logG) + (lane >> logG);
  Out acc                = init;
  if (row < (std::int64_t)N) {
    acc = nt ? sweep_row<In, Out, Idx, true>(data + row * D, D, c, G, acc, main_op, red)
             : sweep_row<In, Out, Idx, false>(data + row * D, D, c, G, acc, main_op, red);
  }
  acc = group_reduce(acc, G, red);
  if (c == 0 && row < (std::int64_t)N)
    dots[row] = fin(inplace ? red(static_cast<Out>(dots[row]), acc) : acc);
}

// Rows of G 16-byte lane loads, G not a power of two (3..32, the row's last load may be the
// pack that ends at the row's end): one lane per load, 64 / G whole rows per wave step, four
// steps in flight, so every load instruction covers one contiguous span of the matrix; the
// wave's last 64 % G lanes idle.  Lanes of a row are folded into its first one (lane c takes
// lane c + s for s = 1, 2, 4 ...).
template <typename T>
__device__ __forceinline__ T shfl_any(const T& v, int src)
{
  constexpr int NW = (sizeof(T) + 3) / 4;
  std::uint32_t w[NW] = {};
  __builtin_memcpy(w, &v, sizeof(T));
#pragma unroll
  for (int i = 0; i < NW; ++i)
    w[i] = (std::uint32_t)__shfl((int)w[i], src, kWave);
  T r;
  __builtin_memcpy(&r, w, sizeof(T));
  return r;
}

template <typename In, typename Out, typename Idx, typename Main, typename Red, typename Fin,
          typename Dst>
__global__ __launch_bounds__(kBlock) void rows_anyg_kernel(Dst* dots, const In* data, Idx D, Idx N,
                                                           Out init, bool inplace, Main main_op,
                                                           Red red, Fin fin, int G, unsigned invG)
{
  constexpr int V = vec_width<In>();
  constexpr int U = 4;
  const int lane  = threadIdx.x & (kWave - 1);
  const std::int64_t wid = (std::int64_t)blockIdx.x * (kBlock / kWave) + (threadIdx.x >> 6);
  const int R     = kWave / G;
  const int g     = (int)(((unsigned)lane * invG) >> 16);  // lane / G
  const int c     = lane - g * G;
  const bool live = g < R;
  const std::int64_t nvec = (std::int64_t)D / V;
  const int tail          = (int)((std::int64_t)D - nvec * V);
  // element offset of this lane's pack: whole pack c, or the pack that ends at the row's end
  const bool last_part    = tail > 0 && c == G - 1;
  const std::int64_t e0   = !live ? 0 : (last_part ? (std::int64_t)D - V : (std::int64_t)c * V);
  const int first         = last_part ? V - tail : 0;  // elements before it are the neighbour's
  pack16 x[U];
  std::int64_t row[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {  // unconditional loads: a row past the matrix re-reads the last one
    row[u] = (wid * U + u) * R + g;
    const std::int64_t rl = row[u] < (std::int64_t)N ? row[u] : (std::int64_t)N - 1;
    x[u] = load_pack16<false>(data + rl * (std::int64_t)D + e0);
  }
  Out acc[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    acc[u] = init;
    if (live && row[u] < (std::int64_t)N) {
      In e[V];
      __builtin_memcpy(e, x[u].w, 16);
#pragma unroll
      for (int j = 0; j < V; ++j)
        if (j >= first) acc[u] = red(acc[u], static_cast<Out>(main_op(e[j], static_cast<Idx>(e0 + j))));
    }
  }
  for (int s = 1; s < G; s <<= 1) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const Out v = shfl_any(acc[u], lane + s);
      if (c + s < G) acc[u] = red(acc[u], v);
    }
  }
#pragma unroll
  for (int u = 0; u < U; ++u)
    if (live && c == 0 && row[u] < (std::int64_t)N)
      dots[row[u]] = fin(inplace ? red(static_cast<Out>(dots[row[u]]), acc[u]) : acc[u]);
}

// one 256-thread workgroup per chunk of a row; B chunks per row.  B == 1 writes the
// outputs, B > 1 writes partials[row * B + b].
template <typename In, typename Out, typename Idx, typename Main, typename Red, typename Fin,
          typename Dst>
__global__ __launch_bounds__(kBlock) void rows_block_kernel(Dst* dots, Out* partial,
                                                            const In* data, Idx D, Idx N, Out init,
                                                            bool inplace, Main main_op, Red red,
                                                            Fin fin, int B, std::int64_t chunk)
{
  __shared__ Out sm[kBlock / kWave];
  const std::int64_t row = blockIdx.x / B;
  const int b            = blockIdx.x % B;
  const std::int64_t j0  = (std::int64_t)b * chunk;
  const std::int64_t j1  = j0 + chunk < (std::int64_t)D ? j0 + chunk : (std::int64_t)D;
  Out acc                = init;
  if (j1 > j0)
    acc = sweep_row<In, Out, Idx>(data + row * D + j0, (Idx)(j1 - j0), (int)threadIdx.x, kBlock,
                                  acc, main_op, red, (Idx)j0);
  acc = group_reduce(acc, kWave, red);
  if ((threadIdx.x & (kWave - 1)) == 0) sm[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kBlock / kWave; ++w)
      acc = red(acc, sm[w]);
    if (B == 1) {
      dots[row] = fin(inplace ? red(static_cast<Out>(dots[row]), acc) : acc);
    } else {
      partial[row * B + b] = acc;
    }
  }
}

// strided: data is N rows of D contiguous elements, one output per column.
// A thread owns V adjacent columns for the whole kernel: V = elements per 16-byte lane load
// (at any element-aligned address) when a row holds at least one, else 1.  A row length that
// is not a multiple of V ends with one more lane whose vector ends at the row's end; its
// first V - D % V columns belong to the lane before it and are dropped at the end.
// Thread t is lane t % TX of row t / TX of a step; TX is the row's lane count itself up to
// 128 (an equal cut of it beyond), TY = 256 / TX whole rows per step, so a step reads one
// contiguous span and the last 256 - TX * TY threads idle.  blockIdx.y strides over the steps
// with four independent loads in flight per thread; the rows of a step are combined
// through LDS.
template <int V, typename In, typename Out, typename Idx, typename Main, typename Red, typename Fin,
          typename Dst>
__global__ __launch_bounds__(kBlock) void cols_kernel(Dst* dots, Out* partial, const In* data,
                                                      Idx D, Idx N, Out init, bool inplace,
                                                      Main main_op, Red red, Fin fin, int TX,
                                                      int TY, int treeTY, int B)
{
  constexpr int U = 4;
  struct pack {
    In x[V];
  };
  __shared__ Out sm[kBlock * V];
  const int t             = threadIdx.x;
  const int ty            = (int)((unsigned)t / (unsigned)TX);
  const int tx            = t - ty * TX;
  const std::int64_t lane = (std::int64_t)blockIdx.x * TX + tx;  // lane load along the row
  const std::int64_t nw   = (std::int64_t)D / V;                 // whole lane loads
  const int tail          = (int)((std::int64_t)D - nw * V);
  const bool whole        = lane < nw;
  const bool part         = V > 1 && lane == nw && tail > 0;
  const std::int64_t col0 = whole ? lane * V : (std::int64_t)D - V;  // first column owned
  Out acc[V];
#pragma unroll
  for (int j = 0; j < V; ++j)
    acc[j] = init;
  if (ty < TY && (whole || part)) {
    const In* p             = data + col0;
    const std::int64_t step = (std::int64_t)B * TY;
    std::int64_t r          = (std::int64_t)blockIdx.y * TY + ty;
    for (; r + (U - 1) * step < (std::int64_t)N; r += U * step) {
      pack x[U];
#pragma unroll
      for (int u = 0; u < U; ++u)
        load_elems<V>(p + (r + u * step) * (std::int64_t)D, x[u].x);
#pragma unroll
      for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int j = 0; j < V; ++j)
          acc[j] = red(acc[j], static_cast<Out>(main_op(x[u].x[j], static_cast<Idx>(r + u * step))));
      }
    }
    for (; r < (std::int64_t)N; r += step) {
      pack x;
      load_elems<V>(p + r * (std::int64_t)D, x.x);
#pragma unroll
      for (int j = 0; j < V; ++j)
        acc[j] = red(acc[j], static_cast<Out>(main_op(x.x[j], static_cast<Idx>(r))));
    }
  }
#pragma unroll
  for (int j = 0; j < V; ++j)
    sm[t * V + j] = acc[j];
  __syncthreads();
  for (int s = treeTY >> 1; s >= 1; s >>= 1) {
    if (ty < s && ty + s < TY) {
#pragma unroll
      for (int j = 0; j < V; ++j)
        sm[t * V + j] = red(sm[t * V + j], sm[(t + s * TX) * V + j]);
    }
    __syncthreads();
  }
  if (ty == 0 && (whole || part)) {
    const int first = whole ? 0 : V - tail;
#pragma unroll
    for (int j = 0; j < V; ++j) {
      if (j >= first) {
        const std::int64_t col = col0 + j;
        if (B == 1) {
          dots[col] = fin(inplace ? red(static_cast<Out>(dots[col]), sm[t * V + j]) : sm[t * V + j]);
        } else {
          partial[col * B + blockIdx.y] = sm[t * V + j];
        }
      }
    }
  }
}

// second pass over partials[n_out][B]: LB lanes of a wave per output (LB a power of
// two <= 64), each folding every LB-th partial, then a butterfly: a fixed order
template <typename Out, typename Red, typename Fin, typename Dst>
__global__ __launch_bounds__(kBlock) void fold_kernel(Dst* dots, const Out* partial,
                                                      std::int64_t n_out, int B, Out init,
                                                      bool inplace, Red red, Fin fin, int LB,
                                                      int logLB)
{
  const std::int64_t gtid = (std::int64_t)blockIdx.x * kBlock + threadIdx.x;
  const std::int64_t o    = gtid >> logLB;
  const int lb            = (int)(gtid & (LB - 1));
  Out acc                 = init;
  if (o < n_out) {
    const Out* p = partial + o * B;
    int b        = lb;
    for (; b + 7 * LB < B; b += 8 * LB) {  // eight loads in flight, folded in order
      Out x[8];
#pragma unroll
      for (int u = 0; u < 8; ++u)
        x[u] = p[b + u * LB];
#pragma unroll
      for (int u = 0; u < 8; ++u)
        acc = red(acc, x[u]);
    }
    for (; b < B; b += LB)
      acc = red(acc, p[b]);
  }
  acc = group_reduce(acc, LB, red);
  if (lb == 0 && o < n_out) dots[o] = fin(inplace ? red(static_cast<Out>(dots[o]), acc) : acc);
}

inline int pow2ceil(std::int64_t x)
{
  int p = 1;
  while (p < x)
    p <<= 1;
  return p;
}
inline int ilog2(int x)
{
  int l = 0;
  while ((1 << l) < x)
    ++l;
  return l;
}

// CUs of the current device, asked once per device (the library's planner does the same);
// grids that aim at "k workgroups per CU" are sized from it.
inline int cu_count()
{
  static std::mutex guard;
  static std::map<int, int> by_device;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    (void)hipGetLastError();
    return 256;
  }
  std::lock_guard<std::mutex> lock(guard);
  auto it = by_device.find(dev);
  if (it != by_device.end()) return it->second;
  int n = 0;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
    (void)hipGetLastError();
    n = 256;
  }
  by_device.emplace(dev, n);
  return n;
}

inline void check_launch(const char* what)
{
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess)
    throw raft::hip_error(std::string("HIP error encountered at: ") + what + ": " +
                          hipGetErrorString(e));
}

template <typename Out, typename Red, typename Fin, typename Dst>
void launch_fold(Dst* dots, const Out* partial, std::int64_t n_out, int B, Out init, bool inplace,
                 Red red, Fin fin, hipStream_t stream)
{
  const int LB             = B >= 64 ? 64 : pow2ceil(B);
  const std::int64_t grid  = (n_out * LB + kBlock - 1) / kBlock;
  hipLaunchKernelGGL((fold_kernel<Out, Red, Fin, Dst>), dim3((unsigned)grid), dim3(kBlock), 0, stream,
                     dots, partial, n_out, B, init, inplace, red, fin, LB, ilog2(LB));
}

// dots[N] from N contiguous rows of D elements
template <typename In, typename Out, typename Idx, typename Main, typename Red, typename Fin,
          typename Dst>
void coalesced(Dst* dots, const In* data, Idx D, Idx N, Out init, hipStream_t stream, bool inplace,
               Main main_op, Red red, Fin fin)
{
  if (N <= 0) return;
  constexpr int V           = vec_width<In>();
  const std::int64_t nloads = ((std::int64_t)D + V - 1) / V;
  if constexpr (V > 1) {
    // lane-load counts that are not a power of two: one lane per load, whole rows per wave step
    // (accumulators wider than 8 bytes pay twice per cross-lane step: up to 12 loads only)
    if (nloads >= 3 && nloads <= (sizeof(Out) > 8 ? 12 : 32) && (nloads & (nloads - 1)) != 0 &&
        (std::int64_t)D >= V && (kWave / nloads) * nloads >= 48) {
      const int G              = (int)nloads;
      const int rows_per_block = (kWave / G) * 4 * (kBlock / kWave);
      const std::int64_t grid  = ((std::int64_t)N + rows_per_block - 1) / rows_per_block;
      hipLaunchKernelGGL((rows_anyg_kernel<In, Out, Idx, Main, Red, Fin, Dst>), dim3((unsigned)grid),
                         dim3(kBlock), 0, stream, dots, data, D, N, init, inplace, main_op, red, fin,
                         G, 65536u / (unsigned)G + 1);
      check_launch("rows_anyg_kernel");
      return;
    }
  }
  if (nloads <= 256 || (std::int64_t)N >= 8192) {
    // lanes per row: about four loads per lane
    std::int64_t g = (nloads + 3) / 4;
    const int G    = g >= 64 ? 64 : pow2ceil(g < 1 ? 1 : g);
    const int rows_per_block = (kWave / G) * (kBlock / kWave);
    // non-temporal loads where no cache line is shared between load instructions
    const bool nt = ((std::int64_t)D * (std::int64_t)sizeof(In)) % 128 == 0 &&
                    reinterpret_cast<std::uintptr_t>(data) % 128 == 0;
    const std::int64_t grid  = ((std::int64_t)N + rows_per_block - 1) / rows_per_block;
    hipLaunchKernelGGL((rows_group_kernel<In, Out, Idx, Main, Red, Fin, Dst>), dim3((unsigned)grid),
                       dim3(kBlock), 0, stream, dots, data, D, N, init, inplace, main_op, red, fin,
                       G, ilog2(G), nt);
    check_launch("rows_group_kernel");
    return;
  }
  // few long rows: split each into B chunks so that the grid fills the device
  // chunks are whole multiples of one block sweep (256 lanes x 4 loads x V elements), so
  // every chunk starts on a vector boundary of its row
  constexpr std::int64_t quantum = (std::int64_t)kBlock * 4 * V;
  std::int64_t B = ((std::int64_t)4 * cu_count() + (std::int64_t)N - 1) / (std::int64_t)N;
  const std::int64_t max_b = ((std::int64_t)D + quantum - 1) / quantum;
  if (B > max_b) B = max_b;
  if (B < 1) B = 1;
  std::int64_t chunk = ((std::int64_t)D + B - 1) / B;
  chunk              = (chunk + quantum - 1) / quantum * quantum;
  B                  = ((std::int64_t)D + chunk - 1) / chunk;
  Out* partial             = nullptr;
  if (B > 1) partial = static_cast<Out*>(scratch_alloc(sizeof(Out) * (std::size_t)N * B, stream));
  hipLaunchKernelGGL((rows_block_kernel<In, Out, Idx, Main, Red, Fin, Dst>),
                     dim3((unsigned)((std::int64_t)N * B)), dim3(kBlock), 0, stream, dots, partial,
                     data, D, N, init, inplace, main_op, red, fin, (int)B, chunk);
  check_launch("rows_block_kernel");
  if (B > 1) {
    launch_fold(dots, partial, (std::int64_t)N, (int)B, init, inplace, red, fin, stream);
    check_launch("fold_kernel");
    scratch_free(partial, stream);
  }
}

template <int V, typename In, typename Out, typename Idx, typename Main, typename Red, typename Fin,
          typename Dst>
void launch_cols(Dst* dots, const In* data, Idx D, Idx N, Out init, hipStream_t stream, bool inplace,
                 Main main_op, Red red, Fin fin)
{
  const std::int64_t lanes = ((std::int64_t)D + V - 1) / V;
  const std::int64_t cuts  = (lanes + 127) / 128;
  const int TX             = (int)((lanes + cuts - 1) / cuts);
  const int TY             = kBlock / TX;
  const std::int64_t gridx = (lanes + TX - 1) / TX;
  // 16-byte lane loads: two workgroups per CU read one compact, advancing window of the
  // matrix (measured 74 % of 8 TB/s on 10M x 64 floats where 1024 workgroups give 63 %);
  // element loads want eight times as many in flight.  At least four steps each.
  // (rounded down: one workgroup more lands on a CU that then finishes last)
  std::int64_t B           = ((std::int64_t)cu_count() * (V > 1 ? 2 : 16)) / gridx;
  const std::int64_t max_b = ((std::int64_t)N + 4 * TY - 1) / (4 * TY);
  if (B > max_b) B = max_b;
  if (B < 1) B = 1;
  if (B > 4096) B = 4096;
  Out* partial = nullptr;
  if (B > 1) partial = static_cast<Out*>(scratch_alloc(sizeof(Out) * (std::size_t)D * B, stream));
  hipLaunchKernelGGL((cols_kernel<V, In, Out, Idx, Main, Red, Fin, Dst>),
                     dim3((unsigned)gridx, (unsigned)B), dim3(kBlock), 0, stream, dots, partial,
                     data, D, N, init, inplace, main_op, red, fin, TX, TY, pow2ceil(TY), (int)B);
  check_launch("cols_kernel");
  if (B > 1) {
    launch_fold(dots, partial, (std::int64_t)D, (int)B, init, inplace, red, fin, stream);
    check_launch("fold_kernel");
    scratch_free(partial, stream);
  }
}

// ---- columns of wide rows ------------------------------------------------------------------
// Rows of more than 128 lane-loads: a workgroup streams whole adjacent rows (of rows that
// outgrow its load slots, one of the fewest equal pieces), i.e. long contiguous spans, where
// cols_kernel reads pieces of at most 2 KB at the row's stride.  A thread has K load slots
// with V accumulators each, as many as 256 bytes hold (at most 5); the workgroup's 256 * K
// slots are dealt densely over the lane-loads of `rb` adjacent rows (a bundle): slot k of
// thread t is lane-load (256 k + t) % piece of row (256 k + t) / piece, so a slot always meets
// the same columns.  R bundles are in flight, every load issued before the first use and none
// under a condition (idle slots load the piece's first vector, run the caller's main_op and
// reduce_op on it like every other slot, and are dropped: functors must be free of side
// effects, as the reference's are).  At the end the
// rows of a bundle are combined through LDS in row order and the partials are stored
// [workgroup][column], whole lines at a time; fold_rows_kernel is the second pass.
template <typename Out, int V>
constexpr int cols_wide_slots()
{
  constexpr int k = 256 / (V * (int)sizeof(Out));
  return k < 1 ? 1 : (k > 5 ? 5 : k);
}
constexpr int cols_wide_bundles(int K) { return (10 + K - 1) / K; }

template <int V, typename In, typename Out, typename Idx, typename Main, typename Red>
__global__ __launch_bounds__(kBlock) void cols_wide_kernel(Out* partial, const In* data, Idx D,
                                                           Idx N, Out init, Main main_op, Red red,
                                                           int piece, int rb, int B)
{
  static_assert(std::is_trivially_copyable_v<Out>, "accumulators must be trivially copyable");
  constexpr int K = cols_wide_slots<Out, V>();
  constexpr int R = cols_wide_bundles(K);
  extern __shared__ __align__(16) unsigned char cols_wide_lds[];
  Out* sm                  = reinterpret_cast<Out*>(cols_wide_lds);  // [rb][lane-loads of the piece * V]
  const int t              = threadIdx.x;
  const std::int64_t nvec  = (std::int64_t)D / V;
  const int tail           = (int)((std::int64_t)D - nvec * V);
  const std::int64_t total = nvec + (tail > 0 ? 1 : 0);
  const std::int64_t l0    = (std::int64_t)blockIdx.x * piece;
  const int nload          = (int)(total - l0 < piece ? total - l0 : piece);
  // element offset of lane-load l within a row: whole vector l, or the vector that ends at the
  // row's end (its first V - tail columns belong to the lane-load before it)
  auto first_col = [&](std::int64_t l) { return l < nvec ? l * V : (std::int64_t)D - V; };
  std::int64_t off[K];
  int sub[K], lane[K];
  bool live[K];
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const unsigned f = (unsigned)(k * kBlock + t);
    const unsigned q = f / (unsigned)piece;
    sub[k]           = (int)q;
    lane[k]          = (int)(f - q * (unsigned)piece);
    live[k]          = (int)q < rb && lane[k] < nload;
    off[k] = live[k] ? (std::int64_t)q * (std::int64_t)D + first_col(l0 + lane[k]) : first_col(l0);
  }
  Out acc[K][V];
#pragma unroll
  for (int k = 0; k < K; ++k)
#pragma unroll
    for (int j = 0; j < V; ++j)
      acc[k][j] = init;

  const std::int64_t step   = (std::int64_t)R * rb;
  const std::int64_t stride = (std::int64_t)B * step;
  std::int64_t r            = (std::int64_t)blockIdx.y * step;
  for (; r + step <= (std::int64_t)N; r += stride) {
    pack16 x[R][K];
#pragma unroll
    for (int q = 0; q < R; ++q)
#pragma unroll
      for (int k = 0; k < K; ++k)
        x[q][k] = load_pack16<true>(data + (r + (std::int64_t)q * rb) * (std::int64_t)D + off[k]);
    __builtin_amdgcn_sched_barrier(0);  // all of the step's loads before the first use
#pragma unroll
    for (int q = 0; q < R; ++q)
#pragma unroll
      for (int k = 0; k < K; ++k) {
        In e[V];
        __builtin_memcpy(e, x[q][k].w, 16);
        const Idx row = static_cast<Idx>(r + (std::int64_t)q * rb + sub[k]);
#pragma unroll
        for (int j = 0; j < V; ++j)
          acc[k][j] = red(acc[k][j], static_cast<Out>(main_op(e[j], row)));
      }
  }
  // the rows after the last whole step go to the workgroup whose turn it is, bundle by bundle
  for (; r < (std::int64_t)N; r += rb) {
#pragma unroll
    for (int k = 0; k < K; ++k)
      if (live[k] && r + sub[k] < (std::int64_t)N) {
        const pack16 x = load_pack16<true>(data + r * (std::int64_t)D + off[k]);
        In e[V];
        __builtin_memcpy(e, x.w, 16);
#pragma unroll
        for (int j = 0; j < V; ++j)
          acc[k][j] = red(acc[k][j], static_cast<Out>(main_op(e[j], static_cast<Idx>(r + sub[k]))));
      }
  }

  const int width = nload * V;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    if (live[k]) {
#pragma unroll
      for (int j = 0; j < V; ++j)
        sm[sub[k] * width + lane[k] * V + j] = acc[k][j];
    }
  }
  __syncthreads();
  Out* out = partial + (std::int64_t)blockIdx.y * (std::int64_t)D;
  for (int idx = t; idx < width; idx += kBlock) {
    const int ll = idx / V, j = idx - ll * V;
    const std::int64_t l = l0 + ll;
    if (l == nvec && j < V - tail) continue;  // columns of the lane-load before the last, partial one
    Out v = sm[idx];
    for (int q = 1; q < rb; ++q)
      v = red(v, sm[q * width + idx]);
    out[l < nvec ? l * V + j : (std::int64_t)D - V + j] = v;
  }
}

// second pass over partials[B][n_out]: a workgroup folds 16 adjacent outputs; thread (c, s)
// folds partials s, s + 16, ... of output c in that order, then the 16 s in a fixed tree
template <typename Out, typename Red, typename Fin, typename Dst>
__global__ __launch_bounds__(kBlock) void fold_rows_kernel(Dst* dots, const Out* partial,
                                                           std::int64_t n_out, int B, Out init,
                                                           bool inplace, Red red, Fin fin)
{
  __shared__ Out sm[kBlock];
  const int t          = threadIdx.x;
  const int c          = t & 15;
  const int s          = t >> 4;
  const std::int64_t o = (std::int64_t)blockIdx.x * 16 + c;
  Out acc              = init;
  if (o < n_out) {
    const Out* p = partial + o;
    int b        = s;
    for (; b + 7 * 16 < B; b += 8 * 16) {
      Out x[8];
#pragma unroll
      for (int u = 0; u < 8; ++u)
        x[u] = p[(std::int64_t)(b + u * 16) * n_out];
#pragma unroll
      for (int u = 0; u < 8; ++u)
        acc = red(acc, x[u]);
    }
    for (; b < B; b += 16)
      acc = red(acc, p[(std::int64_t)b * n_out]);
  }
  sm[t] = acc;
  __syncthreads();
  for (int h = 8; h >= 1; h >>= 1) {
    if (s < h) sm[t] = red(sm[t], sm[t + h * 16]);
    __syncthreads();
  }
  if (s == 0 && o < n_out) dots[o] = fin(inplace ? red(static_cast<Out>(dots[o]), sm[t]) : sm[t]);
}

// true when the wide-row layout was taken
template <int V, typename In, typename Out, typename Idx, typename Main, typename Red, typename Fin,
          typename Dst>
bool launch_cols_wide(Dst* dots, const In* data, Idx D, Idx N, Out init, hipStream_t stream,
                      bool inplace, Main main_op, Red red, Fin fin)
{
  constexpr int K          = cols_wide_slots<Out, V>();
  const int kCus           = cu_count();  // one workgroup per CU
  const std::int64_t lanes = ((std::int64_t)D + V - 1) / V;
  const std::int64_t slots = (std::int64_t)kBlock * K;
  const std::int64_t cuts  = (lanes + slots - 1) / slots;
  // rows of several pieces that are whole multiples of 64 lane-loads are cols_kernel's best case
  if (lanes <= 128 || cuts > kCus || (cuts > 1 && lanes % 64 == 0 && (std::int64_t)D % V == 0))
    return false;
  const std::int64_t piece = (lanes + cuts - 1) / cuts;
  const std::int64_t rb    = slots / piece;
  const std::int64_t step  = rb * cols_wide_bundles(K);
  const std::int64_t B     = kCus / cuts;
  if ((std::int64_t)N < B * step * 16) return false;  // every workgroup gets sixteen steps
  const std::int64_t gridx = (lanes + piece - 1) / piece;
  Out* partial = static_cast<Out*>(scratch_alloc(sizeof(Out) * (std::size_t)D * B, stream));
  const std::size_t lds = (std::size_t)rb * piece * V * sizeof(Out);  // at most 64 KB
  hipLaunchKernelGGL((cols_wide_kernel<V, In, Out, Idx, Main, Red>),
                     dim3((unsigned)gridx, (unsigned)B), dim3(kBlock), lds, stream, partial, data, D,
                     N, init, main_op, red, (int)piece, (int)rb, (int)B);
  check_launch("cols_wide_kernel");
  hipLaunchKernelGGL((fold_rows_kernel<Out, Red, Fin, Dst>),
                     dim3((unsigned)(((std::int64_t)D + 15) / 16)), dim3(kBlock), 0, stream, dots,
                     partial, (std::int64_t)D, (int)B, init, inplace, red, fin);
  check_launch("fold_rows_kernel");
  scratch_free(partial, stream);
  return true;
}

// dots[D] from N rows of D contiguous elements (one output per column)
template <typename In, typename Out, typename Idx, typename Main, typename Red, typename Fin,
          typename Dst>
void strided(Dst* dots, const In* data, Idx D, Idx N, Out init, hipStream_t stream, bool inplace,
             Main main_op, Red red, Fin fin)
{
  if (D <= 0) return;
  // 16-byte lane loads when a row holds at least one and the per-thread accumulators of a
  // workgroup fit 32 KB of LDS
  constexpr int V = vec_width<In>();
  if constexpr (V > 1 && sizeof(Out) * V * kBlock <= 32 * 1024) {
    if ((std::int64_t)D >= V) {
      if (launch_cols_wide<V, In, Out, Idx>(dots, data, D, N, init, stream, inplace, main_op, red, fin))
        return;
      launch_cols<V, In, Out, Idx>(dots, data, D, N, init, stream, inplace, main_op, red, fin);
      return;
    }
  }
  launch_cols<1, In, Out, Idx>(dots, data, D, N, init, stream, inplace, main_op, red, fin);
}

// layout x axis dispatch of linalg/detail/reduce.cuh:36-48
template <typename In, typename Acc, typename Out, typename Main, typename Red, typename Fin>
void reduce_as(hipStream_t stream, Out* dots, const In* data, std::int64_t n_rows,
               std::int64_t n_cols, bool row_major, bool along_rows, Acc init, bool inplace,
               Main main_op, Red red, Fin fin)
{
  using Idx = std::int64_t;
  const Idx D = row_major ? n_cols : n_rows, N = row_major ? n_rows : n_cols;
  if (row_major == along_rows) {
    // fold the contiguous dimension
    coalesced<In, Acc, Idx>(dots, data, D, N, init, stream, inplace, main_op, red, fin);
  } else {
    strided<In, Acc, Idx>(dots, data, D, N, init, stream, inplace, main_op, red, fin);
  }
}

template <typename In, typename Out, typename Main, typename Red, typename Fin>
void reduce(hipStream_t stream, Out* dots, const In* data, std::int64_t n_rows,
            std::int64_t n_cols, bool row_major, bool along_rows, Out init, bool inplace,
            Main main_op, Red red, Fin fin)
{
  if constexpr (sums_wide<Out, Red>()) {
    using Acc = typename wide_sum<Out>::type;
    reduce_as<In, Acc>(stream, dots, data, n_rows, n_cols, row_major, along_rows,
                       Acc((double)init), inplace, main_op, wide_add{}, narrow_then<Out, Fin>{fin});
  } else {
    reduce_as<In, Out>(stream, dots, data, n_rows, n_cols, row_major, along_rows, init, inplace,
                       main_op, red, fin);
  }
}

// ---- map over several equally long arrays, then reduce to one value -------------------
// out = fold over i of map(in[i], args[i]...) starting from `neutral`
// (linalg/detail/map_then_reduce.cuh:47-95 in the reference, whose blocks accumulate
// into the output with atomics; here partials are folded in a fixed order).  Lanes move
// packs of R elements per array as the elementwise map does.
template <int R, typename Out, typename Map, typename Red, typename... Done>
__device__ __forceinline__ void fold_pack_set(Out& acc, Map& map, Red& red,
                                              const raft::linalg::detail::map_pack_set<R>&,
                                              const raft::linalg::detail::map_pack<Done, R>&... xs)
{
#pragma unroll
  for (int j = 0; j < R; ++j)
    acc = red(acc, static_cast<Out>(map(xs.v[j]...)));
}
template <int R, typename Out, typename Map, typename Red, typename T, typename... Rest,
          typename... Done>
__device__ __forceinline__ void fold_pack_set(
  Out& acc, Map& map, Red& red, const raft::linalg::detail::map_pack_set<R, T, Rest...>& s,
  const raft::linalg::detail::map_pack<Done, R>&... xs)
{
  fold_pack_set<R>(acc, map, red, s.tail, xs..., s.head);
}

template <int R, typename Out, typename Map, typename Red, typename... InTs>
__global__ __launch_bounds__(kBlock) void map_reduce_multi_kernel(Out* partial, std::int64_t len,
                                                                  std::int64_t packs_per_block,
                                                                  Out neutral, Map map, Red red,
                                                                  const InTs*... ins)
{
  constexpr int U = 4;
  __shared__ Out sm[kBlock / kWave];
  const std::int64_t npack = len / R;
  const std::int64_t begin = (std::int64_t)blockIdx.x * packs_per_block;
  const std::int64_t end   = begin + packs_per_block < npack ? begin + packs_per_block : npack;
  Out acc                  = neutral;
  for (std::int64_t p0 = begin + threadIdx.x; p0 < end; p0 += (std::int64_t)kBlock * U) {
    raft::linalg::detail::map_pack_set<R, InTs...> held[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {  // unconditional, clamped: see map_kernel
      const std::int64_t p = p0 + (std::int64_t)u * kBlock;
      raft::linalg::detail::map_load_set(held[u], (p < end ? p : end - 1) * R, ins...);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const std::int64_t p = p0 + (std::int64_t)u * kBlock;
      if (p < end) fold_pack_set<R>(acc, map, red, held[u]);
    }
  }
  // the last len % R elements, on the first workgroup
  const std::int64_t i = npack * R + (std::int64_t)threadIdx.x;
  if (blockIdx.x == 0 && i < len) acc = red(acc, static_cast<Out>(map(ins[i]...)));
  acc = group_reduce(acc, kWave, red);
  if ((threadIdx.x & (kWave - 1)) == 0) sm[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kBlock / kWave; ++w)
      acc = red(acc, sm[w]);
    partial[blockIdx.x] = acc;
  }
}

template <typename Out, typename Dst, typename Map, typename Red, typename Fin, typename... InTs>
void map_reduce_multi_as(hipStream_t stream, Dst* out, std::int64_t len, Out neutral, Map map,
                         Red red, Fin fin, const InTs*... ins)
{
  using raft::linalg::detail::map_min;
  using raft::linalg::detail::map_ratio_of;
  constexpr int R                = map_min(16, map_ratio_of<InTs>()...);
  constexpr std::int64_t quantum = (std::int64_t)kBlock * 4;  // packs per block sweep
  const std::int64_t npack       = len / R;
  std::int64_t B                 = (npack + quantum - 1) / quantum;
  if (B > 1024) B = 1024;
  if (B < 1) B = 1;
  std::int64_t per = (npack + B - 1) / B;
  per              = (per + quantum - 1) / quantum * quantum;
  if (per < quantum) per = quantum;
  B = (npack + per - 1) / per;
  if (B < 1) B = 1;
  Out* partial = static_cast<Out*>(scratch_alloc(sizeof(Out) * (std::size_t)B, stream));
  hipLaunchKernelGGL((map_reduce_multi_kernel<R, Out, Map, Red, InTs...>), dim3((unsigned)B),
                     dim3(kBlock), 0, stream, partial, len, per, neutral, map, red, ins...);
  check_launch("map_reduce_multi_kernel");
  launch_fold(out, partial, (std::int64_t)1, (int)B, neutral, false, red, fin, stream);
  check_launch("fold_kernel");
  scratch_free(partial, stream);
}

template <typename Out, typename Map, typename Red, typename... InTs>
void map_reduce_multi(hipStream_t stream, Out* out, std::int64_t len, Out neutral, Map map, Red red,
                      const InTs*... ins)
{
  if constexpr (sums_wide<Out, Red>()) {
    using Acc = typename wide_sum<Out>::type;
    map_reduce_multi_as<Acc>(stream, out, len, Acc((double)neutral), map, wide_add{},
                             narrow_then<Out, raft::identity_op>{raft::identity_op()}, ins...);
  } else {
    map_reduce_multi_as<Out>(stream, out, len, neutral, map, red, raft::identity_op(), ins...);
  }
}

}  // namespace raft::detail::rmi::generic
