// out = op(matrix, vec[, vec2]) with the vector(s) broadcast along the rows or along the
// columns of a contiguous matrix (linalg/detail/matrix_vector_op.cuh:17-90 in the
// reference, which forwards to matrix::linewise_op).  The functor is the caller's, so the
// kernel is instantiated in the caller's translation unit: include from files compiled by
// hipcc.
//
// The matrix is seen as [lines][C] with C the contiguous extent.  A thread owns V adjacent
// positions of a line for the whole kernel (V = elements per 16-byte access, at any
// element-aligned address; the last C % V elements of a line go to one more lane) and
// walks tiles of lines with four independent loads in flight; thread t is lane t % TX of line t / TX of a step, TX the
// line's lane count itself up to 128 (an equal cut of it beyond), so a step reads and
// writes one contiguous span.  A vector indexed along the contiguous extent is read once,
// into registers; one indexed by line is read once per line.  Matrix loads and stores are
// non-temporal (every element is touched once) where lines are whole cache lines.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

#include <raft/core/error.hpp>
#include <raft/linalg/detail/map.cuh>

namespace raft::linalg::detail {

constexpr int kMvBlock  = 256;
constexpr int kMvUnroll = 4;


// op(x, a) or op(x, a, b): one or two vectors
template <bool TWO, typename Op, typename MatT, typename Vec1T, typename Vec2T>
__device__ __forceinline__ MatT mv_apply(Op& op, const MatT& x, const Vec1T& a, const Vec2T& b)
{
  if constexpr (TWO) {
    return op(x, a, b);
  } else {
    return op(x, a);
  }
}

template <int V, bool ALONG_CONTIG, bool TWO, bool NT, typename MatT, typename Op, typename Vec1T,
          typename Vec2T>
__global__ __launch_bounds__(kMvBlock) void matrix_vector_kernel(
  MatT* out, const MatT* matrix, std::int64_t C, std::int64_t lines, Op op, int TX, int TY, int B,
  const Vec1T* vec1, const Vec2T* vec2)
{
  const int t             = threadIdx.x;
  const int ty            = (int)((unsigned)t / (unsigned)TX);
  const int tx            = t - ty * TX;
  const std::int64_t lane = (std::int64_t)blockIdx.x * TX + tx;
  const std::int64_t nw   = C / V;  // lanes that own a whole pack
  const int tail          = (int)(C - nw * V);
  const bool whole        = lane < nw;
  // The line's last C % V elements go to one more lane.  It READS the pack that ends at
  // the line's end (every lane issues the same loads: lanes that branch around their loads
  // are waited for one load at a time) and STORES only its last `tail` elements: the rest
  // of that pack is its neighbour's, which may already hold results when out == matrix.
  const bool part = V > 1 && lane == nw && tail > 0;
  if (ty >= TY || !(whole || part)) return;
  const std::int64_t c0 = whole ? lane * V : C - V;  // first contiguous position read
  const int first       = whole ? 0 : V - tail;      // first element of the pack owned
  // tiles of TY * kMvUnroll consecutive lines, dealt round-robin over blockIdx.y: at any
  // moment the grid reads and writes one compact, advancing window of the matrix
  const std::int64_t tile_lines = (std::int64_t)TY * kMvUnroll;
  const std::int64_t n_full     = lines / tile_lines;

  // a vector indexed along the contiguous extent: this thread's entries, read once
  Vec1T a[V];
  Vec2T b[V];
  if constexpr (ALONG_CONTIG) {
#pragma unroll
    for (int j = 0; j < V; ++j) {
      a[j] = vec1[c0 + j];
      if constexpr (TWO) b[j] = vec2[c0 + j];
    }
  }
  auto apply = [&](const map_pack<MatT, V>& x, std::int64_t line) {
    map_pack<MatT, V> y;
    if constexpr (ALONG_CONTIG) {
#pragma unroll
      for (int j = 0; j < V; ++j)
        y.v[j] = mv_apply<TWO>(op, x.v[j], a[j], b[j]);
    } else {
      const Vec1T la = vec1[line];
      Vec2T lb{};
      if constexpr (TWO) lb = vec2[line];
#pragma unroll
      for (int j = 0; j < V; ++j)
        y.v[j] = mv_apply<TWO>(op, x.v[j], la, lb);
    }
    return y;
  };
  auto store = [&](std::int64_t line, const map_pack<MatT, V>& y) {
    if (whole) {
      map_store<MatT, V, NT>(out, line * C + c0, y);
    } else {
#pragma unroll
      for (int j = 0; j < V; ++j)
        if (j >= first) out[line * C + c0 + j] = y.v[j];
    }
  };
  for (std::int64_t tile = blockIdx.y; tile < n_full; tile += B) {
    const std::int64_t r = tile * tile_lines + ty;
    map_pack<MatT, V> x[kMvUnroll];
#pragma unroll
    for (int u = 0; u < kMvUnroll; ++u)
      x[u] = map_load<MatT, V, NT>(matrix, (r + (std::int64_t)u * TY) * C + c0);
    map_pack<MatT, V> y[kMvUnroll];
#pragma unroll
    for (int u = 0; u < kMvUnroll; ++u)
      y[u] = apply(x[u], r + (std::int64_t)u * TY);
#pragma unroll
    for (int u = 0; u < kMvUnroll; ++u)
      store(r + (std::int64_t)u * TY, y[u]);
  }
  if ((std::int64_t)blockIdx.y == n_full % B) {  // the lines past the last whole tile
    for (std::int64_t r = n_full * tile_lines + ty; r < lines; r += TY)
      store(r, apply(map_load<MatT, V, NT>(matrix, r * C + c0), r));
  }
}

template <int V, bool ALONG_CONTIG, bool TWO, typename MatT, typename Op, typename Vec1T,
          typename Vec2T>
void launch_matrix_vector(MatT* out, const MatT* matrix, std::int64_t C, std::int64_t lines, Op op,
                          hipStream_t stream, const Vec1T* vec1, const Vec2T* vec2)
{
  const std::int64_t lanes = (C + V - 1) / V;
  // lines of whole multiples of 64 lanes keep pieces of exactly 64 lanes (1 KB at 1 KB
  // offsets within the line), others the fewest equal cuts of at most 128
  const std::int64_t cuts  = lanes % 64 == 0 ? lanes / 64 : (lanes + 127) / 128;
  const int TX             = (int)((lanes + cuts - 1) / cuts);
  const int TY             = kMvBlock / TX;
  const std::int64_t gridx = (lanes + TX - 1) / TX;
  // two workgroups per CU of a 256-CU device (measured best: 77 % of 8 TB/s in + out on
  // 1M x 128 floats, 72-75 % with 1024 or 4096), at least one tile each
  std::int64_t B           = (512 + gridx - 1) / gridx;
  const std::int64_t max_b = (lines + (std::int64_t)TY * kMvUnroll - 1) / ((std::int64_t)TY * kMvUnroll);
  if (B > max_b) B = max_b;
  if (B < 1) B = 1;
  if (B > 65535) B = 65535;
  RAFT_EXPECTS(gridx <= 0x7fffffffLL, "matrix_vector_op: row too long");
  // non-temporal accesses where no cache line is shared between two instructions: lines of
  // whole 128-byte cache lines at aligned addresses (10M x 13 floats: 53 % with plain
  // accesses, 21 % with non-temporal ones)
  const bool nt = (C * (std::int64_t)sizeof(MatT)) % 128 == 0 &&
                  reinterpret_cast<std::uintptr_t>(matrix) % 128 == 0 &&
                  reinterpret_cast<std::uintptr_t>(out) % 128 == 0;
  const dim3 grid((unsigned)gridx, (unsigned)B);
  if (nt)
    hipLaunchKernelGGL((matrix_vector_kernel<V, ALONG_CONTIG, TWO, true, MatT, Op, Vec1T, Vec2T>), grid,
                       dim3(kMvBlock), 0, stream, out, matrix, C, lines, op, TX, TY, (int)B, vec1, vec2);
  else
    hipLaunchKernelGGL((matrix_vector_kernel<V, ALONG_CONTIG, TWO, false, MatT, Op, Vec1T, Vec2T>), grid,
                       dim3(kMvBlock), 0, stream, out, matrix, C, lines, op, TX, TY, (int)B, vec1, vec2);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess)
    throw raft::hip_error(std::string("HIP error encountered at: matrix_vector_kernel: ") +
                          hipGetErrorString(e));
}

// D columns, N rows; bcastAlongRows: the vector has D entries (one per column), else N
template <bool rowMajor, bool bcastAlongRows, bool TWO, typename MatT, typename Lambda,
          typename IdxType, typename Vec1T, typename Vec2T>
void matrixVectorOpImpl(MatT* out, const MatT* matrix, IdxType D, IdxType N, Lambda op,
                        hipStream_t stream, const Vec1T* vec1, const Vec2T* vec2)
{
  if (D <= 0 || N <= 0) return;
  const std::int64_t C     = rowMajor ? (std::int64_t)D : (std::int64_t)N;  // contiguous extent
  const std::int64_t lines = rowMajor ? (std::int64_t)N : (std::int64_t)D;
  constexpr bool along_contig = rowMajor == bcastAlongRows;  // vector indexed within a line
  constexpr int V             = map_ratio_of<MatT>();
  if constexpr (V > 1) {
    if (C >= V) {
      launch_matrix_vector<V, along_contig, TWO>(out, matrix, C, lines, op, stream, vec1, vec2);
      return;
    }
  }
  launch_matrix_vector<1, along_contig, TWO>(out, matrix, C, lines, op, stream, vec1, vec2);
}

}  // namespace raft::linalg::detail
