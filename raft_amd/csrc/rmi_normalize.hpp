// Row normalisation fused with its norm: out[i, :] = in[i, :] / norm_i, where
// norm_i = final_op(reduce_op-fold of main_op(in[i, j])) and rows whose norm is
// <= eps are left untouched (linalg/detail/normalize.cuh:36-57,112-134 of the
// reference; a NaN norm is not <= eps, so such a row is written, as NaN).  Rows of up to 256 lane-loads stay in registers between the reduction
// and the scaling, so the matrix is read once and written once; longer rows are
// swept twice by one team (the second sweep finds the row in the caches).
#pragma once

#include "rmi_kernels.hpp"

namespace rmi {

struct NormArgs {
  const void* in;
  void* out;
  i64 n_rows;
  i64 len;
  i64 row_bytes;
  i64 nvec;    // whole lane-loads per row
  int tail;    // elements after the last whole vector
  int G;       // lanes per row (wave kernel)
  int logG;
  int tiles;   // wave kernel: rows per lane group and step (L * tiles lane-loads in flight)
  int L;       // wave kernel: lane-loads per lane and row (1 to 4); 0: one per lane with
               // G = the row's lane-load count itself (not a power of two)
  u32 invG;    // L == 0: 65536 / G + 1, so that (lane * invG) >> 16 == lane / G
  int final_op;
  double init;
  double eps;
  // flat kernel: a workgroup takes `chunk_rows` whole rows that start on a 16-byte boundary
  int chunk_rows;
  int logL;        // 2^logL lanes sum the partial norms of one row
  float inv_row_bytes;
};

// Element stores, the inverse of In<T>::get.
template <class T>
struct Put;
template <>
struct Put<float> {
  template <int J>
  static __device__ __forceinline__ void at(u32x4& v, float x)
  {
    v[J] = as_u32(x);
  }
  static __device__ __forceinline__ void st(float* p, float x) { *p = x; }
};
template <>
struct Put<double> {
  template <int J>
  static __device__ __forceinline__ void at(u32x4& v, double x)
  {
    v[2 * J]     = (u32)__double2loint(x);
    v[2 * J + 1] = (u32)__double2hiint(x);
  }
  static __device__ __forceinline__ void st(double* p, double x) { *p = x; }
};
template <>
struct Put<f16_t> {
  static __device__ __forceinline__ u32 bits(float x)
  {
    const f16_t h = (f16_t)x;
    uint16_t b;
    __builtin_memcpy(&b, &h, 2);
    return b;
  }
  template <int J>
  static __device__ __forceinline__ void at(u32x4& v, float x)
  {
    if constexpr (J & 1) {
      v[J / 2] = (v[J / 2] & 0xffffu) | (bits(x) << 16);
    } else {
      v[J / 2] = (v[J / 2] & 0xffff0000u) | bits(x);
    }
  }
  static __device__ __forceinline__ void st(f16_t* p, float x) { *p = (f16_t)x; }
};
template <>
struct Put<bf16_t> {
  template <int J>
  static __device__ __forceinline__ void at(u32x4& v, float x)
  {
    const u32 b = f32_to_bf16(x);
    if constexpr (J & 1) {
      v[J / 2] = (v[J / 2] & 0xffffu) | (b << 16);
    } else {
      v[J / 2] = (v[J / 2] & 0xffff0000u) | b;
    }
  }
  static __device__ __forceinline__ void st(bf16_t* p, float x) { p->bits = f32_to_bf16(x); }
};

// STREAM: the store is marked non-temporal (a compile-time choice: a run-time one is folded
// into one plain store by the compiler).  That pays where a store instruction writes
// whole cache lines that no other instruction touches (rows of whole 128-byte lines at an
// aligned address: 75 -> 78 % of 8 TB/s in + out; the 4 KB and longer pieces of the team
// kernels: 68 -> 71 %); rows whose pieces share lines lose up to 18 points with it.
template <bool STREAM>
__device__ __forceinline__ void store16(void* p, const u32x4& v)
{
  if constexpr (STREAM) {
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4_unaligned*>(p));
  } else {
    *reinterpret_cast<u32x4_unaligned*>(p) = v;
  }
}

// x / d for many x and one d, as the reference's element-wise division computes it, at three
// instructions per element instead of the ten or more of a division: with r = RN(1 / d), the
// quotient estimate q = RN(x * r) is corrected once with the exact residual, q' = RN(q + RN(x -
// q * d) * r), which is the correctly rounded x / d (Markstein) as long as r is normal and the
// residual x - q * d, some 2^-24 (2^-53) of x, is exactly representable.  A divisor outside
// [2^-100, 2^100] (fp32; 2^-900, 2^900 fp64), an infinite or a NaN one, and every element
// smaller than 2^-100 (2^-900) in magnitude, whose residual would fall below the subnormal
// spacing, take the division itself.
template <class T>
struct Quot {
  T d, r;
  bool fast;
  static constexpr T lo = sizeof(T) == 4 ? (T)7.888609052210118e-31 : (T)1.183e-271;   // 2^-100, ~2^-900
  static constexpr T hi = sizeof(T) == 4 ? (T)1.2676506002282294e30 : (T)8.452e270;    // 2^100, ~2^900
  __device__ __forceinline__ explicit Quot(T divisor) : d(divisor), r((T)1 / divisor)
  {
    fast = fabs(divisor) >= lo && fabs(divisor) <= hi;
  }
  // with the reciprocal RN(1 / divisor) computed elsewhere
  __device__ __forceinline__ Quot(T divisor, T recip) : d(divisor), r(recip)
  {
    fast = fabs(divisor) >= lo && fabs(divisor) <= hi;
  }
  __device__ __forceinline__ T operator()(T x) const
  {
    if (!fast || fabs(x) < lo) return x / d;
    const T q  = x * r;
    const T q2 = fma(fma(-q, d, x), r, q);
    // an infinite x has no residual (inf - inf): its product with r already is the quotient
    return q2 == q2 ? q2 : q;
  }
};

// norm of a row from its folded accumulator, in the element's own arithmetic
template <class P>
__device__ __forceinline__ typename P::nat row_norm(const NormArgs& a, typename P::acc_t acc)
{
  using nat               = typename P::nat;
  typename P::acc_t total = P::from_f64(a.init);
  P::merge(total, acc);
  nat n = (nat)P::to_f64(total);
  if (a.final_op == RMI_FIN_SQRT) n = sqrt(n);
  return n;
}

// lane-load `v` of a row, scaled by 1/norm and written to the same place of `orow`.
// TAIL_EACH: the overlapping last vector stores only its `tail` new elements, one by one.
// A kernel that re-reads the row for the scaling needs that when `out` is `in`: the vector's
// first VEC - tail elements belong to the lane before it, which may sit in another wave and
// may already have stored them scaled.
template <class P, bool VEC16, bool STREAM, bool TAIL_EACH = false>
__device__ __forceinline__ void write_scaled(const NormArgs& a,
                                             char* orow,
                                             const typename Held<P, VEC16>::type& x,
                                             i64 v,
                                             typename P::nat norm)
{
  using in_t = typename P::in_t;
  if constexpr (VEC16) {
    // The overlapping last vector (v == nvec) is stored whole where it was read: its first
    // VEC - tail elements repeat what the lane before it stores, bit for bit (as long as it
    // was loaded before any lane stored, i.e. the row is held in registers).
    if constexpr (TAIL_EACH) {
      if (v >= a.nvec) {
        in_t* o   = reinterpret_cast<in_t*>(orow) + (a.len - P::VEC);
        const int first = P::VEC - a.tail;
        if constexpr (sizeof(in_t) == 2) {
          const typename P::nat inv = (typename P::nat)1 / norm;
          static_for<P::VEC>([&](auto j) {
            if (decltype(j)::value >= first)
              Put<in_t>::st(o + decltype(j)::value, In<in_t>::template get<decltype(j)::value>(x) * inv);
          });
        } else {
          const Quot<typename P::nat> quot(norm);
          static_for<P::VEC>([&](auto j) {
            if (decltype(j)::value >= first)
              Put<in_t>::st(o + decltype(j)::value, quot(In<in_t>::template get<decltype(j)::value>(x)));
          });
        }
        return;
      }
    }
    u32x4 y = x;
    if constexpr (sizeof(in_t) == 2) {
      // 16-bit elements: one division per lane-load, then products in fp32 that are rounded
      // to 11 or 8 significant bits anyway (eight divisions per lane-load made these rows
      // ALU-bound); fp32 and fp64 rows divide element by element as the reference does
      const typename P::nat inv = (typename P::nat)1 / norm;
      static_for<P::VEC>([&](auto j) {
        Put<in_t>::template at<decltype(j)::value>(y, In<in_t>::template get<decltype(j)::value>(x) * inv);
      });
    } else {
      const Quot<typename P::nat> quot(norm);
      static_for<P::VEC>([&](auto j) {
        Put<in_t>::template at<decltype(j)::value>(y, quot(In<in_t>::template get<decltype(j)::value>(x)));
      });
    }
    store16<STREAM>(v < a.nvec ? orow + v * 16 : orow + (a.len - P::VEC) * (i64)sizeof(in_t), y);
  } else {
    Put<in_t>::st(reinterpret_cast<in_t*>(orow) + v, x / norm);
  }
}

// G lanes of one wave per row, L lane-loads per lane and row, kUnroll / L rows per
// lane group and step: kUnroll loads in flight per lane whatever the row length, and
// the rows stay in registers from the reduction to the scaling.
template <class P, bool VEC16, int L, int TILES, bool STREAM>
__device__ __forceinline__ void normalize_wave_body(const NormArgs& a)
{
  using acc_t         = typename P::acc_t;
  using H             = Held<P, VEC16>;
  const int lane      = threadIdx.x & (kWave - 1);
  const i64 wid       = (i64)blockIdx.x * (kBlock / kWave) + (threadIdx.x >> 6);
  const int G         = a.G;
  const int R         = kWave >> a.logG;
  const int c         = lane & (G - 1);
  const int g         = lane >> a.logG;
  const i64 nload     = a.nvec + (a.tail > 0 ? 1 : 0);

  typename H::type x[L * TILES];
  i64 row[TILES];
#pragma unroll
  for (int t = 0; t < TILES; ++t) {
    // Unconditional loads: a lane-load past the row's end re-reads the last one, a row
    // past the matrix the last row.  Loads under a lane mask are conditional
    // definitions, after which the compiler copies registers and waits for every load
    // in turn; the accumulation and the stores below stay masked.
    row[t]         = (wid * TILES + t) * R + g;
    const i64 rl   = row[t] < a.n_rows ? row[t] : a.n_rows - 1;
    const char* rp = static_cast<const char*>(a.in) + rl * a.row_bytes;
#pragma unroll
    for (int u = 0; u < L; ++u) {
      const i64 vl   = c + u * G < nload ? (i64)(c + u * G) : nload - 1;
      x[t * L + u]   = H::load_any(rp, vl, a.nvec, a.len);
    }
  }
  acc_t acc[TILES];
#pragma unroll
  for (int t = 0; t < TILES; ++t) {
    acc[t] = P::neutral();
    if (row[t] < a.n_rows) {
#pragma unroll
      for (int u = 0; u < L; ++u)
        if (c + u * G < nload) H::push_any(acc[t], x[t * L + u], c + u * G, a.nvec, a.len, a.tail);
    }
  }
#pragma unroll
  for (int t = 0; t < TILES; ++t)
    group_allreduce<P>(acc[t], G);
#pragma unroll
  for (int t = 0; t < TILES; ++t) {
    if (row[t] < a.n_rows) {
      const auto norm = row_norm<P>(a, acc[t]);
      if (!(norm <= (typename P::nat)a.eps)) {  // a NaN norm is not skipped: the row becomes NaN
        char* orow = static_cast<char*>(a.out) + row[t] * a.row_bytes;
#pragma unroll
        for (int u = 0; u < L; ++u)
          if (c + u * G < nload) write_scaled<P, VEC16, STREAM>(a, orow, x[t * L + u], c + u * G, norm);
      }
    }
  }
}

// Rows of G lane-loads, G not a power of two: one lane per lane-load, 64 / G whole rows per
// wave step and kUnroll steps in flight, so every load and store instruction covers one
// contiguous span of the matrix; the wave's last 64 % G lanes idle.  The row's lanes are
// folded into its first one (lane c takes lane c + s for s = 1, 2, 4 ...), which hands the
// norm back to all of them.
template <class P, bool STREAM>
__device__ __forceinline__ void normalize_anyg_body(const NormArgs& a)
{
  using acc_t     = typename P::acc_t;
  using H         = Held<P, true>;
  const int lane  = threadIdx.x & (kWave - 1);
  const i64 wid   = (i64)blockIdx.x * (kBlock / kWave) + (threadIdx.x >> 6);
  const int G     = a.G;
  const int R     = kWave / G;
  const int g     = (int)(((u32)lane * a.invG) >> 16);
  const int c     = lane - g * G;
  const bool live = g < R;

  typename H::type x[kUnroll];
  i64 row[kUnroll];
  const i64 cl = live ? (i64)c : (i64)G - 1;
#pragma unroll
  for (int t = 0; t < kUnroll; ++t) {  // unconditional, clamped: see normalize_wave_body
    row[t]       = (wid * kUnroll + t) * R + g;
    const i64 rl = row[t] < a.n_rows ? row[t] : a.n_rows - 1;
    x[t] = H::load_any(static_cast<const char*>(a.in) + rl * a.row_bytes, cl, a.nvec, a.len);
  }
  acc_t acc[kUnroll];
#pragma unroll
  for (int t = 0; t < kUnroll; ++t) {
    acc[t] = P::neutral();
    if (live && row[t] < a.n_rows) H::push_any(acc[t], x[t], c, a.nvec, a.len, a.tail);
  }
  for (int s = 1; s < G; s <<= 1) {
#pragma unroll
    for (int t = 0; t < kUnroll; ++t) {
      const acc_t v = shfl_acc<P>(acc[t], lane + s);
      if (c + s < G) P::merge(acc[t], v);
    }
  }
  const int first = live ? g * G : lane;
#pragma unroll
  for (int t = 0; t < kUnroll; ++t) {
    const acc_t total = shfl_acc<P>(acc[t], first);
    if (live && row[t] < a.n_rows) {
      const auto norm = row_norm<P>(a, total);
      if (!(norm <= (typename P::nat)a.eps))  // a NaN norm is not skipped: the row becomes NaN
        write_scaled<P, true, STREAM>(a, static_cast<char*>(a.out) + row[t] * a.row_bytes, x[t], c, norm);
    }
  }
}

template <class P, bool VEC16, bool STREAM = false>
__global__ __launch_bounds__(kBlock) void normalize_wave_kernel(NormArgs a)
{
  if constexpr (VEC16) {
    if (a.L == 0) {
      normalize_anyg_body<P, STREAM>(a);
      return;
    }
  }
  if (a.L == 1) {
    normalize_wave_body<P, VEC16, 1, 4, STREAM>(a);
  } else if (a.L == 2) {
    if (a.tiles == 1) normalize_wave_body<P, VEC16, 2, 1, STREAM>(a);
    else normalize_wave_body<P, VEC16, 2, 2, STREAM>(a);
  } else if (a.L == 3) {
    normalize_wave_body<P, VEC16, 3, 1, STREAM>(a);
  } else if (a.L == 4) {
    normalize_wave_body<P, VEC16, 4, 1, STREAM>(a);
  } else if constexpr (VEC16) {
    // rows of 257 to 512 lane-loads on one wave: a 256-thread team would hold one or two
    // lane-loads per thread and a quarter of its load slots
    if (a.L == 5) normalize_wave_body<P, true, 5, 1, STREAM>(a);
    else if (a.L == 6) normalize_wave_body<P, true, 6, 1, STREAM>(a);
    else if (a.L == 7) normalize_wave_body<P, true, 7, 1, STREAM>(a);
    else normalize_wave_body<P, true, 8, 1, STREAM>(a);
  }
}

// One team of blockDim.x threads per row; the row (at most UH lane-loads per thread)
// stays in registers from the reduction to the scaling.
template <class P, int UH>
__global__ __launch_bounds__(1024) void normalize_team_kernel(NormArgs a)
{
  using acc_t = typename P::acc_t;
  using H     = Held<P, true>;
  using nat   = typename P::nat;
  __shared__ acc_t sm[16];
  __shared__ nat sm_norm;

  const int T     = blockDim.x;
  const int t     = threadIdx.x;
  const i64 row   = blockIdx.x;
  const i64 nload = a.nvec + (a.tail > 0 ? 1 : 0);
  const char* rp  = static_cast<const char*>(a.in) + row * a.row_bytes;

  typename H::type x[UH];
#pragma unroll
  for (int u = 0; u < UH; ++u) {  // unconditional, clamped: see normalize_wave_body
    const i64 vl = t + (i64)u * T < nload ? t + (i64)u * T : nload - 1;
    x[u]         = H::load_any(rp, vl, a.nvec, a.len);
  }
  acc_t acc = P::neutral();
#pragma unroll
  for (int u = 0; u < UH; ++u)
    if (t + (i64)u * T < nload) H::push_any(acc, x[u], t + (i64)u * T, a.nvec, a.len, a.tail);
  wave_allreduce<P>(acc);
  if ((t & (kWave - 1)) == 0) sm[t >> 6] = acc;
  __syncthreads();
  if (t == 0) {
    for (int w = 1; w < (T >> 6); ++w)
      P::merge(acc, sm[w]);
    sm_norm = row_norm<P>(a, acc);
  }
  __syncthreads();
  const nat norm = sm_norm;
  if (norm <= (nat)a.eps) return;  // a NaN norm is not skipped: the row becomes NaN
  char* orow = static_cast<char*>(a.out) + row * a.row_bytes;
#pragma unroll
  for (int u = 0; u < UH; ++u)
    if (t + (i64)u * T < nload) write_scaled<P, true, true>(a, orow, x[u], t + (i64)u * T, norm);
}

// Rows too long for a team's registers: one team of 1024 threads sweeps the row
// twice (the second sweep finds most of it in the caches).
template <class P>
__global__ __launch_bounds__(1024) void normalize_sweep_kernel(NormArgs a)
{
  using acc_t = typename P::acc_t;
  using H     = Held<P, true>;
  using nat   = typename P::nat;
  __shared__ acc_t sm[16];
  __shared__ nat sm_norm;

  const int T     = blockDim.x;
  const int t     = threadIdx.x;
  const i64 row   = blockIdx.x;
  const i64 nload = a.nvec + (a.tail > 0 ? 1 : 0);
  const char* rp  = static_cast<const char*>(a.in) + row * a.row_bytes;

  acc_t acc = P::neutral();
  for (i64 v = t; v < nload; v += (i64)kUnroll * T) {
    typename H::type x[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {  // unconditional, clamped: see normalize_wave_body
      const i64 vl = v + (i64)u * T < nload ? v + (i64)u * T : nload - 1;
      x[u]         = H::load_any(rp, vl, a.nvec, a.len);
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
      if (v + (i64)u * T < nload) H::push_any(acc, x[u], v + (i64)u * T, a.nvec, a.len, a.tail);
  }
  wave_allreduce<P>(acc);
  if ((t & (kWave - 1)) == 0) sm[t >> 6] = acc;
  __syncthreads();
  if (t == 0) {
    for (int w = 1; w < (T >> 6); ++w)
      P::merge(acc, sm[w]);
    sm_norm = row_norm<P>(a, acc);
  }
  __syncthreads();
  const nat norm = sm_norm;
  if (norm <= (nat)a.eps) return;  // a NaN norm is not skipped: the row becomes NaN
  char* orow = static_cast<char*>(a.out) + row * a.row_bytes;
  for (i64 v = t; v < nload; v += (i64)kUnroll * T) {
    typename H::type x[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {  // unconditional, clamped: see normalize_wave_body
      const i64 vl = v + (i64)u * T < nload ? v + (i64)u * T : nload - 1;
      x[u]         = H::load_any(rp, vl, a.nvec, a.len);
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
      if (v + (i64)u * T < nload) write_scaled<P, true, true, true>(a, orow, x[u], v + (i64)u * T, norm);
  }
}

// ---------------------------------------------------------------------------
// Flat kernel, for rows whose lane-loads would straddle 16-byte boundaries (row bytes no
// multiple of 16) when input and output start on one: the matrix is read and written as a
// flat run of ALIGNED 16-byte vectors, whatever the row length.  A workgroup takes a chunk of
// whole rows that starts on a 16-byte boundary (a multiple of 16 / gcd(16, row bytes) rows,
// at most 16 KB), each thread kFlatVecs vectors of it, all loaded before anything else
// happens.  A vector holds elements of at most two rows (rows are 16 bytes or longer): every
// thread reduces the two parts of each of its vectors and leaves them in LDS; 2^logL lanes
// per row then fold the row's parts in vector order (fixed order: repeatable bits) and leave
// the norm in LDS; every thread scales the elements of its vectors by their rows' norms and
// stores the vectors whole.  Rows whose norm is <= eps must not be written: a vector that
// touches such a row stores its other elements one by one.  In place is safe: a chunk is
// in registers before any of it is written, and chunks do not overlap.
// 16-bit elements take their products and the sums inside a vector in fp32 (products of
// 8- and 11-bit significands are exact there; the sum of a vector's eight is rounded, 2^-22
// of it at most, far below the 2^-9 / 2^-12 the outputs are rounded to), everything else in
// the accumulator type as in the other kernels.
// ---------------------------------------------------------------------------
template <int MAIN>
__device__ __forceinline__ float main_f32(float x)
{
  if constexpr (MAIN == RMI_MAIN_SQ) return x * x;
  if constexpr (MAIN == RMI_MAIN_ABS) return fabsf(x);
  return x;
}
template <int RED>
__device__ __forceinline__ float red_f32(float a, float b)
{
  if constexpr (RED == RMI_RED_MAX) return fmaxf(a, b);
  if constexpr (RED == RMI_RED_MIN) return fminf(a, b);
  return a + b;
}
template <int RED>
__device__ __forceinline__ float neutral_f32()
{
  if constexpr (RED == RMI_RED_MAX) return -__builtin_inff();
  if constexpr (RED == RMI_RED_MIN) return __builtin_inff();
  return 0.0f;
}

template <class P>
__global__ __launch_bounds__(kBlock) void normalize_flat_kernel(NormArgs a)
{
  using in_t  = typename P::in_t;
  using acc_t = typename P::acc_t;
  using nat   = typename P::nat;
  constexpr bool k16 = sizeof(in_t) == 2;
  using part_t       = std::conditional_t<k16, float, acc_t>;
  constexpr int VEC  = P::VEC;
  constexpr int ES   = (int)sizeof(in_t);
  __shared__ part_t part0[kFlatChunkVec];  // a vector's elements of the row it starts in
  __shared__ part_t part1[kFlatChunkVec];  // ... and of the next row
  __shared__ nat norms[kFlatChunkVec];     // a chunk has no more rows than vectors
  // 1 / norm, computed once per row; not for fp64 rows, whose accumulators already take 32 KB
  // of LDS: 8 KB more cost a resident workgroup and 4-6 % there
  constexpr bool kRecips = sizeof(nat) < 8;
  __shared__ nat recips[kRecips ? kFlatChunkVec : 1];

  const int t         = threadIdx.x;
  const int rb        = (int)a.row_bytes;
  const i64 row0      = (i64)blockIdx.x * a.chunk_rows;
  const i64 left      = a.n_rows - row0;
  const int rows      = left < a.chunk_rows ? (int)left : a.chunk_rows;
  const int nvec      = (rows * rb) >> 4;  // whole vectors: the caller passes rows that end on a boundary
  const char* base    = static_cast<const char*>(a.in) + row0 * rb;
  char* obase         = static_cast<char*>(a.out) + row0 * rb;
  const int shift     = (int)((reinterpret_cast<uintptr_t>(obase) >> 4) & 7);

  u32x4 x[kFlatVecs];
#pragma unroll
  for (int k = 0; k < kFlatVecs; ++k) {  // unconditional, clamped
    const int v = t + k * kBlock - shift;
    x[k]        = load16(base + 16 * (i64)(v < 0 ? 0 : (v < nvec ? v : nvec - 1)));
  }
  int r0v[kFlatVecs], split[kFlatVecs];
#pragma unroll
  for (int k = 0; k < kFlatVecs; ++k) {
    const int v = t + k * kBlock - shift;
    const int b = 16 * (v < 0 ? 0 : v);
    // row that byte b belongs to: b < 16384, so the float quotient is off by one at most
    int r0 = (int)((float)b * a.inv_row_bytes);
    if ((r0 + 1) * rb <= b) ++r0;
    if (r0 * rb > b) --r0;
    const int own = (r0 + 1) * rb - b;  // bytes from b on that belong to row r0
    r0v[k]        = r0;
    split[k]      = own < 16 ? own / ES : VEC;
    if constexpr (k16) {
      float s0 = neutral_f32<P::kRed>(), s1 = neutral_f32<P::kRed>();
      static_for<VEC>([&](auto j) {
        const float m = main_f32<P::kMain>(In<in_t>::template get<decltype(j)::value>(x[k]));
        const bool lo = decltype(j)::value < split[k];
        s0            = red_f32<P::kRed>(s0, lo ? m : neutral_f32<P::kRed>());
        s1            = red_f32<P::kRed>(s1, lo ? neutral_f32<P::kRed>() : m);
      });
      if (v >= 0 && v < nvec) part0[v] = s0, part1[v] = s1;
    } else {
      acc_t s0 = P::neutral(), s1 = P::neutral();
      static_for<VEC>([&](auto j) {
        const nat e = In<in_t>::template get<decltype(j)::value>(x[k]);
        if (decltype(j)::value < split[k]) P::push(s0, e, 0);
        else P::push(s1, e, 0);
      });
      if (v >= 0 && v < nvec) part0[v] = s0, part1[v] = s1;
    }
  }
  __syncthreads();
  {
    const int L    = 1 << a.logL;
    const int c    = t & (L - 1);
    const int step = kBlock >> a.logL;
    const int npass = (rows + step - 1) / step;  // uniform: every lane of a group takes part in its exchanges
    for (int pass = 0; pass < npass; ++pass) {
      const int r  = pass * step + (t >> a.logL);
      const int rr = r < rows ? r : rows - 1;
      const int bs = rr * rb;
      const int vf = bs >> 4, vl = (bs + rb - 1) >> 4;
      acc_t acc    = P::neutral();
      for (int v = vf + c; v <= vl; v += L) {
        acc_t p;
        if constexpr (k16) p = P::from_f64((double)((v == vf && (bs & 15)) ? part1[v] : part0[v]));
        else p = (v == vf && (bs & 15)) ? part1[v] : part0[v];
        P::merge(acc, p);
      }
      group_allreduce<P>(acc, L);
      if (c == 0 && r < rows) {
        const nat n = row_norm<P>(a, acc);
        norms[r]    = n;
        if constexpr (kRecips) recips[r] = (nat)1 / n;
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < kFlatVecs; ++k) {
    const int v = t + k * kBlock - shift;
    if (v < 0 || v >= nvec) continue;
    const int r0  = r0v[k];
    const int r1  = r0 + 1 < rows ? r0 + 1 : r0;
    const nat n0  = norms[r0];
    const nat n1  = norms[r1];
    const nat i0  = kRecips ? recips[r0] : (nat)1 / n0;
    const nat i1  = kRecips ? recips[r1] : (nat)1 / n1;
    const bool k0 = n0 <= (nat)a.eps;                       // rows that are left untouched
    const bool k1 = split[k] < VEC && n1 <= (nat)a.eps;     // (a NaN norm is not: the row becomes NaN)
    u32x4 y       = x[k];
    if constexpr (k16) {
      // two products rounded to 16 bits (nearest even) and packed by one conversion
      typedef float f32x2 __attribute__((ext_vector_type(2)));
      using half_t = std::conditional_t<std::is_same_v<in_t, bf16_t>, __bf16, _Float16>;
      typedef half_t h16x2 __attribute__((ext_vector_type(2)));
      static_for<VEC / 2>([&](auto w) {
        constexpr int W = decltype(w)::value;
        f32x2 p;
        p[0] = In<in_t>::template get<2 * W>(x[k]) * (2 * W < split[k] ? i0 : i1);
        p[1] = In<in_t>::template get<2 * W + 1>(x[k]) * (2 * W + 1 < split[k] ? i0 : i1);
        y[W] = __builtin_bit_cast(u32, __builtin_convertvector(p, h16x2));
      });
    } else {
      const Quot<nat> q0(n0, i0), q1(n1, i1);
      static_for<VEC>([&](auto j) {
        constexpr int J = decltype(j)::value;
        Quot<nat> q     = q0;
        if (J >= split[k]) q = q1;
        Put<in_t>::template at<J>(y, q(In<in_t>::template get<J>(x[k])));
      });
    }
    if (!(k0 || k1)) {
      store16<true>(obase + 16 * (i64)v, y);
    } else {
      in_t* o = reinterpret_cast<in_t*>(obase + 16 * (i64)v);
      static_for<VEC>([&](auto j) {
        constexpr int J = decltype(j)::value;
        if (!(J < split[k] ? k0 : k1)) {
          if constexpr (ES == 2) {
            reinterpret_cast<uint16_t*>(o)[J] = (uint16_t)(y[J / 2] >> (16 * (J & 1)));
          } else if constexpr (ES == 4) {
            reinterpret_cast<u32*>(o)[J] = y[J];
          } else {
            reinterpret_cast<u32*>(o)[2 * J]     = y[2 * J];
            reinterpret_cast<u32*>(o)[2 * J + 1] = y[2 * J + 1];
          }
        }
      });
    }
  }
}

// ---------------------------------------------------------------------------
// Rows shorter than a 16-byte vector (three floats, five halves): a lane per ELEMENT read and
// wrote them at 20-45 % of the memory rate.  Here a workgroup reads a chunk of whole rows (a
// multiple of 16 rows, at most 16 KB, from a 16-byte boundary of input and output) as aligned
// vectors into LDS, every thread norms whole rows out of LDS, element by element, and the
// chunk leaves as whole vectors, scaled with the arithmetic of the other kernels.
//   PER_VECTOR = false: the thread that normed a row scales it in place in LDS.
//   PER_VECTOR = true: the threads leave the reciprocals of their rows' norms in LDS and the
//     chunk is scaled vector by vector on its way out, an element's row being its index over
//     the row length (at most kSmallNormRows rows per chunk).  For 16-bit rows of an odd
//     length, whose rows share 32-bit words of LDS: written by different lanes, they cost the
//     first variant half of its rate.
// A row whose norm is <= eps must not be written: a chunk that holds one is stored row by
// row, element by element, by the threads that own its rows.
// ---------------------------------------------------------------------------
constexpr int kSmallNormRows = 2048;
template <class P, bool PER_VECTOR>
__global__ __launch_bounds__(kBlock) void normalize_small_kernel(NormArgs a)
{
  using in_t  = typename P::in_t;
  using nat   = typename P::nat;
  using acc_t = typename P::acc_t;
  constexpr int ES  = (int)sizeof(in_t);
  constexpr int VEC = P::VEC;
  __shared__ __align__(16) unsigned char sm[kSmallBytes];
  __shared__ nat recips[PER_VECTOR ? kSmallNormRows : 1];
  __shared__ int any_skipped;
  const int t     = threadIdx.x;
  const int rb    = (int)a.row_bytes;
  const i64 row0  = (i64)blockIdx.x * a.chunk_rows;
  const i64 left  = a.n_rows - row0;
  const int rows  = left < a.chunk_rows ? (int)left : a.chunk_rows;
  const int bytes = rows * rb;   // kSmallBytes at most
  const int nfull = bytes >> 4;  // whole vectors of the chunk
  const char* base = static_cast<const char*>(a.in) + row0 * rb;
  char* obase      = static_cast<char*>(a.out) + row0 * rb;
  if (t == 0) any_skipped = 0;
  if (nfull > 0) {
    u32x4 x[kSmallVecs];
#pragma unroll
    for (int k = 0; k < kSmallVecs; ++k) {  // unconditional, clamped
      const int v = t + k * kBlock;
      x[k]        = load16(base + 16 * (v < nfull ? v : nfull - 1));
    }
#pragma unroll
    for (int k = 0; k < kSmallVecs; ++k) {
      const int v = t + k * kBlock;
      if (v < nfull) *reinterpret_cast<u32x4*>(sm + 16 * v) = x[k];
    }
  }
  // what follows the last whole vector (the matrix's last chunk only), element by element
  for (int i = (nfull << 4) / ES + t; i < bytes / ES; i += kBlock)
    reinterpret_cast<in_t*>(sm)[i] = reinterpret_cast<const in_t*>(base)[i];
  __syncthreads();
  in_t* e     = reinterpret_cast<in_t*>(sm);
  const int D = (int)a.len;
  // x / norm as the other kernels compute it: 16-bit elements times the reciprocal in fp32,
  // fp32 and fp64 correctly rounded
  auto scaled = [&](nat x, nat norm, nat recip) __attribute__((always_inline)) {
    if constexpr (ES == 2) {
      return x * recip;
    } else {
      return Quot<nat>(norm, recip)(x);
    }
  };
  u32 skipped = 0;  // bit k: this thread's k-th row is left untouched (32 rows per thread at most)
  int k       = 0;
  for (int r = t; r < rows; r += kBlock, ++k) {
    acc_t acc = P::neutral();
    for (int j = 0; j < D; ++j)
      P::push(acc, stored_to_nat<in_t>(e[r * D + j]), (i64)j);
    const nat norm  = row_norm<P>(a, acc);
    const nat recip = (nat)1 / norm;
    if (norm <= (nat)a.eps) {  // a NaN norm is not skipped: the row becomes NaN
      skipped |= 1u << k;
      any_skipped = 1;
    }
    if constexpr (PER_VECTOR) {
      recips[r] = recip;
    } else if (!(norm <= (nat)a.eps)) {
      for (int j = 0; j < D; ++j)
        Put<in_t>::st(e + r * D + j, scaled(stored_to_nat<in_t>(e[r * D + j]), norm, recip));
    }
  }
  __syncthreads();
  if (any_skipped == 0) {
    const float inv_len = 1.0f / (float)D;
#pragma unroll
    for (int q = 0; q < kSmallVecs; ++q) {
      const int v = t + q * kBlock;
      if (v < nfull) {
        u32x4 y = *reinterpret_cast<const u32x4*>(sm + 16 * v);
        if constexpr (PER_VECTOR) {
          static_assert(!PER_VECTOR || ES == 2, "scaled by the reciprocal alone");
          const u32x4 x = y;
          static_for<VEC>([&](auto j) {
            constexpr int J = decltype(j)::value;
            // the element's row: its index is below 8192 and D below 16, so the quotient is exact
            const int r = (int)(((float)(v * VEC + J) + 0.5f) * inv_len);
            Put<in_t>::template at<J>(y, In<in_t>::template get<J>(x) * recips[r]);
          });
        }
        store16<false>(obase + 16 * v, y);
      }
    }
    for (int i = (nfull << 4) / ES + t; i < bytes / ES; i += kBlock) {
      if constexpr (PER_VECTOR) {
        Put<in_t>::st(reinterpret_cast<in_t*>(obase) + i,
                      stored_to_nat<in_t>(e[i]) * recips[(int)(((float)i + 0.5f) * inv_len)]);
      } else {
        reinterpret_cast<in_t*>(obase)[i] = e[i];
      }
    }
  } else {
    k = 0;
    for (int r = t; r < rows; r += kBlock, ++k) {
      if ((skipped >> k) & 1u) continue;
      for (int j = 0; j < D; ++j) {
        if constexpr (PER_VECTOR) {
          Put<in_t>::st(reinterpret_cast<in_t*>(obase) + r * D + j, stored_to_nat<in_t>(e[r * D + j]) * recips[r]);
        } else {
          reinterpret_cast<in_t*>(obase)[r * D + j] = e[r * D + j];
        }
      }
    }
  }
}

}  // namespace rmi
