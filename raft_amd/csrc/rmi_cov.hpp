// Covariance of the columns of a dense matrix around a given mean vector:
//   covar = (X - 1 mu^T)^T (X - 1 mu^T) * alpha,   X: [N][D], covar: [D][D].
// The one contraction on this path, so the one place that uses the matrix cores.
//
// The columns are cut into blocks of 64; a workgroup owns one pair of blocks (bi <= bj: the
// upper triangle, the fold mirrors it) and one of S interleaved sets of rows (a slab), and
// accumulates that pair's 64 x 64 piece of X^T X as sixteen 16 x 16 tiles (ten on the
// diagonal): fp64 data with v_mfma_f64_16x16x4_f64, fp32 data, split into three bf16 terms
// per value, with v_mfma_f32_16x16x32_bf16 (see gram_rows_body_bf16).  The operands go from
// global memory straight into the registers the instruction reads them from; for the
// 16 x 16 x 4 instruction:
//
//   row-major X   lane l loads four consecutive columns 4 * (l % 16) .. + 3 of row l / 16 of
//                 a wave-load of four rows; register j then holds, for the lanes 16 k .. 16 k
//                 + 15, the columns {4 m + j} of row k, which is the A (and B) operand of a
//                 16 x 16 x 4 step.  The result tile (ja, jb) is therefore the columns
//                 {4 m + ja} x {4 n + jb}: a permutation the fold undoes.
//   col-major X   lane l loads four consecutive rows of column 16 a + l % 16, the four lane
//                 quarters reading four consecutive runs of rows; register j of column group
//                 a and register j of group b are one 16 x 16 x 4 step of tile (a, b).
//
// x - mu happens in registers; with `center` set (one pair only, i.e. D <= 64) the centred
// values are also written back, which is what the reference leaves in `data`.  Every wave
// keeps its tiles for its whole share of the rows, the four waves of a workgroup meet in
// LDS, and the workgroup stores its tiles as a partial [slab][pair][tile][256] that
// cov_fold_kernel sums over the slabs in f64, in slab order, scales and writes to both
// halves of the symmetric result.  Nothing is accumulated with atomics: results are
// bitwise repeatable.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "rmi_reduce.h"

namespace rmi {
namespace cov {

constexpr int kBlockCols    = 64;   // columns of a column block
constexpr int kThreads      = 256;  // a workgroup: four waves
constexpr int kWaves        = 4;
constexpr int kTile         = 256;  // elements of a 16 x 16 result tile
constexpr int kTilesPerPair = 16;   // 4 x 4 tiles of a 64 x 64 piece
#ifndef RMI_COV_ROW_UNIT_LOADS
#define RMI_COV_ROW_UNIT_LOADS 4
#endif
#ifndef RMI_COV_ROW_RING
#define RMI_COV_ROW_RING 3
#endif
constexpr int kRowUnitLoads = RMI_COV_ROW_UNIT_LOADS;  // row-major: wave-loads of a unit
constexpr int kRowRing      = RMI_COV_ROW_RING;        // ... and units in the ring
constexpr int kRowUnitRows  = 4 * kRowUnitLoads;      // rows of a unit
constexpr int kColUnitRows  = 16;   // col-major: rows of a unit (four per lane quarter)
constexpr int kFoldSplit    = 16;   // fold: threads that share the slabs of one element

// units a wave keeps in flight, given the 32-bit registers one unit takes: about 64
// registers' worth, at least two and at most eight
constexpr int ring_depth(int unit_regs)
{
  const int p = 64 / unit_regs;
  return p < 2 ? 2 : (p > 8 ? 8 : p);
}

template <class T>
struct Mma;
template <>
struct Mma<float> {
  using acc_t = float __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ acc_t mma(float a, float b, acc_t c)
  {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
  }
  // row of the 16 x 16 result that register i of lane l holds (its column is l % 16)
  static __device__ __forceinline__ int row(int lane, int i) { return 4 * (lane >> 4) + i; }
};
template <>
struct Mma<double> {
  using acc_t = double __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ acc_t mma(double a, double b, acc_t c)
  {
    return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ int row(int lane, int i) { return (lane >> 4) + 4 * i; }
};

struct GramArgs {
  void* data;        // [N][D] row-major or [D][N] col-major; written only with `center`
  const void* mu;    // D means, or nullptr: the data is centred already
  void* partial;     // [S][npairs][16][256] accumulators of T
  int64_t N;
  int64_t D;
  int nb;            // column blocks
  int npairs;        // nb * (nb + 1) / 2
  int S;             // slabs
  int total;         // S * npairs workgroups do work; the grid is rounded up to 8
  // A matrix of at most 32 columns is contracted as one of f D <= 64: f consecutive rows (row-
  // major) or the first f pieces of N rows of every column (col-major) side by side.  Column c
  // of the wide matrix then has the mean mu[(c / mu_div) % mu_mod]; mu_mod == 0: mu[c].
  int mu_div;
  int mu_mod;
  // col-major: column c of the (wide) matrix starts at (c / col_f) * col_ld + (c % col_f) * N
  // (col_f pieces of the columns of a matrix whose columns are col_ld apart; 1: c * col_ld)
  int64_t col_ld;
  int col_f;
};
__device__ __forceinline__ int64_t mean_index(const GramArgs& a, int64_t c)
{
  return a.mu_mod == 0 ? c : (c / a.mu_div) % a.mu_mod;
}
__device__ __forceinline__ int64_t col_offset(const GramArgs& a, int64_t c)
{
  return a.col_f <= 1 ? c * a.col_ld : (c / a.col_f) * a.col_ld + (c % a.col_f) * a.N;
}

struct FoldArgs {
  const void* partial;
  void* out;         // [D][D]
  int64_t D;
  int nb;
  int npairs;
  int S;
  int permuted;      // tiles hold the columns {4 m + ja} x {4 n + jb} (row-major kernel)
  double alpha;      // 1 / (N - 1) or 1 / N, rounded to T as the reference's scalar is
  double* wide;      // not null: the scaled sums go here as [D][D] doubles instead of `out`
                     // (the 64-column contraction of a narrower matrix, see cov_blocks_kernel)
};

// Four elements at any element-aligned address (gfx950 serves unaligned vector loads).
template <class T>
struct Quad {
  T v[4];
};
// STREAM: the data is read once, keep it out of the caches (non-temporal).  A template
// parameter: chosen by a run-time flag, the two forms are merged into one plain load.
template <class T, bool STREAM>
__device__ __forceinline__ Quad<T> load_quad(const T* p)
{
  typedef T full_t __attribute__((ext_vector_type(4)));
  typedef full_t vec_t __attribute__((aligned(sizeof(T))));
  vec_t x;
  if constexpr (STREAM)
    x = __builtin_nontemporal_load(reinterpret_cast<const vec_t*>(p));
  else
    x = *reinterpret_cast<const vec_t*>(p);
  Quad<T> q;
#pragma unroll
  for (int j = 0; j < 4; ++j)
    q.v[j] = x[j];
  return q;
}
// STREAM: the centred rows are not read again by this kernel; measured 3 % faster streamed
// where a store instruction writes whole lines (row-major), 6 % slower where it writes 16-byte
// pieces of 64 lines (col-major).
template <class T, bool STREAM = false>
__device__ __forceinline__ void store_quad(T* p, const Quad<T>& q)
{
  typedef T full_t __attribute__((ext_vector_type(4)));
  typedef full_t vec_t __attribute__((aligned(sizeof(T))));
  vec_t x;
#pragma unroll
  for (int j = 0; j < 4; ++j)
    x[j] = q.v[j];
  if constexpr (STREAM)
    __builtin_nontemporal_store(x, reinterpret_cast<vec_t*>(p));
  else
    *reinterpret_cast<vec_t*>(p) = x;
}

// Workgroup ids are dealt round-robin over the 8 XCDs, each with an L2 of its own.  The
// pairs of one slab read the same rows, so they are given ids that land on one XCD: id
// 8 q + x becomes unit x * (grid / 8) + q, and units are numbered slab-major.
__device__ __forceinline__ int xcd_local_unit()
{
  const int per_xcd = gridDim.x >> 3;
  return (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
}

__device__ __forceinline__ void pair_blocks(int p, int nb, int& bi, int& bj)
{
  bi = 0;
  while (p >= nb - bi) {
    p -= nb - bi;
    ++bi;
  }
  bj = bi + p;
}

// The four waves' tiles meet in LDS, one wave at a time; wave 0 ends up with the sums.
template <class T, int NT>
__device__ __forceinline__ void combine_waves(typename Mma<T>::acc_t (&acc)[NT], T* sm, int wave,
                                              int lane)
{
  for (int w = 1; w < kWaves; ++w) {
    __syncthreads();
    if (wave == w) {
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          sm[t * kTile + i * 64 + lane] = acc[t][i];
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          acc[t][i] += sm[t * kTile + i * 64 + lane];
    }
  }
}

template <class T>
__device__ __forceinline__ void store_tile(T* partial, const typename Mma<T>::acc_t& acc, int lane)
{
#pragma unroll
  for (int i = 0; i < 4; ++i)
    partial[i * 64 + lane] = acc[i];
}

// ---------------------------------------------------------------------------
// Row-major X.  VEC: rows are whole quads of columns (D % 4 == 0), one vector load per
// lane and block; otherwise four element loads with the column clamped.
// ---------------------------------------------------------------------------
template <class T, bool VEC, bool DIAG, bool CENTER, bool STREAM>
__device__ __forceinline__ void gram_rows_body(const GramArgs& a, int unit, int slab, int bi, int bj,
                                               T* sm)
{
  using M     = Mma<T>;
  using acc_t = typename M::acc_t;
  constexpr int NS = DIAG ? 1 : 2;  // blocks read: one on the diagonal
  constexpr int UL = kRowUnitLoads;
  constexpr int UR = 4 * UL;        // rows of a unit
  constexpr int P  = kRowRing;

  const int lane = threadIdx.x & 63;
  // (read from the first lane so that the compiler knows it, and every row and unit index
  // derived from it, to be the same for the whole wave: scalar registers and scalar
  // arithmetic instead of 64-bit vector multiplies per lane-load)
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lr   = lane >> 4;  // row of the wave-load
  const int cg   = lane & 15;  // quad of columns within the block
  T* const data  = static_cast<T*>(a.data);
  const T* mu    = static_cast<const T*>(a.mu);
  const int64_t D = a.D;

  // columns of this lane in the block(s), whether they exist, and their means
  int64_t col[NS][4];
  bool ok[NS][4];
  T mean[NS][4];
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    const int64_t c0 = (int64_t)(s == 0 ? bi : bj) * kBlockCols + 4 * cg;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      ok[s][j]   = c0 + j < D;
      col[s][j]  = ok[s][j] ? c0 + j : 0;
      mean[s][j] = (mu != nullptr && ok[s][j]) ? mu[mean_index(a, col[s][j])] : T(0);
    }
  }

  acc_t acc[kTilesPerPair];
#pragma unroll
  for (int t = 0; t < kTilesPerPair; ++t)
    acc[t] = acc_t{0, 0, 0, 0};

  // A unit is UL wave-loads of four rows each: UR adjacent rows of the block(s).  Units are
  // dealt round-robin over the G waves that share the rows of a pair, the four waves of a
  // workgroup side by side, so the grid reads one compact, advancing window of the matrix
  // in contiguous pieces of 4 * UR rows per workgroup.
  const int64_t G     = (int64_t)a.S * kWaves;
  const int64_t g     = (int64_t)slab * kWaves + wave;
  // Rows that are no whole quads of columns are read as quads all the same, the last quad of a
  // row running up to three elements into the next row (masked like the columns beyond D): the
  // units of the main loop therefore end before the matrix's last row, which the guarded unit
  // reads element by element.  (Rows of one or two columns would reach beyond the next row.)
  const bool quads    = VEC || D >= 3;
  const int64_t nfull = (VEC || !quads) ? a.N / UR : (a.N - 1) / UR;
  const int64_t K     = g < nfull ? (nfull - g + G - 1) / G : 0;  // whole units of this wave

  auto load_unit = [&](Quad<T> (&x)[NS][UL], int64_t q, bool guard) {
#pragma unroll
    for (int u = 0; u < UL; ++u) {
      // the wave's first row of this load (uniform) plus the lane's row within it
      const int64_t r0 = q * UR + u * 4;
      const int64_t dr = (guard && r0 + lr >= a.N) ? a.N - 1 - r0 : lr;
      const T* rp      = data + r0 * D + dr * D;
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        if (VEC || (quads && !guard)) {
          x[s][u] = load_quad<T, STREAM>(rp + col[s][0]);
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            x[s][u].v[j] = rp[col[s][j]];
        }
      }
    }
  };
  // `live`: the unit exists (wave-uniform); `guard`: its rows may run past the matrix
  auto fold_unit = [&](const Quad<T> (&x)[NS][UL], int64_t q, bool live, bool guard) {
#pragma unroll
    for (int u = 0; u < UL; ++u) {
      const int64_t r = q * UR + u * 4 + lr;
      const bool in   = live && (!guard || r < a.N);
      T xa[4], xb[4];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        xa[j] = (ok[0][j] && in) ? x[0][u].v[j] - mean[0][j] : T(0);
      if constexpr (DIAG) {
        // (CENTER is a template parameter: a store behind a run-time flag, even one that is
        // never taken, makes the compiler wait for every load of the ring at the loop's top)
        if (CENTER && in) {
          if constexpr (VEC) {
            if (ok[0][0]) {
              Quad<T> w;
#pragma unroll
              for (int j = 0; j < 4; ++j)
                w.v[j] = xa[j];
              store_quad<T>(data + r * D + col[0][0], w);
            }
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
              if (ok[0][j]) data[r * D + col[0][j]] = xa[j];
          }
        }
#pragma unroll
        for (int ja = 0; ja < 4; ++ja)
#pragma unroll
          for (int jb = ja; jb < 4; ++jb)
            acc[ja * 4 + jb] = M::mma(xa[ja], xa[jb], acc[ja * 4 + jb]);
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          xb[j] = (ok[NS - 1][j] && in) ? x[NS - 1][u].v[j] - mean[NS - 1][j] : T(0);
#pragma unroll
        for (int ja = 0; ja < 4; ++ja)
#pragma unroll
          for (int jb = 0; jb < 4; ++jb)
            acc[ja * 4 + jb] = M::mma(xa[ja], xb[jb], acc[ja * 4 + jb]);
      }
    }
  };

  // A ring of P units: every slot is used and at once refilled with the unit P further on, so
  // the other slots' loads stay in flight behind the matrix instructions and no register is
  // copied.  All of it is unconditional (past the end a slot reloads the wave's last unit and
  // counts as zero): behind a branch, or with a copy of the prefetched registers at the loop's
  // end, the compiler waits for the prefetch before the next step and nothing overlaps.
  if (K > 0) {
    Quad<T> ring[P][NS][UL];
#pragma unroll
    for (int i = 0; i < P; ++i) {
      load_unit(ring[i], g + (i < K ? i : K - 1) * G, false);
      // in slot order, like the refills: issued in another order, the loop's first wait would
      // have to cover all of them on the way in, and so (the paths merge) on every trip
      __builtin_amdgcn_sched_barrier(0);
    }
    for (int64_t k0 = 0; k0 < K; k0 += P) {
#pragma unroll
      for (int i = 0; i < P; ++i) {
        const int64_t k = k0 + i;
        fold_unit(ring[i], g + k * G, k < K, false);
        __builtin_amdgcn_sched_barrier(0);
        load_unit(ring[i], g + (k + P < K ? k + P : K - 1) * G, false);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  // the rows after the last whole unit
  if (nfull * UR < a.N && g == nfull % G) {
    Quad<T> x[NS][UL];
    load_unit(x, nfull, true);
    fold_unit(x, nfull, true, true);
  }

  combine_waves<T, kTilesPerPair>(acc, sm, wave, lane);
  if (wave == 0) {
    T* out = static_cast<T*>(a.partial) + (int64_t)unit * kTilesPerPair * kTile;
#pragma unroll
    for (int ja = 0; ja < 4; ++ja)
#pragma unroll
      for (int jb = 0; jb < 4; ++jb)
        if (!DIAG || jb >= ja) store_tile<T>(out + (ja * 4 + jb) * kTile, acc[ja * 4 + jb], lane);
  }
}


// ---------------------------------------------------------------------------
// fp32 data on the bf16 matrix cores.  v_mfma_f32_16x16x4_f32 runs at 1/16 of the bf16
// rate (and, fed random data, at a clock that the power limit pulls down to 1.7-1.9 GHz), so
// fp32 Gram matrices are bound by it from 64 columns on.  Instead every centred value is
// split exactly into three bf16 terms, x = h + m + l with eight significant bits each (two
// truncations and two exact subtractions), and the product x * y is taken as
//   h h' + h m' + m h' + m m' + h l' + l h'
// with v_mfma_f32_16x16x32_bf16: products of bf16 values are exact in the fp32 accumulator,
// and the three terms left out (m l', l m', l l') are below 2^-23 |x y|, the size of one
// fp32 rounding of the product.  Six bf16 instructions of 32 rows take 96 cycles where eight
// fp32 ones take 256; the splitting is 5.5 vector instructions per value.
//
// Operand layout of the 16 x 16 x 32 instruction: lane l supplies, for row (A) or column (B)
// l % 16 of the tile, the eight k values 8 * (l / 16) .. + 7.  A unit is therefore 32 rows and
// a lane holds eight of them: rows 8 * (l / 16) + r of its four columns (row-major, load r)
// or eight consecutive rows of its column in each of the four groups (col-major).
// ---------------------------------------------------------------------------
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
constexpr int kBf16UnitRows = 32;

struct Split3 {
  u32x4 h, m, l;  // eight bf16 each, value 2 w in the low half of word w
};

__device__ __forceinline__ Split3 split_bf16x3(const float (&x)[8])
{
  Split3 s;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const float a = x[2 * w], b = x[2 * w + 1];
    const float ah = __uint_as_float(__float_as_uint(a) & 0xFFFF0000u);
    const float bh = __uint_as_float(__float_as_uint(b) & 0xFFFF0000u);
    const float ar = a - ah, br = b - bh;  // exact: the low 16 bits of the significand
    const float am = __uint_as_float(__float_as_uint(ar) & 0xFFFF0000u);
    const float bm = __uint_as_float(__float_as_uint(br) & 0xFFFF0000u);
    const float al = ar - am, bl = br - bm;  // exact, eight significant bits or fewer
    // the upper halves of two words side by side (v_perm_b32)
    s.h[w] = __builtin_amdgcn_perm(__float_as_uint(b), __float_as_uint(a), 0x07060302u);
    s.m[w] = __builtin_amdgcn_perm(__float_as_uint(br), __float_as_uint(ar), 0x07060302u);
    s.l[w] = __builtin_amdgcn_perm(__float_as_uint(bl), __float_as_uint(al), 0x07060302u);
  }
  return s;
}

using f32x4 = float __attribute__((ext_vector_type(4)));
__device__ __forceinline__ f32x4 mma_bf16(const u32x4& a, const u32x4& b, f32x4 c)
{
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                 __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// acc[ca * 4 + cb] += A-class ca x B-class cb over the unit's 32 rows, term by term so that
// consecutive instructions never wait for each other's accumulator
template <bool DIAG>
__device__ __forceinline__ void mma_unit_bf16(f32x4 (&acc)[kTilesPerPair], const Split3 (&A)[4],
                                              const Split3 (&B)[4])
{
#define RMI_COV_TERM(TA, TB)                                                      \
  _Pragma("unroll") for (int ca = 0; ca < 4; ++ca)                                \
    _Pragma("unroll") for (int cb = DIAG ? ca : 0; cb < 4; ++cb)                  \
      acc[ca * 4 + cb] = mma_bf16(A[ca].TA, B[cb].TB, acc[ca * 4 + cb]);
  RMI_COV_TERM(l, h)
  RMI_COV_TERM(h, l)
  RMI_COV_TERM(m, m)
  RMI_COV_TERM(m, h)
  RMI_COV_TERM(h, m)
  RMI_COV_TERM(h, h)
#undef RMI_COV_TERM
}

// The matrix instruction adds into its accumulator with truncation: over the hundreds of
// instructions of a wave's share of the rows a sum of squares came out 1e-5 too small.  So
// the instruction's accumulator is kept short-lived: every kBf16FlushTrips trips of the ring
// (a handful of units) it is added (an ordinary, correctly rounded fp32 addition) to a second
// set of totals and cleared, which leaves a bias of about 3 * units * 2^-25.
#ifndef RMI_COV_BF16_RING
#define RMI_COV_BF16_RING 3
#endif
constexpr int kBf16Ring       = RMI_COV_BF16_RING;  // units of 32 rows a wave keeps loaded or in flight
constexpr int kBf16FlushTrips = 2;
// The diagonal body (one column block against itself, the whole job when D <= 64) runs one
// wave per SIMD, so nothing but the wave's own instruction order can overlap the ~230 vector
// instructions that split a unit with the 60 matrix instructions that multiply one.  Its loop
// is therefore pipelined by hand: while unit k is multiplied, unit k + 1 is split into a
// second set of operands, and the scheduler is told to issue kPipeValuPerMma vector
// instructions behind every matrix instruction (a 16 x 16 x 32 instruction occupies the
// matrix core for 16 cycles and the issue port for 4).
#ifndef RMI_COV_BF16_PIPE_RING
#define RMI_COV_BF16_PIPE_RING 4
#endif
#ifndef RMI_COV_BF16_PIPE_VALU
#define RMI_COV_BF16_PIPE_VALU 4
#endif
constexpr int kPipeRing       = RMI_COV_BF16_PIPE_RING;  // even: the operand sets alternate
constexpr int kPipeValuPerMma = RMI_COV_BF16_PIPE_VALU;
constexpr int kPipeMmas       = 60;  // six terms of the ten tiles on and above the diagonal
static_assert(kPipeRing % 2 == 0, "operand sets alternate with the ring slots");
__device__ __forceinline__ void interleave_split_with_mma()
{
#pragma unroll
  for (int i = 0; i < kPipeMmas; ++i) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                // one matrix instruction
    __builtin_amdgcn_sched_group_barrier(0x002, kPipeValuPerMma, 0);  // vector instructions
  }
}
__device__ __forceinline__ void flush_tiles(f32x4 (&total)[kTilesPerPair], f32x4 (&acc)[kTilesPerPair])
{
#pragma unroll
  for (int t = 0; t < kTilesPerPair; ++t) {
    total[t] += acc[t];
    acc[t] = f32x4{0, 0, 0, 0};
  }
}

// FULL: the block has all of its 64 columns (and VEC holds), so nothing in the loop depends
// on a lane's column mask; together with a main loop over units that are all live this
// leaves the centring stores unconditional, and the loop body one basic block that the
// interleaving above applies to.
template <bool VEC, bool DIAG, bool CENTER, bool STREAM, bool FULL = false>
__device__ __forceinline__ void gram_rows_body_bf16(const GramArgs& a, int unit, int slab, int bi,
                                                    int bj, float* sm)
{
  using T          = float;
  constexpr int NS = DIAG ? 1 : 2;
  constexpr int UR = kBf16UnitRows;
  constexpr int P  = kBf16Ring;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform, see above
  const int g    = lane >> 4;  // the lane holds rows 8 g .. 8 g + 7 of a unit
  const int cg   = lane & 15;  // quad of columns within the block
  T* const data  = static_cast<T*>(a.data);
  const T* mu    = static_cast<const T*>(a.mu);
  const int64_t D = a.D;

  int64_t col[NS][4];
  bool ok[NS][4];
  T mean[NS][4];
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    const int64_t c0 = (int64_t)(s == 0 ? bi : bj) * kBlockCols + 4 * cg;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      ok[s][j]   = c0 + j < D;
      col[s][j]  = ok[s][j] ? c0 + j : 0;
      mean[s][j] = (mu != nullptr && ok[s][j]) ? mu[mean_index(a, col[s][j])] : T(0);
    }
  }

  f32x4 acc[kTilesPerPair], total[kTilesPerPair];
#pragma unroll
  for (int t = 0; t < kTilesPerPair; ++t)
    acc[t] = total[t] = f32x4{0, 0, 0, 0};

  const int64_t G     = (int64_t)a.S * kWaves;
  const int64_t gw    = (int64_t)slab * kWaves + wave;
  // (rows that are no whole quads of columns: see gram_rows_body)
  const bool quads    = VEC || D >= 3;
  const int64_t nfull = (VEC || !quads) ? a.N / UR : (a.N - 1) / UR;
  const int64_t K     = gw < nfull ? (nfull - gw + G - 1) / G : 0;

  auto load_unit = [&](Quad<T> (&x)[NS][8], int64_t q, bool guard) {
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const int64_t r0 = q * UR + r;   // uniform part of the row; the lane adds 8 g
      const int64_t dr = (guard && r0 + 8 * g >= a.N) ? a.N - 1 - r0 : 8 * g;
      const T* rp      = data + r0 * D + dr * D;
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        if (VEC || (quads && !guard)) {
          x[s][r] = load_quad<T, STREAM>(rp + col[s][0]);
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            x[s][r].v[j] = rp[col[s][j]];
        }
      }
    }
  };
  auto split_unit = [&](Split3 (&ops)[NS][4], const Quad<T> (&x)[NS][8], int64_t q, bool live,
                        bool guard) {
#pragma unroll
    for (int s = 0; s < NS; ++s) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float v[8];
#pragma unroll
        for (int r = 0; r < 8; ++r) {
          const bool in = live && (!guard || q * UR + 8 * g + r < a.N);
          v[r]          = ((FULL || ok[s][j]) && in) ? x[s][r].v[j] - mean[s][j] : T(0);
        }
        ops[s][j] = split_bf16x3(v);
      }
    }
    if constexpr (DIAG && CENTER) {
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        const int64_t row = q * UR + 8 * g + r;
        if (live && (!guard || row < a.N)) {
          if constexpr (VEC) {
            if (FULL || ok[0][0]) {
              Quad<T> w;
#pragma unroll
              for (int j = 0; j < 4; ++j)
                w.v[j] = x[0][r].v[j] - mean[0][j];
              store_quad<T, STREAM>(data + row * D + col[0][0], w);
            }
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
              if (ok[0][j]) data[row * D + col[0][j]] = x[0][r].v[j] - mean[0][j];
          }
        }
      }
    }
  };
  auto fold_unit = [&](const Quad<T> (&x)[NS][8], int64_t q, bool live, bool guard) {
    Split3 ops[NS][4];
    split_unit(ops, x, q, live, guard);
    mma_unit_bf16<DIAG>(acc, ops[0], ops[NS - 1]);
  };

  if constexpr (DIAG) {
    // pipelined: slot s of the ring holds the units s, s + PD, ...; unit k is multiplied from
    // operand set k % 2 while unit k + 1 is split into the other and its slot is refilled
    constexpr int PD = kPipeRing;
    if (K > 0) {
      Quad<T> ring[PD][NS][8];
#pragma unroll
      for (int i = 0; i < PD; ++i) {
        load_unit(ring[i], gw + (i < K ? i : K - 1) * G, false);
        __builtin_amdgcn_sched_barrier(0);
      }
      Split3 ops[2][NS][4];
      split_unit(ops[0], ring[0], gw, true, false);
      __builtin_amdgcn_sched_barrier(0);
      load_unit(ring[0], gw + (PD < K ? PD : K - 1) * G, false);
      __builtin_amdgcn_sched_barrier(0);
      // a trip of PD units; `all_live`: none of its units is past the wave's last one
      auto trip = [&](int64_t k0, auto all_live) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < PD; ++i) {
          const int64_t k = k0 + i;
          const int slot  = (i + 1) % PD;
          const bool live = decltype(all_live)::value || k + 1 < K;
          split_unit(ops[(i + 1) & 1], ring[slot], gw + (k + 1) * G, live, false);
          mma_unit_bf16<true>(acc, ops[i & 1][0], ops[i & 1][0]);
          interleave_split_with_mma();
          __builtin_amdgcn_sched_barrier(0);
          load_unit(ring[slot], gw + (k + 1 + PD < K ? k + 1 + PD : K - 1) * G, false);
          __builtin_amdgcn_sched_barrier(0);
        }
        flush_tiles(total, acc);
      };
      int64_t k0 = 0;
      for (; k0 + PD < K; k0 += PD)
        trip(k0, std::true_type{});
      for (; k0 < K; k0 += PD)
        trip(k0, std::false_type{});
    }
  } else
  // the ring of gram_rows_body: the other units in flight while one is split and multiplied
  if (K > 0) {
    Quad<T> ring[P][NS][8];
#pragma unroll
    for (int i = 0; i < P; ++i) {
      load_unit(ring[i], gw + (i < K ? i : K - 1) * G, false);
      __builtin_amdgcn_sched_barrier(0);
    }
    int trips = 0;
    for (int64_t k0 = 0; k0 < K; k0 += P) {
#pragma unroll
      for (int i = 0; i < P; ++i) {
        const int64_t k = k0 + i;
        fold_unit(ring[i], gw + k * G, k < K, false);
        __builtin_amdgcn_sched_barrier(0);
        load_unit(ring[i], gw + (k + P < K ? k + P : K - 1) * G, false);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (++trips == kBf16FlushTrips) {
        flush_tiles(total, acc);
        trips = 0;
      }
    }
  }
  if (nfull * UR < a.N && gw == nfull % G) {
    Quad<T> x[NS][8];
    load_unit(x, nfull, true);
    fold_unit(x, nfull, true, true);
  }

  flush_tiles(total, acc);
  combine_waves<T, kTilesPerPair>(total, sm, wave, lane);
  if (wave == 0) {
    T* out = static_cast<T*>(a.partial) + (int64_t)unit * kTilesPerPair * kTile;
#pragma unroll
    for (int ja = 0; ja < 4; ++ja)
#pragma unroll
      for (int jb = 0; jb < 4; ++jb)
        if (!DIAG || jb >= ja) store_tile<T>(out + (ja * 4 + jb) * kTile, total[ja * 4 + jb], lane);
  }
}

template <bool DIAG, bool CENTER, bool STREAM, bool FULL = false>
__device__ __forceinline__ void gram_cols_body_bf16(const GramArgs& a, int unit, int slab, int bi,
                                                    int bj, float* sm)
{
  using T          = float;
  constexpr int NS = DIAG ? 1 : 2;
  constexpr int UR = kBf16UnitRows;
  constexpr int P  = kBf16Ring;

  const int lane  = threadIdx.x & 63;
  const int wave  = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int g     = lane >> 4;  // the lane holds rows 8 g .. 8 g + 7 of a unit
  const int cl    = lane & 15;  // column within a group of 16
  T* const data   = static_cast<T*>(a.data);
  const T* mu     = static_cast<const T*>(a.mu);
  const int64_t N = a.N;

  T* colp[NS][4];
  bool ok[NS][4];
  T mean[NS][4];
#pragma unroll
  for (int s = 0; s < NS; ++s) {
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) {
      const int64_t c = (int64_t)(s == 0 ? bi : bj) * kBlockCols + 16 * gq + cl;
      ok[s][gq]       = c < a.D;
      colp[s][gq]     = data + col_offset(a, ok[s][gq] ? c : 0);
      mean[s][gq]     = (mu != nullptr && ok[s][gq]) ? mu[mean_index(a, c)] : T(0);
    }
  }

  f32x4 acc[kTilesPerPair], total[kTilesPerPair];
#pragma unroll
  for (int t = 0; t < kTilesPerPair; ++t)
    acc[t] = total[t] = f32x4{0, 0, 0, 0};

  const int64_t G     = (int64_t)a.S * kWaves;
  const int64_t gw    = (int64_t)slab * kWaves + wave;
  const int64_t nfull = N / UR;
  const int64_t K     = gw < nfull ? (nfull - gw + G - 1) / G : 0;

  // x[s][gq][h]: rows kLaneRows g + kHalfRows h .. + 3 of the unit in the lane's column of group gq
  constexpr int kLaneRows = 8, kHalfRows = 4;
  auto load_unit = [&](Quad<T> (&x)[NS][4][2], int64_t q, bool guard) {
    const int64_t r0 = q * UR + kLaneRows * g;
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
      for (int gq = 0; gq < 4; ++gq)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          if (!guard) {
            x[s][gq][h] = load_quad<T, STREAM>(colp[s][gq] + r0 + kHalfRows * h);
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const int64_t r  = r0 + kHalfRows * h + j;
              x[s][gq][h].v[j] = colp[s][gq][r < N ? r : N - 1];
            }
          }
        }
  };
  auto split_unit = [&](Split3 (&ops)[NS][4], const Quad<T> (&x)[NS][4][2], int64_t q, bool live,
                        bool guard) {
    const int64_t r0 = q * UR + kLaneRows * g;
#pragma unroll
    for (int s = 0; s < NS; ++s) {
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        float v[8];
#pragma unroll
        for (int r = 0; r < 8; ++r) {
          const bool in = live && (FULL || ok[s][gq]) && (!guard || r0 + kHalfRows * (r >> 2) + (r & 3) < N);
          v[r]          = in ? x[s][gq][r >> 2].v[r & 3] - mean[s][gq] : T(0);
        }
        if constexpr (DIAG && CENTER) {
          if (s == 0 && live && (FULL || ok[0][gq])) {
            if (!guard) {
#pragma unroll
              for (int h = 0; h < 2; ++h) {
                Quad<T> w;
#pragma unroll
                for (int j = 0; j < 4; ++j)
                  w.v[j] = v[4 * h + j];
                store_quad<T>(colp[0][gq] + r0 + kHalfRows * h, w);
              }
            } else {
#pragma unroll
              for (int r = 0; r < 8; ++r)
                if (r0 + kHalfRows * (r >> 2) + (r & 3) < N)
                  colp[0][gq][r0 + kHalfRows * (r >> 2) + (r & 3)] = v[r];
            }
          }
        }
        ops[s][gq] = split_bf16x3(v);
      }
    }
  };
  auto fold_unit = [&](const Quad<T> (&x)[NS][4][2], int64_t q, bool live, bool guard) {
    Split3 ops[NS][4];
    split_unit(ops, x, q, live, guard);
    mma_unit_bf16<DIAG>(acc, ops[0], ops[NS - 1]);
  };

  if constexpr (DIAG) {
    // Pipelined as in gram_rows_body_bf16.  The operand layout (lane = column, the lane groups
    // four runs of eight rows) makes a load instruction touch 64 lines, 16 bytes of each; the
    // units are therefore loaded in a coalesced layout instead (eight consecutive lanes read the
    // 128 bytes that a column has in the unit, eight columns per instruction) and turned into
    // the operand layout through the wave's own piece of LDS when they are split (10M x 64:
    // 458 -> 440 us; what is left to the row-major kernel's 380 us goes with the number of
    // columns, i.e. of streams 40 MB apart that every wave reads side by side).
    constexpr int PD      = kPipeRing;
    constexpr int kColLds = 128 + 16;  // bytes of a column in LDS: its 32 rows and a pad
    __shared__ __align__(16) char turn_lds[kWaves][kBlockCols * kColLds];
    char* const turn = turn_lds[wave];
    const int c8     = lane >> 3;  // coalesced layout: column 8 i + c8 of load i ...
    const int p8     = lane & 7;   // ... rows 4 p8 .. + 3 of the unit
    const T* cop[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int64_t c = (int64_t)bi * kBlockCols + 8 * i + c8;
      cop[i]          = data + col_offset(a, (FULL || c < a.D) ? c : 0) + 4 * p8;
    }
    auto load_unit_co = [&](Quad<T> (&x)[8], int64_t q) __attribute__((always_inline)) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        x[i] = load_quad<T, STREAM>(cop[i] + q * UR);
    };
    auto turn_unit = [&](Quad<T> (&x)[NS][4][2], const Quad<T> (&c)[8]) __attribute__((always_inline)) {
      typedef T full_t __attribute__((ext_vector_type(4)));
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        full_t v;
#pragma unroll
        for (int j = 0; j < 4; ++j)
          v[j] = c[i].v[j];
        *reinterpret_cast<full_t*>(turn + (8 * i + c8) * kColLds + 16 * p8) = v;
      }
#pragma unroll
      for (int gq = 0; gq < 4; ++gq)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const full_t v = *reinterpret_cast<const full_t*>(turn + (16 * gq + cl) * kColLds + 16 * (2 * g + h));
#pragma unroll
          for (int j = 0; j < 4; ++j)
            x[0][gq][h].v[j] = v[j];
        }
    };
    if (K > 0) {
      Quad<T> ring[PD][8];
#pragma unroll
      for (int i = 0; i < PD; ++i) {
        load_unit_co(ring[i], gw + (i < K ? i : K - 1) * G);
        __builtin_amdgcn_sched_barrier(0);
      }
      Split3 ops[2][NS][4];
      {
        Quad<T> x[NS][4][2];
        turn_unit(x, ring[0]);
        split_unit(ops[0], x, gw, true, false);
      }
      __builtin_amdgcn_sched_barrier(0);
      load_unit_co(ring[0], gw + (PD < K ? PD : K - 1) * G);
      __builtin_amdgcn_sched_barrier(0);
      // a trip of PD units; `all_live`: none of its units is past the wave's last one
      auto trip = [&](int64_t k0, auto all_live) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < PD; ++i) {
          const int64_t k = k0 + i;
          const int slot  = (i + 1) % PD;
          const bool live = decltype(all_live)::value || k + 1 < K;
          Quad<T> x[NS][4][2];
          turn_unit(x, ring[slot]);
          split_unit(ops[(i + 1) & 1], x, gw + (k + 1) * G, live, false);
          mma_unit_bf16<true>(acc, ops[i & 1][0], ops[i & 1][0]);
          interleave_split_with_mma();
          __builtin_amdgcn_sched_barrier(0);
          load_unit_co(ring[slot], gw + (k + 1 + PD < K ? k + 1 + PD : K - 1) * G);
          __builtin_amdgcn_sched_barrier(0);
        }
        flush_tiles(total, acc);
      };
      int64_t k0 = 0;
      for (; k0 + PD < K; k0 += PD)
        trip(k0, std::true_type{});
      for (; k0 < K; k0 += PD)
        trip(k0, std::false_type{});
    }
  } else if (K > 0) {
    Quad<T> ring[P][NS][4][2];
#pragma unroll
    for (int i = 0; i < P; ++i) {
      load_unit(ring[i], gw + (i < K ? i : K - 1) * G, false);
      __builtin_amdgcn_sched_barrier(0);
    }
    int trips = 0;
    for (int64_t k0 = 0; k0 < K; k0 += P) {
#pragma unroll
      for (int i = 0; i < P; ++i) {
        const int64_t k = k0 + i;
        fold_unit(ring[i], gw + k * G, k < K, false);
        __builtin_amdgcn_sched_barrier(0);
        load_unit(ring[i], gw + (k + P < K ? k + P : K - 1) * G, false);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (++trips == kBf16FlushTrips) {
        flush_tiles(total, acc);
        trips = 0;
      }
    }
  }
  if (nfull * UR < N && gw == nfull % G) {
    Quad<T> x[NS][4][2];
    load_unit(x, nfull, true);
    fold_unit(x, nfull, true, true);
  }

  flush_tiles(total, acc);
  combine_waves<T, kTilesPerPair>(total, sm, wave, lane);
  if (wave == 0) {
    T* out = static_cast<T*>(a.partial) + (int64_t)unit * kTilesPerPair * kTile;
#pragma unroll
    for (int ga = 0; ga < 4; ++ga)
#pragma unroll
      for (int gb = 0; gb < 4; ++gb)
        if (!DIAG || gb >= ga) store_tile<T>(out + (ga * 4 + gb) * kTile, total[ga * 4 + gb], lane);
  }
}

// ONE: the matrix has one column block (D <= 64), so only the diagonal body is compiled in,
// the kernel's register count is that body's, and the matrix, read once, is streamed past
// the caches (with several blocks the pairs of a slab share their rows through the L2).
template <class T, bool VEC, bool ONE, bool CENTER = false, bool FULL = false>
__global__ __launch_bounds__(kThreads) void gram_rows_kernel(GramArgs a)
{
  __shared__ T sm[kTilesPerPair * kTile];
  const int unit = xcd_local_unit();
  if (unit >= a.total) return;
  const int slab = unit / a.npairs;
  int bi, bj;
  pair_blocks(unit - slab * a.npairs, a.nb, bi, bj);
  // one wave-uniform branch around two bodies whose loads are unconditional
  static_assert(ONE || !CENTER, "the centred data is written back by the one-block kernel only");
  static_assert(!FULL || (ONE && VEC && std::is_same_v<T, float>), "FULL: one whole block of floats");
  if constexpr (std::is_same_v<T, float>) {  // bf16 matrix cores, three exact terms per value
    if (ONE || bi == bj) {
      gram_rows_body_bf16<VEC, true, CENTER, ONE, FULL>(a, unit, slab, bi, bj, sm);
    } else {
      if constexpr (!ONE) gram_rows_body_bf16<VEC, false, false, false>(a, unit, slab, bi, bj, sm);
    }
  } else if (ONE || bi == bj) {
    gram_rows_body<T, VEC, true, CENTER, ONE>(a, unit, slab, bi, bj, sm);
  } else {
    if constexpr (!ONE) gram_rows_body<T, VEC, false, false, false>(a, unit, slab, bi, bj, sm);
  }
}

// ---------------------------------------------------------------------------
// Col-major X: column c is N consecutive values at data + c * N.
// ---------------------------------------------------------------------------
template <class T, bool DIAG, bool CENTER, bool STREAM>
__device__ __forceinline__ void gram_cols_body(const GramArgs& a, int unit, int slab, int bi, int bj,
                                               T* sm)
{
  using M     = Mma<T>;
  using acc_t = typename M::acc_t;
  constexpr int NS = DIAG ? 1 : 2;
  constexpr int P  = ring_depth(NS * 16 * (int)sizeof(T) / 4);

  const int lane  = threadIdx.x & 63;
  const int wave  = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform, see above
  const int rq    = lane >> 4;  // quarter of the unit's rows
  const int cl    = lane & 15;  // column within a group of 16
  T* const data   = static_cast<T*>(a.data);
  const T* mu     = static_cast<const T*>(a.mu);
  const int64_t N = a.N;

  // the lane's column in each of the four groups of the block(s)
  T* colp[NS][4];
  bool ok[NS][4];
  T mean[NS][4];
#pragma unroll
  for (int s = 0; s < NS; ++s) {
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) {
      const int64_t c = (int64_t)(s == 0 ? bi : bj) * kBlockCols + 16 * gq + cl;
      ok[s][gq]       = c < a.D;
      colp[s][gq]     = data + col_offset(a, ok[s][gq] ? c : 0);
      mean[s][gq]     = (mu != nullptr && ok[s][gq]) ? mu[mean_index(a, c)] : T(0);
    }
  }

  acc_t acc[kTilesPerPair];
#pragma unroll
  for (int t = 0; t < kTilesPerPair; ++t)
    acc[t] = acc_t{0, 0, 0, 0};

  // A unit is sixteen rows: every lane holds four consecutive rows of its column in each
  // group, the four lane quarters four consecutive runs.
  const int64_t G     = (int64_t)a.S * kWaves;
  const int64_t g     = (int64_t)slab * kWaves + wave;
  const int64_t nfull = N / kColUnitRows;
  const int64_t K     = g < nfull ? (nfull - g + G - 1) / G : 0;

  auto load_unit = [&](Quad<T> (&x)[NS][4], int64_t q, bool guard) {
    const int64_t r0 = q * kColUnitRows + rq * 4;
#pragma unroll
    for (int s = 0; s < NS; ++s) {
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        if (!guard) {
          x[s][gq] = load_quad<T, STREAM>(colp[s][gq] + r0);
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            x[s][gq].v[j] = colp[s][gq][r0 + j < N ? r0 + j : N - 1];
        }
      }
    }
  };
  auto fold_unit = [&](const Quad<T> (&x)[NS][4], int64_t q, bool live, bool guard) {
    const int64_t r0 = q * kColUnitRows + rq * 4;
    Quad<T> c[NS][4];
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
      for (int gq = 0; gq < 4; ++gq)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const bool in = live && ok[s][gq] && (!guard || r0 + j < N);
          c[s][gq].v[j] = in ? x[s][gq].v[j] - mean[s][gq] : T(0);
        }
    if constexpr (DIAG) {
      if (CENTER && live) {
#pragma unroll
        for (int gq = 0; gq < 4; ++gq) {
          if (!ok[0][gq]) continue;
          if (!guard) {
            store_quad<T>(colp[0][gq] + r0, c[0][gq]);
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
              if (r0 + j < N) colp[0][gq][r0 + j] = c[0][gq].v[j];
          }
        }
      }
    }
#pragma unroll
    for (int ga = 0; ga < 4; ++ga)
#pragma unroll
      for (int gb = DIAG ? ga : 0; gb < 4; ++gb) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[ga * 4 + gb] = M::mma(c[0][ga].v[j], c[NS - 1][gb].v[j], acc[ga * 4 + gb]);
      }
  };

  // the same ring as gram_rows_body's
  if (K > 0) {
    Quad<T> ring[P][NS][4];
#pragma unroll
    for (int i = 0; i < P; ++i) {
      load_unit(ring[i], g + (i < K ? i : K - 1) * G, false);
      // in slot order, like the refills: issued in another order, the loop's first wait would
      // have to cover all of them on the way in, and so (the paths merge) on every trip
      __builtin_amdgcn_sched_barrier(0);
    }
    for (int64_t k0 = 0; k0 < K; k0 += P) {
#pragma unroll
      for (int i = 0; i < P; ++i) {
        const int64_t k = k0 + i;
        fold_unit(ring[i], g + k * G, k < K, false);
        __builtin_amdgcn_sched_barrier(0);
        load_unit(ring[i], g + (k + P < K ? k + P : K - 1) * G, false);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  if (nfull * kColUnitRows < N && g == nfull % G) {
    Quad<T> x[NS][4];
    load_unit(x, nfull, true);
    fold_unit(x, nfull, true, true);
  }

  combine_waves<T, kTilesPerPair>(acc, sm, wave, lane);
  if (wave == 0) {
    T* out = static_cast<T*>(a.partial) + (int64_t)unit * kTilesPerPair * kTile;
#pragma unroll
    for (int ga = 0; ga < 4; ++ga)
#pragma unroll
      for (int gb = 0; gb < 4; ++gb)
        if (!DIAG || gb >= ga) store_tile<T>(out + (ga * 4 + gb) * kTile, acc[ga * 4 + gb], lane);
  }
}

template <class T, bool ONE, bool CENTER = false, bool FULL = false>
__global__ __launch_bounds__(kThreads) void gram_cols_kernel(GramArgs a)
{
  __shared__ T sm[kTilesPerPair * kTile];
  const int unit = xcd_local_unit();
  if (unit >= a.total) return;
  const int slab = unit / a.npairs;
  int bi, bj;
  pair_blocks(unit - slab * a.npairs, a.nb, bi, bj);
  static_assert(ONE || !CENTER, "the centred data is written back by the one-block kernel only");
  if constexpr (std::is_same_v<T, float>) {
    if (ONE || bi == bj) {
      // (streamed loads where the units are loaded line by line, i.e. the one-block kernel that
      // does not write the data back: 10M x 64 437 -> 429 us; in the operand layout, where the
      // eight 16-byte pieces of a column's line are read by eight instructions, a streamed line
      // may be gone before the next piece is asked for: 450 -> 500 us)
      gram_cols_body_bf16<true, CENTER, ONE && !CENTER, FULL>(a, unit, slab, bi, bj, sm);
    } else {
      if constexpr (!ONE) gram_cols_body_bf16<false, false, false>(a, unit, slab, bi, bj, sm);
    }
  } else if (ONE || bi == bj) {
    gram_cols_body<T, true, CENTER, ONE>(a, unit, slab, bi, bj, sm);
  } else {
    if constexpr (!ONE) gram_cols_body<T, false, false, false>(a, unit, slab, bi, bj, sm);
  }
}

// ---------------------------------------------------------------------------
// Second pass: one workgroup per (pair, tile, quarter of the tile's 256 elements).  Thread
// (e, q) sums the slabs q, q + 16, ... of element e in f64, eight loads in flight, the
// sixteen meet in LDS in q order, the total is scaled and written to covar[r][c] and
// covar[c][r].
// ---------------------------------------------------------------------------
constexpr int kFoldElems = 64;  // elements of a tile per workgroup

template <class T>
__global__ __launch_bounds__(kFoldElems* kFoldSplit) void cov_fold_kernel(FoldArgs a)
{
  using M = Mma<T>;
  __shared__ double sm[kFoldSplit][kFoldElems];
  constexpr int kParts = kTile / kFoldElems;
  const int part = blockIdx.x % kParts;
  const int pt   = blockIdx.x / kParts;
  const int pair = pt / kTilesPerPair;
  const int tile = pt - pair * kTilesPerPair;
  const int ta   = tile >> 2;
  const int tb   = tile & 3;
  int bi, bj;
  pair_blocks(pair, a.nb, bi, bj);
  if (bi == bj && tb < ta) return;  // the lower triangle is the mirror of the upper

  const int le = threadIdx.x & (kFoldElems - 1);
  const int q  = threadIdx.x / kFoldElems;
  const int e  = part * kFoldElems + le;
  const T* p   = static_cast<const T*>(a.partial) + ((int64_t)pair * kTilesPerPair + tile) * kTile + e;
  const int64_t slab_stride = (int64_t)a.npairs * kTilesPerPair * kTile;
  double sum = 0.0;
  int s      = q;
  constexpr int U = 8;
  for (; s + (U - 1) * kFoldSplit < a.S; s += U * kFoldSplit) {
    T v[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
      v[u] = p[(int64_t)(s + u * kFoldSplit) * slab_stride];
#pragma unroll
    for (int u = 0; u < U; ++u)
      sum += (double)v[u];
  }
  for (; s < a.S; s += kFoldSplit)
    sum += (double)p[(int64_t)s * slab_stride];
  sm[q][le] = sum;
  __syncthreads();
  if (q != 0) return;
  for (int k = 1; k < kFoldSplit; ++k)
    sum += sm[k][le];

  const int lane = e & 63;
  const int m    = M::row(lane, e >> 6);
  const int n    = lane & 15;
  const int64_t r = (int64_t)bi * kBlockCols + (a.permuted ? 4 * m + ta : 16 * ta + m);
  const int64_t c = (int64_t)bj * kBlockCols + (a.permuted ? 4 * n + tb : 16 * tb + n);
  if (r >= a.D || c >= a.D) return;
  // A diagonal tile holds both (r, c) and (c, r), summed in two orders that may differ in the
  // last bit: its upper half is kept and mirrored like every other tile, so the result is
  // symmetric bit for bit.
  if (bi == bj && ta == tb && r > c) return;
  if (a.wide != nullptr) {
    a.wide[r * a.D + c] = sum * a.alpha;
    if (r != c) a.wide[c * a.D + r] = sum * a.alpha;
    return;
  }
  const T val = (T)(sum * a.alpha);
  T* out      = static_cast<T*>(a.out);
  out[r * a.D + c] = val;
  if (r != c) out[c * a.D + r] = val;
}

// A matrix of D <= 32 columns contracted as one of f D <= 64 (f consecutive rows side by side,
// row-major; the f pieces of every column side by side, col-major): its covariance is the sum
// of the f diagonal D x D blocks of the wide result (row-major: rows and columns b D + r; col-
// major: r f + b), summed in block order in f64 and rounded once.  The `left` rows that the
// contraction leaves over (row k, column r at tail[k tail_rs + r tail_cs]) are added here, from
// the data as it was given.
// One thread per element of the upper half; the lower half is its mirror.
template <class T>
__global__ __launch_bounds__(kThreads) void cov_blocks_kernel(const double* wide, T* out, int D, int f,
                                                              int row_major, const T* tail, const T* mu,
                                                              int left, int64_t tail_rs, int64_t tail_cs,
                                                              double alpha)
{
  const int i = blockIdx.x * kThreads + threadIdx.x;
  if (i >= D * D) return;
  const int r = i / D, c = i - r * D;
  if (r > c) return;
  double sum = 0.0;
  for (int b = 0; b < f; ++b) {
    const int wr = row_major ? b * D + r : r * f + b;
    const int wc = row_major ? b * D + c : c * f + b;
    sum += wide[wr * (f * D) + wc];  // the wide result has f D rows and columns
  }
  if (left > 0) {
    const double mr = mu != nullptr ? (double)mu[r] : 0.0, mc = mu != nullptr ? (double)mu[c] : 0.0;
    double rest     = 0.0;
    for (int k = 0; k < left; ++k)
      rest += ((double)tail[k * tail_rs + r * tail_cs] - mr) * ((double)tail[k * tail_rs + c * tail_cs] - mc);
    sum += rest * alpha;
  }
  out[r * D + c] = (T)sum;
  if (r != c) out[c * D + r] = (T)sum;
}

// the rows left over, centred like the others (after cov_blocks_kernel has read them)
template <class T>
__global__ __launch_bounds__(kThreads) void center_tail_kernel(T* tail, const T* mu, int left, int D,
                                                               int64_t tail_rs, int64_t tail_cs)
{
  for (int i = blockIdx.x * kThreads + threadIdx.x; i < left * D; i += gridDim.x * kThreads) {
    const int k = i / D, r = i - k * D;
    tail[k * tail_rs + r * tail_cs] -= mu[r];
  }
}

// ---------------------------------------------------------------------------
// data[n][c] -= mu[c], for matrices of more than one column block whose caller wants the
// centred data left behind (the kernels above then run with mu == nullptr).
// `lead` is the extent of the contiguous dimension, `by_lead` says that dimension is the
// columns (row-major); `total` = N * D.
// ---------------------------------------------------------------------------
template <class T>
__global__ __launch_bounds__(kThreads) void center_kernel(T* data, const T* mu, int64_t total,
                                                          int64_t lead, int by_lead)
{
  // element i sits at position i % lead of line i / lead; both are carried along the
  // grid-stride loop instead of divided out again
  const int64_t stride    = (int64_t)gridDim.x * kThreads;
  const int64_t step_line = stride / lead;
  const int64_t step_pos  = stride - step_line * lead;
  int64_t i               = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  int64_t line            = i / lead;
  int64_t pos             = i - line * lead;
  for (; i < total; i += stride) {
    data[i] -= mu[by_lead ? pos : line];
    line += step_line;
    pos += step_pos;
    if (pos >= lead) {
      pos -= lead;
      ++line;
    }
  }
}

}  // namespace cov
}  // namespace rmi
