// Host-side launch of one planned reduction for one accumulator policy.
// Every policy instantiates run<P>; a per-input-type translation unit collects
// them behind a lookup function so the policies compile in parallel.
#pragma once

#include <hip/hip_runtime.h>

#include "rmi_kernels.hpp"
#include "rmi_normalize.hpp"
#include "rmi_plan.hpp"

namespace rmi {

struct Problem {
  const void* in;
  void* ws;
  Epilogue epi;
};

using run_fn = int (*)(const PlanX&, const Problem&, hipStream_t);

// partials start after the workspace's ticket words
inline void* partials_of(void* ws) { return ws == nullptr ? nullptr : static_cast<char*>(ws) + kTicketBytes; }
inline int fold_lanes(int B) { return B >= 64 ? 64 : pow2ceil(B < 1 ? 1 : B); }

template <class P>
int launch_fold(const PlanX& pl, const Problem& pr, int B, hipStream_t st)
{
  FoldArgs f{};
  f.partial = partials_of(pr.ws);
  f.n_out   = pl.n_out;
  f.B       = B;
  f.LB      = fold_lanes(B);
  f.logLB   = ilog2(f.LB);
  f.epi     = pr.epi;
  const int64_t threads = pl.n_out * f.LB;
  const int64_t grid    = ceildiv(threads, kBlock);
  if (grid > 0x7fffffffLL) return RMI_ERR_BAD_SHAPE;
  hipLaunchKernelGGL((fold_kernel<P>), dim3((unsigned)grid), dim3(kBlock), 0, st, f);
  return RMI_OK;
}

template <class P, int K>
int launch_lanes(const PlanX& pl, const RowArgs& a, hipStream_t st)
{
  if constexpr (K <= P::VEC) {
    const dim3 grid((unsigned)pl.grid_blocks);
    if (pl.lanes_loads == 1)
      hipLaunchKernelGGL((row_lanes_kernel<P, K, 1>), grid, dim3(kBlock), 0, st, a);
    else
      hipLaunchKernelGGL((row_lanes_kernel<P, K, kUnroll>), grid, dim3(kBlock), 0, st, a);
    return RMI_OK;
  } else {
    return RMI_ERR_UNSUPPORTED;
  }
}

template <class P>
int run(const PlanX& pl, const Problem& pr, hipStream_t st)
{
  static_assert(kBlock == kPlanBlock && kUnroll == kPlanUnroll && kColUnroll == kPlanUnroll &&
                  kTeamUnroll == kPlanTeamUnroll && kStageBytes == kStageBytesPerWave &&
                  kFan == kTicketFan && kLineWords * 4 == kTicketLineBytes,
                "plan selector and kernels must agree on block size and unroll");
  static_assert(kSmallBytes == kPlanSmallBytes, "the planner's chunk of small rows is the kernel's");
  static_assert(col_wide_bundles(1) == col_wide_bundles_of(1) && col_wide_bundles(2) == col_wide_bundles_of(2) &&
                  col_wide_bundles(3) == col_wide_bundles_of(3) && col_wide_bundles(4) == col_wide_bundles_of(4) &&
                  col_wide_bundles(5) == col_wide_bundles_of(5) && kColWideMaxSets == 5 &&
                  kDenseSlots == kPlanDenseSlots && kDenseBundles == kPlanDenseBundles &&
                  kFlatChunkVec == kPlanFlatChunkVec && kFlatMaxVec == kPlanFlatMaxVec,
                "plan selector and wide-row column kernel must agree on rows per step");
  int rc = RMI_OK;
  switch (pl.kind) {
    case RMI_PLAN_EMPTY:
      if (pl.n_out > 0) rc = launch_fold<P>(pl, pr, 0, st);
      break;
    case RMI_PLAN_ROW_LANES:
    case RMI_PLAN_ROW_WAVE:
    case RMI_PLAN_ROW_BLOCK:
    case RMI_PLAN_ROW_SPLIT: {
      RowArgs a{};
      a.in      = pr.in;
      a.partial = partials_of(pr.ws);
      a.ticket  = pl.fused_fold ? static_cast<u32*>(pr.ws) : nullptr;
      a.LB      = fold_lanes(pl.B);
      a.n_out   = pl.n_out;
      a.len     = pl.len;
      a.row_bytes = pl.row_bytes;
      a.nvec    = pl.nvec;
      a.tail    = pl.tail;
      a.chunk   = pl.chunk;
      a.G       = pl.G;
      a.logG    = pl.logG;
      a.B       = pl.B;
      a.logT    = ilog2(pl.threads / 64);
      a.head_skip = pl.head_skip ? 1 : 0;
      a.epi     = pr.epi;
      const dim3 grid((unsigned)pl.grid_blocks);
      const unsigned lds = (unsigned)pl.lds_reserve;
      if (pl.kind == RMI_PLAN_ROW_LANES) {
        switch (pl.K) {
          case 2: rc = launch_lanes<P, 2>(pl, a, st); break;
          case 4: rc = launch_lanes<P, 4>(pl, a, st); break;
          case 8: rc = launch_lanes<P, 8>(pl, a, st); break;
          case 16: rc = launch_lanes<P, 16>(pl, a, st); break;
          default: rc = RMI_ERR_UNSUPPORTED;
        }
      } else if (pl.kind == RMI_PLAN_ROW_WAVE && !pl.team_kernel) {
        if (pl.small_rows) {
          a.chunk_rows = pl.chunk_rows;
          hipLaunchKernelGGL((row_small_kernel<P>), grid, dim3(kBlock), 0, st, a);
        } else if (pl.flat_rows) {
          if constexpr (sizeof(typename P::in_t) == 1 && P::kTail == kTailZero) {  // the planner's rule
            a.chunk_rows    = pl.chunk_rows;
            a.inv_row_bytes = 1.0f / (float)pl.row_bytes;
            hipLaunchKernelGGL((row_flat_kernel<P>), grid, dim3(kBlock), 0, st, a);
          } else {
            rc = RMI_ERR_UNSUPPORTED;
          }
        } else if (pl.dense_rows) {
          a.R = (kBlock * kDenseSlots) / pl.G;
          const size_t lds_bytes =
            (size_t)kDenseBundles * a.R * pl.G * sizeof(typename P::acc_t);  // at most 32 KB
          hipLaunchKernelGGL((row_dense_kernel<P>), grid, dim3(kBlock), lds_bytes, st, a);
        } else if (pl.short_rows) {
          if (pl.any_g) {
            a.R    = 64 / pl.G;
            a.invG = 65536u / (unsigned)pl.G + 1;
            a.invR = 65536u / (unsigned)a.R + 1;
            hipLaunchKernelGGL((row_short_kernel<P, true, true>), grid, dim3(kBlock), 0, st, a);
          } else if (pl.vec16)
            hipLaunchKernelGGL((row_short_kernel<P, true>), grid, dim3(kBlock), 0, st, a);
          else
            hipLaunchKernelGGL((row_short_kernel<P, false>), grid, dim3(kBlock), 0, st, a);
        } else {
          if (pl.vec16 && pl.staged)
            hipLaunchKernelGGL((row_wave_kernel<P, true, true>), grid, dim3(kBlock), lds, st, a);
          else if (pl.vec16)
            hipLaunchKernelGGL((row_wave_kernel<P, true>), grid, dim3(kBlock), lds, st, a);
          else
            hipLaunchKernelGGL((row_wave_kernel<P, false>), grid, dim3(kBlock), 0, st, a);
        }
      } else {
        const dim3 block((unsigned)(pl.threads < kBlock ? kBlock : pl.threads));
        if (pl.vec16)
          hipLaunchKernelGGL((row_block_kernel<P, true>), grid, block, lds, st, a);
        else
          hipLaunchKernelGGL((row_block_kernel<P, false>), grid, block, 0, st, a);
        if (pl.kind == RMI_PLAN_ROW_SPLIT && !pl.fused_fold) rc = launch_fold<P>(pl, pr, pl.B, st);
      }
      break;
    }
    case RMI_PLAN_COL_TILE: {
      ColArgs a{};
      a.in             = pr.in;
      a.partial        = partials_of(pr.ws);
      a.n_out          = pl.n_out;
      a.len            = pl.len;
      a.row_bytes      = pl.row_bytes;
      a.nvec           = pl.nvec;
      a.tail           = pl.tail;
      a.TX             = pl.TX;
      a.TY             = pl.TY;
      a.logTX          = pl.logTX;
      a.dense          = pl.dense ? 1 : 0;
      a.treeTY         = pow2ceil(pl.TY);
      a.B              = pl.B;
      a.epi            = pr.epi;
      if (pl.group > 0) {  // rows read in groups: a [group_len][group * n_out] matrix
        a.n_out     = pl.n_out * pl.group;
        a.len       = pl.group_len;
        a.row_bytes = pl.row_bytes * pl.group;
        a.nvec      = pl.group_nvec;
        a.tail      = 0;
        a.group     = pl.group;
        a.cols      = pl.n_out;
        a.rem       = (pl.len - pl.group_len * pl.group) * pl.n_out;
      }
      const dim3 grid((unsigned)pl.gridx, (unsigned)pl.B);
      if (pl.wide > 0) {
        if constexpr (P::CLS != kClsFloat && P::CLS != kClsKvp && !col_narrow<P>::value) {
          return RMI_ERR_UNSUPPORTED;  // planned for floating sums, arg-reductions and byte sums only
        } else {
          if (col_wide_sets<P>() != pl.wide) return RMI_ERR_UNSUPPORTED;
          const size_t lds_bytes = (size_t)pl.TY * pl.TX * P::VEC *
                                   (col_narrow<P>::value ? 4 : sizeof(typename P::acc_t));  // at most 64 KB
          hipLaunchKernelGGL((col_wide_kernel<P>), grid, dim3(kBlock), lds_bytes, st, a);
          FoldArgs f{};
          f.partial = partials_of(pr.ws);
          f.n_out   = pl.n_out;
          f.B       = pl.B;
          f.epi     = pr.epi;
          hipLaunchKernelGGL((fold_rows_kernel<P>), dim3((unsigned)ceildiv(pl.n_out, 16)),
                             dim3(kBlock), 0, st, f);
        }
        break;
      }
      if (pl.vec16)
        hipLaunchKernelGGL((col_kernel<P, true>), grid, dim3(kBlock), 0, st, a);
      else
        hipLaunchKernelGGL((col_kernel<P, false>), grid, dim3(kBlock), 0, st, a);
      if (pl.group > 0)
        rc = launch_fold<P>(pl, pr, pl.B * pl.group, st);
      else if (pl.B > 1)
        rc = launch_fold<P>(pl, pr, pl.B, st);
      break;
    }
    default: rc = RMI_ERR_BAD_ENUM;
  }
  if (rc != RMI_OK) return rc;
  return hipGetLastError() == hipSuccess ? RMI_OK : RMI_ERR_LAUNCH;
}

// ---- row normalisation -----------------------------------------------------------
struct NormPlan {
  bool vec16   = false;
  int kind     = 0;  // 0: lanes of a wave per row, 1: register-resident team, 2: two sweeps
  int G        = 1;
  int logG     = 0;
  int L        = 4;  // wave kernel: lane-loads per lane and row
  int tiles    = 1;  // wave kernel: rows per lane group and step
  int hold     = 4;  // team kernel: lane-loads held per thread
  int threads  = kBlock;
  int64_t grid = 0;
  int64_t nvec = 0;
  int tail     = 0;
  // kind 3, the flat kernel: `flat_rows` rows (ending on a 16-byte boundary) in chunks of
  // `chunk_rows`, 2^logL lanes per row for the fold; the rows after them take another plan
  int chunk_rows    = 0;
  int logL          = 0;
  int64_t flat_rows = 0;
};

// Rows that the flat kernel (normalize_flat_kernel) takes, or kind != 3 when it does not apply.
// It needs rows of 16 bytes or more and input and output on a 16-byte boundary, and it is
// chosen where the row-wise kernels' accesses do not fall on whole 128-byte lines, i.e. row
// bytes that are no multiple of 128: measured over 512 MB + 512 MB, fp32 rows of 5 to 1001
// elements 53-72 % -> 74-78.5 % of 8 TB/s (D = 129: 60 -> 76, 500: 63 -> 78), bf16 and fp16
// rows of 9 to 2000 43-70 % -> 72-78 %, fp64 rows of 25 to 250 56-67 % -> 65-68 %.  Not chosen,
// by the same measurements: rows of 16, 32 or 64 bytes (whole rows per power-of-two lane group:
// 75-80 % against 70-77 %), fp64 rows below 192 bytes (-2 to -20 %), and rows so long that the
// whole rows of a chunk fill less than 85 % of a workgroup's vector slots.
#ifndef RMI_NORM_WAVE_LONG
#define RMI_NORM_WAVE_LONG 1
#endif
#ifndef RMI_NORM_FLAT_MAX_ROW_BYTES
#define RMI_NORM_FLAT_MAX_ROW_BYTES 4096
#endif
inline NormPlan make_flat_norm_plan(int64_t n_rows, int64_t len, int elem_bytes, const void* in,
                                    const void* out)
{
  NormPlan p;
  const int64_t rb = len * elem_bytes;
  if (rb < 16 || rb % 128 == 0 || rb > RMI_NORM_FLAT_MAX_ROW_BYTES) return p;
  if ((rb & (rb - 1)) == 0) return p;
  if (elem_bytes == 8 && rb < 192) return p;
  if (reinterpret_cast<uintptr_t>(in) % 16 != 0 || reinterpret_cast<uintptr_t>(out) % 16 != 0) return p;
  int g = 16, r = (int)(rb % 16);
  while (r != 0) {  // gcd(16, rb)
    const int q = g % r;
    g = r, r = q;
  }
  const int m0 = 16 / g;  // rows after which a row starts on a 16-byte boundary again
  int chunk_rows = (int)((int64_t)kFlatMaxVec * 16 / rb / m0 * m0);
  if (chunk_rows <= 0 || n_rows < m0) return p;
  // a chunk that fills less than 85 % of the workgroup's 1024 vector slots leaves too many idle
  if ((int64_t)chunk_rows * rb * 100 < (int64_t)kFlatChunkVec * 16 * 85) return p;
  {
    // chunks of whole 128-byte lines where that still fills the workgroup well enough: chunk
    // edges inside a line make two workgroups read and write parts of it
    int g128 = 128, r128 = (int)(rb % 128);
    while (r128 != 0) {
      const int q = g128 % r128;
      g128 = r128, r128 = q;
    }
    const int m128   = 128 / g128;
    const int aligned_rows = (int)((int64_t)kFlatMaxVec * 16 / rb / m128 * m128);
    if (aligned_rows > 0 &&
        (int64_t)aligned_rows * rb * 100 >= (int64_t)kFlatChunkVec * 16 * 90)
      chunk_rows = aligned_rows;
  }
  const int vec_per_row = (int)((rb + 15) / 16);
  int L = 1, logL = 0;
  while (2 * L <= kWave && 2 * L * chunk_rows <= kBlock && 2 * L <= 2 * vec_per_row) L *= 2, ++logL;
  p.kind       = 3;
  p.vec16      = true;
  p.chunk_rows = chunk_rows;
  p.logL       = logL;
  p.flat_rows  = n_rows - n_rows % m0;
  p.grid       = ceildiv(p.flat_rows, (int64_t)chunk_rows);
  return p;
}

// Rows shorter than a vector through LDS (normalize_small_kernel), or kind != 4 when it does not
// apply: input and output on a 16-byte boundary.
inline NormPlan make_small_norm_plan(int64_t n_rows, int64_t len, int elem_bytes, const void* in,
                                     const void* out)
{
  NormPlan p;
  const int64_t rb = len * elem_bytes;
  if (rb >= 16 || rb < 1) return p;
  if (reinterpret_cast<uintptr_t>(in) % 16 != 0 || reinterpret_cast<uintptr_t>(out) % 16 != 0) return p;
  if (len < 2) return p;  // a row of one element: the lane-per-row kernels are as fast
  int chunk_rows = (int)(kSmallBytes / rb / 16 * 16);
  if (elem_bytes == 2 && len % 2 != 0 && chunk_rows > kSmallNormRows) chunk_rows = kSmallNormRows;
  if (chunk_rows < 32 || chunk_rows > 32 * kBlock) return p;
  p.kind       = 4;
  p.vec16      = true;
  p.chunk_rows = chunk_rows;
  p.grid       = ceildiv(n_rows, (int64_t)chunk_rows);
  return p;
}

inline NormPlan make_norm_plan(int64_t n_rows, int64_t len, int elem_bytes)
{
  NormPlan p;
  const int64_t row_bytes = len * elem_bytes;
  p.vec16                 = row_bytes >= 16;
  const int step          = p.vec16 ? 16 / elem_bytes : 1;
  p.nvec                  = len / step;
  p.tail                  = (int)(len % step);
  const int64_t nload     = p.nvec + (p.tail > 0 ? 1 : 0);
  if (nload <= (int64_t)kUnroll * kWave) {
    // at least 8 lanes (128 contiguous bytes) per row and load instruction where the
    // row is that long; shorter rows take one lane-load per lane and several rows
    p.L    = nload <= 8 ? 1 : (nload <= 16 ? 2 : 4);
    p.G    = pow2ceil(ceildiv(nload, p.L));
    p.L    = (int)ceildiv(nload, (int64_t)p.G);  // no load instruction without a lane-load
    p.logG  = ilog2(p.G);
    p.tiles = kUnroll / p.L;
    // Rows of 16, 32, 64 or 128 lane-loads: two loads per lane and ONE row per lane group and
    // step (half the default's bytes in flight per lane, twice the workgroups) measured 2-3 %
    // faster than four loads per lane or two rows per group on fp32, fp64 and bf16 rows
    // (1M x 128 floats 167 -> 162 us; a streaming copy is fastest at one load per lane too).
    if (p.vec16 && nload >= 16 && nload <= 128 && (nload & (nload - 1)) == 0) {
      p.L     = 2;
      p.G     = (int)(nload / 2);
      p.logG  = ilog2(p.G);
      p.tiles = 1;
    }
    p.grid = ceildiv(n_rows, (int64_t)(kWave / p.G) * p.tiles * (kBlock / kWave));
    // Lane-load counts that are not a power of two: one lane per lane-load and 64 / G whole
    // rows per wave step, so that every load and store instruction covers one contiguous
    // span (1M x 33 / 50 / 100 floats: 59 / 60 / 56 % -> 70 / 72 / 71 % of 8 TB/s in + out).
    // One row per step (33..63 lane-loads) pays from 54 lanes on (fp32 D = 220 / 250: 62 / 56 %
    // -> 70 / 67 %, bf16 D = 500: 56 -> 68 %; 50 lanes measured 2 points either way on fp32 and
    // lost 14 on bf16, D = 129 / 160 lose 10 points that way and keep the power-of-two groups).
    // (f64 rows, whose accumulators are twice as wide, lose 13 points with one row per step.)
    if (p.vec16 && (nload & (nload - 1)) != 0 &&
        ((nload >= 3 && nload <= 32) || (nload >= 54 && nload < 64 && elem_bytes < 8))) {
      p.L    = 0;
      p.G    = (int)nload;
      p.logG = 0;
      p.grid = ceildiv(n_rows, (int64_t)(kWave / p.G) * kUnroll * (kBlock / kWave));
    }
  } else if (RMI_NORM_WAVE_LONG != 0 && p.vec16 && nload < (int64_t)2 * kUnroll * kWave) {
    // 257 to 511 lane-loads: one wave per row with five to eight loads per lane, where a
    // 256-thread team holds one or two lane-loads per thread and a quarter to a half of its load
    // slots (256 MB in + out, % of 8 TB/s: bf16 D = 2049 / 2555 / 3137 / 3999: 41 / 50 / 60 / 69 -> 80 /
    // 80 / 80 / 79, fp32 D = 1025 / 1100 / 1500 / 2001: 66 / 71 / 75 / 74 -> 81 / 82 / 81 / 79, fp64 D = 513 /
    // 601 / 901: 62 / 71 / 74 -> 79 / 81 / 79; exactly 512 lane-loads: 79 / 79 / 78 -> 76 / 77 / 77, left
    // to the team)
    p.G     = kWave;
    p.logG  = 6;
    p.L     = (int)ceildiv(nload, (int64_t)kWave);
    p.tiles = 1;
    p.grid  = ceildiv(n_rows, (int64_t)(kBlock / kWave));
  } else {
    p.grid = n_rows;
    if (nload <= 256 * 4) {
      p.kind = 1, p.threads = 256, p.hold = 4;
    } else if (nload <= 256 * 8) {
      p.kind = 1, p.threads = 256, p.hold = 8;
    } else if (nload <= 1024 * 4) {
      p.kind = 1, p.threads = 1024, p.hold = 4;
    } else if (nload <= 1024 * 8) {
      p.kind = 1, p.threads = 1024, p.hold = 8;
    } else if (nload <= 1024 * 16) {
      p.kind = 1, p.threads = 1024, p.hold = 16;
    } else {
      p.kind = 2, p.threads = 1024;
    }
  }
  return p;
}

using norm_fn = int (*)(const NormPlan&, const NormArgs&, hipStream_t);

template <class P>
int run_normalize(const NormPlan& pl, const NormArgs& args, hipStream_t st)
{
  // fp32 rows: six resident workgroups per CU instead of the eight that fit (an LDS reservation
  // the kernels never touch): 512 MB in + out, D = 64 / 128 / 256 / 2048 / 4096 78.8 / 78.8 / 78.8 /
  // 78.4 / 76.7 -> 81.1 / 81.2 / 80.4 / 80.9 / 78.5 % of 8 TB/s, D = 401 / 777 / 1100 +1 to +3; five lose
  // 1-10 points at D <= 512 and 2048, four and three more; bf16 rows gain and lose by shape
  // (D = 256 / 16384 -2, D = 2049 / 4096 +1 to +2) and keep eight.
  const unsigned resident_lds = sizeof(typename P::in_t) == 4 ? (unsigned)(kLdsPerCu / 6 - 768) : 0u;
  NormArgs a = args;
  a.nvec     = pl.nvec;
  a.tail     = pl.tail;
  a.G        = pl.G;
  a.logG     = pl.logG;
  a.L        = pl.L;
  a.tiles    = pl.tiles;
  a.invG     = 65536u / (unsigned)(pl.G > 0 ? pl.G : 1) + 1;
  if (pl.grid > 0x7fffffffLL) return RMI_ERR_BAD_SHAPE;
  const dim3 grid((unsigned)pl.grid);
  if (pl.kind == 4) {
    a.chunk_rows = pl.chunk_rows;
    if constexpr (sizeof(typename P::in_t) == 2) {
      if (a.len % 2 != 0) {  // rows that share 32-bit words: scaled on the way out
        hipLaunchKernelGGL((normalize_small_kernel<P, true>), grid, dim3(kBlock), 0, st, a);
        return hipGetLastError() == hipSuccess ? RMI_OK : RMI_ERR_LAUNCH;
      }
    }
    hipLaunchKernelGGL((normalize_small_kernel<P, false>), grid, dim3(kBlock), 0, st, a);
  } else if (pl.kind == 3) {
    a.n_rows        = pl.flat_rows;
    a.chunk_rows    = pl.chunk_rows;
    a.logL          = pl.logL;
    a.inv_row_bytes = 1.0f / (float)a.row_bytes;
    hipLaunchKernelGGL((normalize_flat_kernel<P>), grid, dim3(kBlock), 0, st, a);
  } else if (pl.kind == 0) {
    if (!pl.vec16) {
      hipLaunchKernelGGL((normalize_wave_kernel<P, false>), grid, dim3(kBlock), 0, st, a);
    } else if ((a.row_bytes % 128 == 0 || (pl.L == 1 && ((kWave / pl.G) * a.row_bytes) % 128 == 0)) &&
               reinterpret_cast<uintptr_t>(a.out) % 128 == 0) {
      // every store instruction writes whole cache lines (rows of whole lines, or the rows
      // of one wave step together) at an aligned address: streamed stores
      hipLaunchKernelGGL((normalize_wave_kernel<P, true, true>), grid, dim3(kBlock), resident_lds, st, a);
    } else {
      hipLaunchKernelGGL((normalize_wave_kernel<P, true>), grid, dim3(kBlock), resident_lds, st, a);
    }
  } else if (pl.kind == 1) {
    // rows of 4 KB and more always hold whole vectors
    const dim3 block((unsigned)pl.threads);
    if (pl.hold == 4)
      hipLaunchKernelGGL((normalize_team_kernel<P, 4>), grid, block, resident_lds, st, a);
    else if (pl.hold == 8)
      hipLaunchKernelGGL((normalize_team_kernel<P, 8>), grid, block, resident_lds, st, a);
    else
      hipLaunchKernelGGL((normalize_team_kernel<P, 16>), grid, block, resident_lds, st, a);
  } else {
    hipLaunchKernelGGL((normalize_sweep_kernel<P>), grid, dim3(pl.threads), 0, st, a);
  }
  return hipGetLastError() == hipSuccess ? RMI_OK : RMI_ERR_LAUNCH;
}

// Norm functor pairs offered for one floating input type: (identity | sq | abs) with
// (add | max | min).
template <class InT, bool IS_F64>
norm_fn lookup_norm_for(int main_op, int red_op)
{
#define RMI_NORM_MAIN(RED_POLICY)                                   \
  switch (main_op) {                                                \
    case RMI_MAIN_IDENTITY: return &run_normalize<RED_POLICY(RMI_MAIN_IDENTITY)>; \
    case RMI_MAIN_SQ: return &run_normalize<RED_POLICY(RMI_MAIN_SQ)>;             \
    case RMI_MAIN_ABS: return &run_normalize<RED_POLICY(RMI_MAIN_ABS)>;           \
    default: return nullptr;                                        \
  }
  if (red_op == RMI_RED_ADD) {
    if constexpr (IS_F64) {
#define POL(M) PolKbn<InT, M>
      RMI_NORM_MAIN(POL)
#undef POL
    } else {
#define POL(M) PolF<InT, M, RMI_RED_ADD>
      RMI_NORM_MAIN(POL)
#undef POL
    }
  }
  if (red_op == RMI_RED_MAX) {
#define POL(M) PolF<InT, M, RMI_RED_MAX>
    RMI_NORM_MAIN(POL)
#undef POL
  }
  if (red_op == RMI_RED_MIN) {
#define POL(M) PolF<InT, M, RMI_RED_MIN>
    RMI_NORM_MAIN(POL)
#undef POL
  }
#undef RMI_NORM_MAIN
  return nullptr;
}

// Policies offered for one input type, keyed by PolicyKey.
template <class InT, bool IS_FLOAT_IN, bool IS_F64>
run_fn lookup_for(const PolicyKey& k)
{
#define RMI_MAIN_CASES(MK)                           \
  switch (k.main_op) {                               \
    case RMI_MAIN_IDENTITY: MK(RMI_MAIN_IDENTITY);   \
    case RMI_MAIN_SQ: MK(RMI_MAIN_SQ);               \
    case RMI_MAIN_ABS: MK(RMI_MAIN_ABS);             \
    case RMI_MAIN_NZ: MK(RMI_MAIN_NZ);               \
    default: return nullptr;                         \
  }
#define RMI_MAIN3_CASES(MK)                          \
  switch (k.main_op) {                               \
    case RMI_MAIN_IDENTITY: MK(RMI_MAIN_IDENTITY);   \
    case RMI_MAIN_SQ: MK(RMI_MAIN_SQ);               \
    case RMI_MAIN_ABS: MK(RMI_MAIN_ABS);             \
    default: return nullptr;                         \
  }
  switch (k.family) {
    case kFamFloat:
      if (k.red_op == RMI_RED_ADD) {
        if constexpr (!IS_F64) {
#define MK(M) return &run<PolF<InT, M, RMI_RED_ADD>>
          RMI_MAIN_CASES(MK)
#undef MK
        }
        return nullptr;
      }
      if constexpr (IS_FLOAT_IN) {
        if (k.red_op == RMI_RED_MAX) {
#define MK(M) return &run<PolF<InT, M, RMI_RED_MAX>>
          RMI_MAIN3_CASES(MK)
#undef MK
        }
        if (k.red_op == RMI_RED_MIN) {
#define MK(M) return &run<PolF<InT, M, RMI_RED_MIN>>
          RMI_MAIN3_CASES(MK)
#undef MK
        }
      }
      return nullptr;
    case kFamKbn:
      if constexpr (IS_F64) {
#define MK(M) return &run<PolKbn<InT, M>>
        RMI_MAIN_CASES(MK)
#undef MK
      }
      return nullptr;
    case kFamInt:
      if constexpr (!IS_FLOAT_IN) {
        if (k.red_op == RMI_RED_ADD) {
#define MK(M) return &run<PolI<InT, M, RMI_RED_ADD>>
          RMI_MAIN_CASES(MK)
#undef MK
        }
        if (k.red_op == RMI_RED_MAX) {
#define MK(M) return &run<PolI<InT, M, RMI_RED_MAX>>
          RMI_MAIN3_CASES(MK)
#undef MK
        }
        if (k.red_op == RMI_RED_MIN) {
#define MK(M) return &run<PolI<InT, M, RMI_RED_MIN>>
          RMI_MAIN3_CASES(MK)
#undef MK
        }
      }
      return nullptr;
    case kFamKvp:
      if constexpr (IS_FLOAT_IN) {
        const bool is_max = k.red_op == RMI_RED_ARGMAX;
        if (k.key64) {
          return is_max ? &run<PolKvp<InT, int64_t, true>> : &run<PolKvp<InT, int64_t, false>>;
        }
        return is_max ? &run<PolKvp<InT, int32_t, true>> : &run<PolKvp<InT, int32_t, false>>;
      }
      return nullptr;
    default: return nullptr;
  }
#undef RMI_MAIN_CASES
#undef RMI_MAIN3_CASES
}

// CU count of the current device (256 when none is visible), cached; rmi_api.hip
int cu_count();

// one definition per input type, each in its own translation unit
run_fn lookup_i8(const PolicyKey&);
run_fn lookup_u8(const PolicyKey&);
run_fn lookup_i32(const PolicyKey&);
run_fn lookup_i64(const PolicyKey&);
run_fn lookup_f16(const PolicyKey&);
run_fn lookup_bf16(const PolicyKey&);
run_fn lookup_f32(const PolicyKey&);
run_fn lookup_f64(const PolicyKey&);
norm_fn lookup_norm_f16(int main_op, int red_op);
norm_fn lookup_norm_bf16(int main_op, int red_op);
norm_fn lookup_norm_f32(int main_op, int red_op);
norm_fn lookup_norm_f64(int main_op, int red_op);
run_fn lookup_meanvar_f32();
run_fn lookup_meanvar_f64();
run_fn lookup_meanvar_f16();
run_fn lookup_meanvar_bf16();

}  // namespace rmi
