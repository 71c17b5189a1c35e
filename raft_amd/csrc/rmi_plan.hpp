// Host-only: validation of a reduction descriptor and the choice of launch
// plan by shape.  No HIP types here, so a plain g++ translation unit can use
// and test it.
//
// The reference picks among Thin / Medium / Thick kernels with thresholds tied
// to 32-lane warps and NVIDIA SM counts
// (linalg/detail/coalesced_reduction-inl.cuh:302-326,640-670) and launches the
// strided kernels with fixed block shapes
// (linalg/detail/strided_reduction.cuh:148-188).  The selector below is
// re-derived for 64-lane wavefronts, 16-byte lane loads and 256 CUs.
#pragma once

#include <stddef.h>
#include <stdint.h>

#include "rmi_reduce.h"

namespace rmi {

constexpr int kPlanBlock  = 256;
constexpr int kPlanUnroll = 4;      // lane-loads in flight: sub-wave and column kernels
constexpr int kPlanTeamUnroll = 4;  // lane-loads per batch: team-per-row kernel
constexpr int kTeamMinLoads   = 16; // a thread of a widened team keeps at least this many loads
constexpr int kWavesPerCu = 32;  // 8 resident waves on each of the 4 SIMDs
// Workgroups per CU of the persistent column kernel.  Measured on MI355X: with two
// tiles in flight per workgroup, 2 per CU (8 waves) sustains ~7.1 TB/s; 4 and 8 per CU
// lose 2 and 8 points to queueing in the memory system.
constexpr int kColBlocksPerCu = 2;
constexpr int kColMaxLanes = 128;     // COL_TILE: most lanes of a workgroup along one row
constexpr int kPlanDenseSlots   = 2;  // ROW_WAVE, dense rows: load slots per thread
constexpr int kPlanDenseBundles = 4;  // ... and bundles of rows in flight
constexpr int kPlanFlatChunkVec = 1024;  // ROW_WAVE, flat rows: vector slots of a workgroup
constexpr int kPlanFlatMaxVec   = kPlanFlatChunkVec - 7;  // ... and the most vectors of its chunk
constexpr int kColWideMaxSets = 5;    // COL_TILE, wide rows: most load slots per thread
// row bundles in flight in the wide-row column kernel whose threads have K load slots
constexpr int col_wide_bundles_of(int K) { return (10 + K - 1) / K; }
#ifndef RMI_LANES_AUTO
#define RMI_LANES_AUTO 0
#endif
#ifndef RMI_SMALL_ROWS
#define RMI_SMALL_ROWS 1
#endif
constexpr int kPlanSmallBytes = 16384;  // ROW_WAVE, small rows: bytes of a workgroup's chunk at most
#ifndef RMI_TEAM_ONE_TRIP
#define RMI_TEAM_ONE_TRIP 1
#endif
#ifndef RMI_COL_GROUP_OFF_WORDS
#define RMI_COL_GROUP_OFF_WORDS 1
#endif
#ifndef RMI_SPLIT_FINE
#define RMI_SPLIT_FINE 1
#endif
#ifndef RMI_HEAD_SKIP
#define RMI_HEAD_SKIP 1
#endif
#ifndef RMI_SPLIT_WG
#define RMI_SPLIT_WG 4
#endif
#ifndef RMI_TEAM_WG_ONE_TRIP
#define RMI_TEAM_WG_ONE_TRIP 6
#endif
#ifndef RMI_TEAM_OT_LOADS
#define RMI_TEAM_OT_LOADS 7
#endif

// ROW_SPLIT: long rows are cut into pieces of at least this many vectors (64 KB; twice that for
// the mean-and-variance accumulators, whose merges at a workgroup's end cost more), at most
// kSplitMaxPieces of them, also where fewer pieces would fill the machine's wave slots
constexpr int64_t kSplitPieceVecs = 4096;
constexpr int64_t kSplitMaxPieces = 32;
constexpr int64_t kGroupMaxRowBytes = 130;  // COL_TILE: longest row that is read in groups
constexpr int64_t kGroupMinLen = 256;  // COL_TILE: fewest row groups worth reading rows in groups
constexpr int kLdsPerCu       = 160 * 1024;  // LDS bytes of one gfx950 CU
constexpr int64_t kBytesInFlightPerCu = 80 * 1024;  // target of the wave-per-row plan
// LDS staging area of one wave: its rows (at most 64 lanes x 4 loads x 16 B) plus the
// lead-in of a line-aligned start and one vector of slack
constexpr int kStageBytesPerWave = 4096 + 128 + 16;
// The first bytes of every workspace are the ticket counters of the single-launch split
// plan; partials start after them, whatever the plan, so that a workspace shared by calls of
// different shapes keeps the counters intact.  A counter sits alone on a 128-byte line, and
// a row's workgroups first count in groups of kTicketFan, the last of each group counting
// once more for the row: atomics on one word are carried out one after the other (256
// workgroups per counter: 15.5 us on 8 rows of 4M bf16, groups of 16: 13.6 us).
inline int64_t ceildiv_i(int64_t a, int64_t b) { return (a + b - 1) / b; }
constexpr size_t kTicketBytes    = RMI_WORKSPACE_TICKET_BYTES;
constexpr int kTicketLineBytes   = 128;
constexpr int64_t kTicketLines   = kTicketBytes / kTicketLineBytes;
constexpr int kTicketFan         = 16;
// lines a split row needs: one per group of kTicketFan chunks, and the row's own
inline int64_t ticket_lines_per_row(int B) { return B <= kTicketFan ? 1 : ceildiv_i(B, kTicketFan) + 1; }

// Descriptor flag of the library's own (rmi_reduce_noalloc sets it on its copy of the
// descriptor, callers' descriptors that carry it are refused): the partials have to fit the
// static buffer of RMI_NOALLOC_SCRATCH_BYTES, so a plan whose partials outgrow it is passed
// over when another one serves the shape with fewer.
constexpr int32_t kFlagSmallWorkspace = 1 << 30;

struct PlanX {
  int kind        = RMI_PLAN_EMPTY;
  bool strided    = false;  // reduce along the strided dimension
  bool vec16      = false;  // 16-byte lane loads
  bool short_rows = false;  // ROW_WAVE served by the one-load-per-lane kernel
  bool any_g      = false;  // short_rows with G = the row's lane-load count (not a power of two)
  bool head_skip  = false;  // team kernel, rows of 1- or 2-byte elements: a row that starts
                            // off a 32-bit word gives its first one to three elements to the
                            // team's first thread and is read from the next whole word on
  bool dense_rows = false;  // ROW_WAVE: G = the row's lane-load count, a workgroup's load slots
                            // dealt over whole adjacent rows, rows combined through LDS
  bool flat_rows  = false;  // ROW_WAVE: the matrix is read as a flat run of aligned vectors, chunks
                            // of `chunk_rows` whole rows per workgroup, 2^logG lanes fold a row
  int chunk_rows  = 0;
  bool team_kernel = false; // served by the team-per-row kernel
  bool small_rows  = false; // ROW_WAVE: rows shorter than a vector that do not divide one, kPlanSmallChunk
                            // whole rows per workgroup through LDS
  bool stage_ok    = false; // ROW_WAVE: rows could be staged through LDS
  bool staged      = false; // ROW_WAVE: rows are staged through LDS (line-aligned span reads)
  int elem_bytes  = 0;
  int step        = 1;  // elements per lane-load
  int64_t n_out   = 0;
  int64_t len     = 0;  // elements folded into one output
  int64_t nvec    = 0;  // whole lane-loads along the contiguous dimension
  int tail        = 0;  // vec16: elements after the last whole vector
  int64_t row_bytes = 0; // bytes of one row of the contiguous dimension
  int K           = 0;  // ROW_LANES: rows per 16-byte vector
  int lanes_loads = kPlanUnroll;  // ROW_LANES: lane-loads per lane (1 or kPlanUnroll)
  int G           = 1;  // ROW_WAVE: lanes per row
  int logG        = 0;
  int threads     = kPlanBlock;  // ROW_BLOCK / ROW_SPLIT block size
  int B           = 1;           // partials per output
  int64_t chunk   = 0;           // ROW_SPLIT: lane-loads per block
  int TX          = 1;           // COL_TILE: lanes along a row per workgroup
  int TY          = 1;           // COL_TILE: rows per workgroup step (TX * TY <= block)
  int logTX       = 0;           // COL_TILE: log2(TX) when TX is a power of two
  bool dense      = false;       // COL_TILE: TX is not a power of two
  int64_t gridx   = 0;  // COL_TILE: blocks along the contiguous dimension
  int group       = 0;  // COL_TILE: > 0 when `group` consecutive rows are read as one row
  int64_t group_len  = 0;  // COL_TILE, grouped: whole groups (rows of the widened matrix)
  int64_t group_nvec = 0;  // COL_TILE, grouped: 16-byte vectors per group
  int wide        = 0;  // COL_TILE: > 0 when a workgroup streams whole rows, or one of gridx equal
                        // pieces of them (TX lane-loads each, TY rows side by side in the `wide`
                        // load slots of its threads; partials laid out [B][n_out])
  int64_t grid_blocks    = 0;
  int passes             = 1;
  bool fused_fold        = false;  // ROW_SPLIT: the last workgroup of a row folds its partials
  int lds_reserve        = 0;  // dynamic LDS bytes reserved only to cap occupancy
  int acc_bytes          = 8;
  size_t ws_bytes        = 0;
};

inline int dtype_size(int dt)
{
  switch (dt) {
    case RMI_I8:
    case RMI_U8: return 1;
    case RMI_F16:
    case RMI_BF16: return 2;
    case RMI_I32:
    case RMI_F32: return 4;
    case RMI_I64:
    case RMI_F64:
    case RMI_KVP_I32_F32: return 8;
    case RMI_KVP_I32_F64:
    case RMI_KVP_I64_F32:
    case RMI_KVP_I64_F64: return 16;
    default: return 0;
  }
}

inline bool is_float_dtype(int dt)
{
  return dt == RMI_F16 || dt == RMI_BF16 || dt == RMI_F32 || dt == RMI_F64;
}
inline bool is_int_dtype(int dt)
{
  return dt == RMI_I8 || dt == RMI_U8 || dt == RMI_I32 || dt == RMI_I64;
}
inline bool is_kvp_dtype(int dt) { return dt >= RMI_KVP_I32_F32 && dt <= RMI_KVP_I64_F64; }

// Which accumulator family serves a descriptor.
enum : int { kFamFloat = 0, kFamKbn = 1, kFamInt = 2, kFamKvp = 3, kFamMeanVar = 4 };

struct PolicyKey {
  int in_dtype = 0;
  int family   = 0;
  int main_op  = 0;
  int red_op   = 0;
  int key64    = 0;  // kFamKvp: 64-bit keys
};

inline int pow2ceil(int64_t x)
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
inline int64_t ceildiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Validates enums, dtype/functor compatibility and shape; fills `key` and the
// accumulator size.  Returns an rmi_status.
inline int classify(const rmi_reduce_desc& d, PolicyKey& key, int& acc_bytes)
{
  if (d.in_dtype < 0 || d.in_dtype >= RMI_DTYPE_COUNT_ || d.out_dtype < 0 ||
      d.out_dtype >= RMI_DTYPE_COUNT_)
    return RMI_ERR_BAD_ENUM;
  if (d.layout != RMI_ROW_MAJOR && d.layout != RMI_COL_MAJOR) return RMI_ERR_BAD_ENUM;
  if (d.apply != RMI_ALONG_ROWS && d.apply != RMI_ALONG_COLUMNS) return RMI_ERR_BAD_ENUM;
  if (d.main_op < RMI_MAIN_IDENTITY || d.main_op > RMI_MAIN_KVP) return RMI_ERR_BAD_ENUM;
  if (d.reduce_op < RMI_RED_ADD || d.reduce_op > RMI_RED_ARGMIN) return RMI_ERR_BAD_ENUM;
  if (d.final_op < RMI_FIN_IDENTITY || d.final_op > RMI_FIN_KEY) return RMI_ERR_BAD_ENUM;
  if (d.plan_hint < RMI_PLAN_AUTO || d.plan_hint > RMI_PLAN_EMPTY) return RMI_ERR_BAD_ENUM;
  if ((d.flags & ~(RMI_FLAG_WORKSPACE_ZEROED | kFlagSmallWorkspace)) != 0) return RMI_ERR_BAD_ENUM;
  if (d.n_rows < 0 || d.n_cols < 0) return RMI_ERR_BAD_SHAPE;
  if (is_kvp_dtype(d.in_dtype)) return RMI_ERR_UNSUPPORTED;

  const bool arg = d.reduce_op == RMI_RED_ARGMAX || d.reduce_op == RMI_RED_ARGMIN;
  key.in_dtype   = d.in_dtype;
  key.main_op    = d.main_op;
  key.red_op     = d.reduce_op;
  key.key64      = 0;
  if (arg) {
    // value -> {index, value}, arg-reduce, then either the pair or its key
    if (d.main_op != RMI_MAIN_KVP) return RMI_ERR_UNSUPPORTED;
    if (!is_float_dtype(d.in_dtype)) return RMI_ERR_UNSUPPORTED;
    const bool val64 = d.in_dtype == RMI_F64;
    if (d.final_op == RMI_FIN_KEY) {
      if (d.out_dtype != RMI_I32 && d.out_dtype != RMI_I64) return RMI_ERR_UNSUPPORTED;
      if (d.inplace) return RMI_ERR_UNSUPPORTED;
      key.key64 = d.out_dtype == RMI_I64;
    } else if (d.final_op == RMI_FIN_IDENTITY) {
      if (!is_kvp_dtype(d.out_dtype)) return RMI_ERR_UNSUPPORTED;
      const bool out_val64 = d.out_dtype == RMI_KVP_I32_F64 || d.out_dtype == RMI_KVP_I64_F64;
      if (out_val64 != val64) return RMI_ERR_UNSUPPORTED;
      key.key64 = d.out_dtype == RMI_KVP_I64_F32 || d.out_dtype == RMI_KVP_I64_F64;
    } else {
      return RMI_ERR_UNSUPPORTED;
    }
    key.family = kFamKvp;
    acc_bytes  = (key.key64 || val64) ? 16 : 8;
  } else {
    if (d.main_op == RMI_MAIN_KVP || d.final_op == RMI_FIN_KEY) return RMI_ERR_UNSUPPORTED;
    if (is_kvp_dtype(d.out_dtype)) return RMI_ERR_UNSUPPORTED;
    if (is_float_dtype(d.out_dtype)) {
      if (d.in_dtype == RMI_F64 && d.reduce_op == RMI_RED_ADD) {
        key.family = kFamKbn;
        acc_bytes  = 16;
      } else {
        // integers feeding a floating output are only summed (means, norms)
        if (is_int_dtype(d.in_dtype) && d.reduce_op != RMI_RED_ADD) return RMI_ERR_UNSUPPORTED;
        key.family = kFamFloat;
        acc_bytes  = 8;
      }
      if ((d.final_op == RMI_FIN_VAR_FROM_SUMSQ || d.final_op == RMI_FIN_STDDEV_FROM_SUMSQ) &&
          d.final_aux == nullptr)
        return RMI_ERR_NULL;
    } else {
      // integer output: integer input, integer arithmetic end to end
      if (!is_int_dtype(d.in_dtype)) return RMI_ERR_UNSUPPORTED;
      if (d.out_dtype != RMI_I32 && d.out_dtype != RMI_I64) return RMI_ERR_UNSUPPORTED;
      if (d.final_op == RMI_FIN_SQRT || d.final_op == RMI_FIN_VAR_FROM_SUMSQ ||
          d.final_op == RMI_FIN_STDDEV_FROM_SUMSQ)
        return RMI_ERR_UNSUPPORTED;
      key.family = kFamInt;
      acc_bytes  = 8;
    }
    if (d.main_op == RMI_MAIN_NZ && d.reduce_op != RMI_RED_ADD) return RMI_ERR_UNSUPPORTED;
  }
  return RMI_OK;
}

// Shape -> plan.  desc.plan_hint forces a plan kind where it applies to the shape.
// Few long rows on wide teams: `cap` teams are resident at once, and the teams of a last,
// partly filled round each run at what their own loads in flight allow (a 1024-thread team
// alone reads ~ 60 GB/s), so 525 rows take as long as 1024.  Rows of at least four pieces are
// split instead (2 GB of fp32, 525 / 600 / 900 / 1300 / 1800 rows: 68 / 81 / 80 / 75 / 76 -> 82 / 86 /
// 84 / 84 / 84 % of 8 TB/s; the mean-and-variance accumulators 512 MB, 525 / 900 / 1300 rows: 58 /
// 63 / 68 -> 74 / 73 / 73 %; 512, 1024 and 2047 rows, whose rounds are full, stay whole: 86-88 %,
// and so do last rounds that are nine tenths full).  Shorter rows get teams of half the width,
// which all fit at once (128 MB, 525 / 768 / 1000 rows: 60 / 66 / 64 -> 64 / 72 / 76 %,
// mean and variance 1000 / 1536 / 2047 rows: 34 / 44 / 39 -> 51 / 58 / 60 %; on rows long enough
// to split, the half-filled machine measured 3-5 points slower than the wide teams).
enum : int { kTailKeep = 0, kTailSplit = 1, kTailNarrow = 2 };
inline int tail_round_rule(int64_t n_rows, int64_t cap, int64_t nvec, int64_t piece)
{
  if (cap < 1 || n_rows <= cap || n_rows % cap == 0) return kTailKeep;
  if (nvec / piece < 4) return kTailNarrow;
  return (n_rows % cap) * 10 < cap * 9 ? kTailSplit : kTailKeep;
}

inline int make_plan(const rmi_reduce_desc& d,
                     const PolicyKey& key,
                     int acc_bytes,
                     int n_cu,
                     PlanX& p,
                     uintptr_t in_misalign = 0)  // the input pointer modulo 128, when known
{
  p            = PlanX{};
  p.acc_bytes  = acc_bytes;
  p.elem_bytes = dtype_size(d.in_dtype);
  const int es = p.elem_bytes;
  // (row-major, along rows) and (col-major, along columns) fold the contiguous
  // dimension; the other two fold the strided one (linalg/detail/reduce.cuh:36-48).
  const bool row_major = d.layout == RMI_ROW_MAJOR;
  const bool along_rows = d.apply == RMI_ALONG_ROWS;
  p.strided            = row_major != along_rows;
  const int64_t contiguous = row_major ? d.n_cols : d.n_rows;
  const int64_t other      = row_major ? d.n_rows : d.n_cols;
  p.n_out = p.strided ? contiguous : other;
  p.len   = p.strided ? other : contiguous;

  if (key.family == kFamKvp && !key.key64 && p.len > (int64_t)INT32_MAX) return RMI_ERR_BAD_SHAPE;
  if (p.n_out > ((int64_t)1 << 40) || p.len > ((int64_t)1 << 40)) return RMI_ERR_BAD_SHAPE;

  const int64_t slots = (int64_t)n_cu * kWavesPerCu;
  const int hint      = d.plan_hint;

  if (p.n_out == 0) {
    p.kind = RMI_PLAN_EMPTY;
    p.passes = 0;
    return RMI_OK;
  }
  if (p.len == 0) {
    p.kind        = RMI_PLAN_EMPTY;
    p.grid_blocks = ceildiv(p.n_out, kPlanBlock);
    return RMI_OK;
  }

  // Rows of at least 16 bytes are read as 16-byte vectors (at any alignment)
  // plus up to VEC-1 tail elements; shorter rows element by element.
  const int64_t row_bytes = contiguous * es;
  p.row_bytes             = row_bytes;
  p.vec16                 = row_bytes >= 16;
  p.step                  = p.vec16 ? 16 / es : 1;
  p.nvec                  = contiguous / p.step;
  p.tail                  = (int)(contiguous % p.step);
  // lane-loads a row needs, counting the tail elements as one more
  const int64_t nload = p.nvec + (p.tail > 0 ? 1 : 0);

  if (p.strided) {
    p.kind = RMI_PLAN_COL_TILE;
    // Rows shorter than one 16-byte vector would be read element by element.  The matrix is
    // one contiguous array, so `group` consecutive rows whose bytes add up to whole vectors
    // are read as ONE row of a matrix with len / group rows.  A thread's columns of the
    // widened row are fixed real columns (widened column c is real column c % n_out of row
    // c / n_out within the group), so each real column ends up with group * B partials,
    // which the second pass folds; the rows after the last whole group are added element by
    // element.  Reductions that need the row index (arg-reductions) stay on the plain path,
    // as do inputs that do not start on a 16-byte boundary and matrices with fewer than
    // kGroupMinLen groups.
    // Rows of up to 130 bytes that are an odd number of bytes or of 16-bit elements are grouped
    // as well: their vectors would start 1 or 2 bytes off a 4-byte boundary, which costs a
    // plain read a quarter of its rate (rows 4 or 8 bytes off read like aligned ones).  512 MB,
    // % of 8 TB/s, plain / grouped: bf16 D = 9 / 17 / 33 / 65: 42 / 50 / 63 / 71 -> 78 / 78 / 78 / 73,
    // int8 D = 17 / 18 / 33 / 50 / 65 / 126: 39 / 41 / 47 / 53 / 56 / 70 -> 71 / 75 / 72 / 74 / 65 / 73;
    // longer rows lose (bf16 D = 101 / 127: 75 / 77 -> 72 / 71, int8 D = 127: 66 -> 63).
    int64_t lanes = nload, rows = p.len;
    const int64_t low = row_bytes & -row_bytes;  // largest power of two in row_bytes
    const bool short_rows = row_bytes < 16;
    // (a group multiplies the partials; the entry point without allocation keeps the plain
    // layout where they would outgrow its buffer)
    const bool off_words = RMI_COL_GROUP_OFF_WORDS != 0 && row_bytes > 16 && low <= 2 &&
                           row_bytes <= kGroupMaxRowBytes && row_bytes / low <= kColMaxLanes &&
                           !((d.flags & kFlagSmallWorkspace) != 0 &&
                             kTicketBytes + (size_t)p.n_out * (16 / low) * ((size_t)n_cu * (kColBlocksPerCu + 1)) *
                                 acc_bytes > RMI_NOALLOC_SCRATCH_BYTES);
    if (key.family != kFamKvp && (short_rows || off_words) && (in_misalign % 16) == 0) {
      if (p.len / (16 / low) >= kGroupMinLen) {
        p.group      = (int)(16 / low);
        p.group_len  = p.len / p.group;
        p.group_nvec = row_bytes / low;
        p.vec16      = true;
        lanes        = p.group_nvec;
        rows         = p.group_len;
      }
    }
    // A workgroup covers TX lane-loads of a row times TY rows per step.  Rows of up to
    // kColMaxLanes lane-loads take exactly that many lanes, and as many whole rows as fit the
    // workgroup: its step then reads one contiguous span, and 33 lane-loads keep 231 of 256
    // lanes busy where a power-of-two 64 would idle every other lane.  Longer rows are cut
    // into the fewest equal pieces of at most kColMaxLanes lanes.  (Measured at 512 MB fp32,
    // D = 260 / 300 / 517 / 4097: 83 / 82 / 77 / 67 % this way, 70 / 71 / 61 / 54 % with
    // pieces of at most 64 lanes; reading such rows in aligned groups did not help.)
    // Rows that are whole multiples of 64 lane-loads keep pieces of exactly 64 lanes (1 KB
    // at a 1 KB stride within the row, four rows per step): 32768 x 32768 floats read 86 %
    // that way and 70 % in 128-lane pieces.
    {
      const int64_t cuts = lanes % 64 == 0 ? lanes / 64 : ceildiv(lanes, kColMaxLanes);
      p.TX    = (int)ceildiv(lanes, cuts);
      p.TY    = kPlanBlock / p.TX;
      p.gridx = ceildiv(lanes, p.TX);
      p.dense = (p.TX & (p.TX - 1)) != 0 || p.TX > 64;
      p.logTX = p.dense ? 0 : ilog2(p.TX);
    }
    // Rows of more than kColMaxLanes lane-loads: a workgroup streams whole adjacent rows (or,
    // of rows that outgrow it, one of the fewest equal pieces), i.e. long contiguous spans.
    // A thread has K load slots, as many as 256 bytes of accumulators allow (5 for 4- and
    // 8-byte elements, 4 for 2-byte ones); the workgroup's 256 * K slots take the lane-loads of
    // 256 * K / piece adjacent rows (a bundle: more than half of the slots get a lane-load),
    // ten or so lane-loads per thread are in flight, one workgroup per CU in all (a 257th
    // workgroup would share a CU and finish last: 3 pieces x 86 workgroups ran 15 % slower than
    // the layout above, 3 x 85 run 20 % faster).  Taken when every workgroup gets sixteen steps
    // or more (4096 x 4097 floats lose 16 % with eight).  Accumulators whose step is
    // arithmetic-bound at four waves per CU (byte sums in 64-bit accumulators: 25 % slower)
    // keep the layout above, and so do rows of several pieces that are whole multiples of 64
    // whole lane-loads, its best case (fp32 D = 32768 / 65536: 80 / 83 % there, 76 / 75 % this
    // way).  Arg-reductions were such accumulators (33-38 % slower here) until they walked
    // their rows downwards; now fp32 arg-max D = 1000 / 2049 / 4097 / 10000 runs 72 / 70 / 71 /
    // 73 % there and 75 / 75 / 73 / 72 % this way.
    // Measured at 512 MB, % of 8 TB/s, the layout above / this one: fp32 D = 513: 76 / 81,
    // 768: 74 / 82, 1025: 70 / 80, 1536: 73 / 82, 2049: 66 / 80, 3000: 65 / 78, 4096: 72 / 81,
    // 4097: 67 / 78, 8191: 71 / 77, 11000: 66 / 81, 14000: 67 / 78, 22000: 66 / 79, 50000: 70 / 77,
    // 200000: 66 / 72 (640 and 1024: 84 / 81 and 82 / 81); fp64 D = 300: 76 / 82, 1025: 67 / 82,
    // 4097: 61 / 80, 8191: 70 / 79; bf16 D = 1030: 72 / 80, 10000: 62 / 72, 16400: 59 / 75.
    // Byte sums gather in 32-bit accumulators here (four slots per thread), which bounds the
    // rows a slot may see: a term is at most 2^14, so 100000 of them stay below 2^31.
#ifndef RMI_COL_WIDE_BYTES
#define RMI_COL_WIDE_BYTES 1
#endif
    const bool byte_sums = RMI_COL_WIDE_BYTES != 0 && (key.family == kFamInt || key.family == kFamFloat) &&
                           es == 1 && key.red_op == RMI_RED_ADD;
    if (p.group == 0 && p.vec16 && lanes > kColMaxLanes &&
        (key.family == kFamFloat || key.family == kFamKbn || key.family == kFamKvp || byte_sums)) {
      int K = 256 / (p.step * (byte_sums ? 4 : acc_bytes));
      K     = K < 1 ? 1 : (K > kColWideMaxSets ? kColWideMaxSets : K);
      const int64_t slots = (int64_t)kPlanBlock * K;
      const int64_t cuts  = ceildiv(lanes, slots);
      if (cuts <= n_cu && (cuts == 1 || lanes % 64 != 0 || p.tail > 0)) {
        const int64_t piece  = ceildiv(lanes, cuts);
        const int64_t bundle = slots / piece;
        const int64_t step   = bundle * col_wide_bundles_of(K);
        const int64_t B      = (int64_t)n_cu / cuts;
        const size_t ws      = kTicketBytes + (size_t)p.n_out * B * acc_bytes;
        const bool too_large = (d.flags & kFlagSmallWorkspace) != 0 && ws > RMI_NOALLOC_SCRATCH_BYTES;
        // (byte sums have 1024 slots and no room to deal them finely: rows that use less than
        // three quarters of them, or that are whole multiples of 64 lane-loads, keep the layout
        // above: int8 D = 8200 / 16400 / 20000 lose 9-18 % here, 4096 / 8192 3-4 %, while D =
        // 2100 / 3000 / 4100 / 5000 / 50000 go from 60-70 % to 70-74 %)
        const bool bytes_ok = !byte_sums || (rows <= 100000 * B * bundle && bundle * piece * 4 >= slots * 3 &&
                                             (lanes % 64 != 0 || p.tail > 0));
        if (rows >= B * step * 16 && !too_large && bytes_ok) {
          p.wide        = K;
          p.TX          = (int)piece;
          p.TY          = (int)bundle;
          p.gridx       = ceildiv(lanes, piece);
          p.B           = (int)B;
          p.grid_blocks = p.gridx * p.B;
          p.passes      = 2;  // the epilogue is the second pass's
          p.ws_bytes    = ws;
          return RMI_OK;
        }
      }
    }
    // row tiles of TY*unroll rows are dealt round-robin to B blocks: kColBlocksPerCu
    // blocks per CU, but at least two tiles per block
    const int64_t tile_rows = (int64_t)p.TY * kPlanUnroll;
    // arg-reductions spend longer in their accumulate step: 3 workgroups per CU measured
    // 84 % where 2 give 78 % (sums lose a point or two at 3)
    const int per_cu = key.family == kFamKvp ? kColBlocksPerCu + 1 : kColBlocksPerCu;
    // (rounded down: one workgroup more than per_cu per CU lands on a CU that then finishes
    // last; 9 pieces x 57 = 513 workgroups ran 10 % slower than 9 x 56, 79 x 7 16 % slower
    // than 79 x 6)
    int64_t B               = ((int64_t)n_cu * per_cu) / p.gridx;
    const int64_t maxB      = ceildiv(rows, tile_rows * 2);
    if (B > maxB) B = maxB;
    if (B < 1) B = 1;
    if (B > 4096) B = 4096;
    p.B = (int)B;
    p.grid_blocks         = p.gridx * p.B;
    const int64_t fold_b  = p.group > 0 ? (int64_t)p.B * p.group : p.B;
    p.passes              = fold_b > 1 ? 2 : 1;
    p.ws_bytes            = fold_b > 1 ? kTicketBytes + (size_t)p.n_out * fold_b * acc_bytes : 0;
    if (p.gridx > 0x7fffffffLL) return RMI_ERR_BAD_SHAPE;
    return RMI_OK;
  }

  // ---- contiguous-dimension plans ----
  // several whole rows per 16-byte vector
  // (Left to itself the planner takes this plan for two rows per vector, for outputs narrower
  // than 32 bits, which it packs, and for inputs off a 16-byte boundary: with four rows and
  // more per vector the rows through LDS of the ROW_WAVE branch measured faster, a lane's K
  // outputs being K separate stores here: int8 -> int64 D = 1 / 2 / 4: 6 / 10 / 59 -> 64 / 64 / 68 % of
  // 8 TB/s, int8 -> int32 D = 1 / 2 / 4: 14 / 30 / 60 -> 63 / 70 / 82, bf16 -> fp32 D = 1 / 2: 66 / 76 ->
  // 70 / 82, fp32 D = 1: 77 -> 82; bf16 -> bf16 D = 2: 67 here, 55 there.  Two rows per vector
  // measured within a point on fp32 and bf16 and either way by 5 points with the matrix's size
  // on int8 -> int64 D = 8: 8M / 17M / 34M / 67M rows 75 / 79 / 81 / 81 % here, 70 / 79 / 86 / 76 there.)
  const bool lanes_auto = RMI_LANES_AUTO != 0 || 16 / row_bytes <= 2 || dtype_size(d.out_dtype) < 4 ||
                          (in_misalign % 16) != 0;
  if (row_bytes < 16 && 16 % row_bytes == 0 &&
      ((hint == RMI_PLAN_AUTO && lanes_auto) || hint == RMI_PLAN_ROW_LANES)) {
    p.kind        = RMI_PLAN_ROW_LANES;
    p.vec16       = true;
    p.step        = 16 / es;
    p.K           = (int)(16 / row_bytes);
    p.nvec        = 1;
    p.tail        = 0;
    // Integer sums whose lane writes as many bytes as it reads (two 8-byte rows into two
    // int64): one load per lane, like the fastest streaming copy (16.7M rows of 8 int8:
    // 44.6 -> 43.4 us); every other shape measured best, or within 1 %, at four.
    if (key.family == kFamInt && p.K == 2 && dtype_size(d.out_dtype) == 8) p.lanes_loads = 1;
    p.grid_blocks = ceildiv(ceildiv(p.n_out, p.K), (int64_t)kPlanBlock * p.lanes_loads);
    if (p.grid_blocks < 1) p.grid_blocks = 1;
    if (p.grid_blocks > 0x7fffffffLL) return RMI_ERR_BAD_SHAPE;
    return RMI_OK;
  }

  int kind = hint;
  if (kind == RMI_PLAN_ROW_LANES || kind == RMI_PLAN_COL_TILE || kind == RMI_PLAN_EMPTY)
    kind = RMI_PLAN_AUTO;
  int threads = 64;
  const int64_t split_piece = key.family == kFamMeanVar ? 2 * kSplitPieceVecs : kSplitPieceVecs;
  // (byte rows of less than 8 KB lose with it: up to three single loads on one thread of a
  // one-wave team, int8 D = 4097 58 -> 53 %, while D = 16385 gains 17 %)
  const bool head_skip      = RMI_HEAD_SKIP != 0 && p.vec16 && es < 4 && key.family != kFamKvp &&
                         ((row_bytes % 4) != 0 || (in_misalign % 4) != 0) && (es == 2 || p.nvec >= 512);
  if (kind == RMI_PLAN_AUTO) {
    if (nload <= 4 * 64) {
      kind = RMI_PLAN_ROW_WAVE;
    } else {
      // widen the team on a row until the machine's wave slots are filled, as long
      // as every thread keeps kTeamMinLoads lane-loads
      while (threads < 1024 && p.n_out * (threads / 64) < slots &&
             p.nvec >= (int64_t)kTeamMinLoads * threads)
        threads *= 2;
      // Long rows: a team wide enough that a thread sees two to four batches (sums) or
      // four to eight (arg-reductions, whose accumulate step is longer).  One wave
      // streaming a long row alone leaves thousands of row streams open at once, which
      // measured 3-7 points slower than 128- or 256-thread teams.
      // Sums over rows of up to 2304 lane-loads take the narrowest team that reads the row in
      // ONE trip of at most nine loads per thread (fp32 D = 1025 / 1100 / 2049: 45 / 50 / 67 % with
      // whole batches of four first and the rest in further trips).
      {
        const bool kvp     = key.family == kFamKvp;
        const int64_t want = p.nvec / (kvp ? 16 : 8);
        int wide           = kvp ? 64 : 128;
        while (wide < 256 && wide * 2 <= want)
          wide *= 2;
        if (!kvp && RMI_TEAM_ONE_TRIP != 0) {
          int narrow = 64;
          while (narrow < 256 && nload > (int64_t)(2 * kPlanTeamUnroll + 1) * narrow)
            narrow *= 2;
          // (where such teams fill the machine's wave slots; fewer rows keep the wider teams)
          if (p.n_out * (narrow / 64) >= slots) wide = narrow;
        }
        if (wide > threads) threads = wide;
      }
      if (threads == 1024 && p.n_out * 16 < slots &&
          p.nvec >= (int64_t)kTeamMinLoads * kPlanBlock) {
        kind = RMI_PLAN_ROW_SPLIT;
      } else {
        kind = RMI_PLAN_ROW_BLOCK;
        if (RMI_SPLIT_FINE != 0 && threads >= 512) {
          const int rule = tail_round_rule(p.n_out, slots / (threads / 64), p.nvec, split_piece);
          if (rule == kTailSplit) kind = RMI_PLAN_ROW_SPLIT;
          if (rule == kTailNarrow) threads /= 2;
        }
      }
    }
  } else if (kind == RMI_PLAN_ROW_BLOCK) {
    threads = kPlanBlock;
  } else if (kind == RMI_PLAN_ROW_WAVE && nload > 4 * 64) {
    kind = RMI_PLAN_ROW_BLOCK;  // one wave per row, served by the team kernel
  }

  if (kind == RMI_PLAN_ROW_WAVE) {
    p.kind = RMI_PLAN_ROW_WAVE;
    // Rows through LDS (row_small_kernel): a workgroup reads a chunk of whole rows as aligned
    // vectors into LDS and its threads reduce whole rows from there, element by element.
    // Rows shorter than a vector that do not divide one (the others are ROW_LANES) would be read
    // a lane per element: fp32 D = 3 34 -> 82 % of 8 TB/s, arg-max 39 -> 84, bf16 D = 3 / 5 / 7:
    // 23 / 17 / 22 -> 74 / 82 / 82, int8 D = 3 ... 15: 16-26 -> 73-84.  Longer rows that are no whole
    // vectors, as long as a chunk holds 32 of them: 16-bit elements (their lane-loads sit 2 bytes
    // off whole words: bf16 D = 9 / 17 / 33 / 65 / 97 / 161: 46 / 43 / 58 / 63 / 68 / 69 -> 79 / 75 / 75 /
    // 78 / 80 / 76, D = 193 / 225: 62 / 65 -> 61 / 68; 42-45 % from 514 bytes on) and 8-byte ones
    // (compensated sums pay most for the steps between lanes: fp64 D = 3 / 5 / 9 / 17 / 33 / 49 / 63:
    // 75 / 56 / 67 / 71 / 75 / 65 / 73 -> 80 / 76 / 76 / 77 / 81 / 77 / 82, D = 65: 76 -> 64); 4-byte rows
    // up to 40 bytes (fp32 D = 6 / 9: 71 / 67 -> 78 / 75, D = 5 / 7 / 10 within 2 points; D = 11 / 13 /
    // 25 lose 3 / 8 / 7).  Byte rows of 17 to 96 bytes keep the flat kernel (int8 D = 33 / 63: 68 /
    // 67 % there, 61 / 58 % here).
    const int64_t small_max = es == 1 ? 15 : es == 4 ? 40 : (es == 2 || es == 8) ? 512 : 15;
    if (RMI_SMALL_ROWS != 0 && row_bytes <= small_max && (row_bytes % 16) != 0 &&
        (in_misalign % 16) == 0 && hint == RMI_PLAN_AUTO &&
        kPlanSmallBytes / row_bytes >= 32) {
      p.small_rows  = true;
      p.vec16       = true;  // the chunk is read as whole vectors
      p.G           = 1;
      p.logG        = 0;
      p.chunk_rows  = (int)(kPlanSmallBytes / row_bytes / 16 * 16);
      p.grid_blocks = ceildiv(p.n_out, (int64_t)p.chunk_rows);
      if (p.grid_blocks > 0x7fffffffLL) return RMI_ERR_BAD_SHAPE;
      return RMI_OK;
    }
    // An input that starts off a 16-byte boundary makes every 128-byte piece of the default
    // layout (8 or 16 lanes per row, several loads per lane) straddle two lines, and each
    // line is then asked for by two load instructions.  With one load per lane and the
    // rows of a wave side by side, a load instruction reads ONE contiguous span and a line
    // is asked for once (plus one per instruction).  Measured on fp32 sums at +4 and +8
    // bytes: 1M x 128 80 -> 74 us (81 -> 87 %), 1M x 100 74 -> 67 us, 1M x 64 43 -> 38 us,
    // 2M x 48 82 -> 64 us.  Not for rows beyond 32 lane-loads (1M x 256: 141 -> 160 us), rows
    // that leave more than a quarter of the lanes idle or end in tail elements (1M x 66:
    // 50 -> 62 us), arg-reductions (85 -> 92 us) or 1- and 2-byte elements (no change).
    const bool side_by_side = (in_misalign % 16) != 0 && es == 4 && key.family != kFamKvp &&
                              p.vec16 && p.tail == 0 && nload <= 32 &&
                              nload * 4 >= (int64_t)pow2ceil(nload) * 3 &&
                              (hint == RMI_PLAN_AUTO || hint == RMI_PLAN_ROW_WAVE);
    if (nload <= 8 || side_by_side) {
      p.short_rows = true;
      p.G          = pow2ceil(nload);  // lane c == nvec loads the overlapping last vector
    } else {
      const int64_t g = ceildiv(nload, kPlanUnroll);
      p.G             = g >= 64 ? 64 : pow2ceil(g);
      // At least 8 lanes (128 contiguous bytes per row and load instruction), except for
      // rows of 9 to 15 whole vectors: 4 lanes with up to 4 loads each keep twice the rows
      // of a wave in flight (1M x 36..60 floats: 55-73 % -> 78-83 %; with tail elements, or
      // at 16 vectors, 8 lanes measured better).
      if (p.G < 8 && !(p.tail == 0 && nload < 16)) p.G = 8;
    }
    // Lane-load counts that are not close to a power of two (times 1..4 loads per lane)
    // leave lanes without work: 9 lane-loads on 8 lanes x 2 loads use 9 slots of 16, and a
    // row cut over two load instructions is fetched as two pieces.  The one-load-per-lane
    // kernel also runs with G = the lane-load count itself, 64 / G whole rows per wave step
    // (one contiguous span per load instruction).  Its cross-lane steps cost more, so the
    // rule follows what was measured on 1M-row fp32 matrices: 5 lane-loads, and 6 or 9 to 16
    // when the row ends in tail elements (D = 20 / 21 / 33 / 41 / 45 / 54 / 62: 69 / 66 / 52 /
    // 59 / 62 / 69 / 72 % -> 78 / 77 / 74 / 70 / 75 / 79 / 80 %), and 18 to 32 with a tail where
    // the groups fill at least 54 lanes (D = 79 / 83 / 125: 69 / 71 / 72 % -> 77 / 79 / 80 %; at
    // 23 lane-loads, 46 lanes, it lost 13 points).  At 7 lane-loads with a tail, or at 6, 7,
    // 19, 21 without one, it measured 2 to 10 points slower.
    // Accumulators of 16 bytes and more (f64 sums, 64-bit keys or values) pay twice as much
    // per cross-lane step: they keep the variant up to 12 lane-loads only (f64 D = 9 / 17: 48 ->
    // 61 / 57 %; D = 25 / 33 / 63 lost 12 to 21 points with it).
    const int64_t any_g_max = acc_bytes > 8 ? 12 : 32;
    if (p.vec16 && nload <= any_g_max &&
        (nload == 5 || (p.tail > 0 && (nload == 6 || (nload >= 9 && nload <= 16) ||
                                       (nload >= 18 && nload <= 32 && (64 / nload) * nload >= 54)))) &&
        (hint == RMI_PLAN_AUTO || hint == RMI_PLAN_ROW_WAVE)) {
      p.short_rows = true;
      p.any_g      = true;
      p.G          = (int)nload;
    }
    // Some lane-load counts suit neither layout: 17 fill 17 of 32 lanes, or 51 of 64 as three
    // whole rows per wave.  There a workgroup's load slots are dealt densely over whole adjacent
    // rows, one lane-load each, and the rows are combined through LDS (row_dense_kernel).  It
    // costs a pass through LDS and two barriers per step, so the rule is what was measured on
    // 512 MB matrices (% of 8 TB/s, before -> dense): rows ending in tail elements with 17 or 18
    // lane-loads (fp32 D = 65 / 66 / 67 / 69: 65 / 64 / 67 / 72 -> 76 / 76 / 75 / 77, bf16 D = 130:
    // 65 -> 75, int8 D = 270: 58 -> 63, arg-max D = 66: 61 -> 73), with 33 (fp32 D = 129: 76 -> 79,
    // bf16 D = 260: 73 -> 78, f64 D = 65: 68 -> 73; not arg-reductions: 69 -> 63), 16-bit rows of 9
    // to 16 (bf16 D = 66 / 100: 64 / 63 -> 70 / 72) and compensated f64 sums of 5 to 18 or 34 (D =
    // 9 / 17 / 25 / 33 / 35 / 67: 53 / 52 / 59 / 60 / 62 / 70 -> 60 / 67 / 68 / 71 / 72 / 74).  Everywhere
    // else it measured 1 to 30 % slower than the layouts above (fp32 D = 100: 88 -> 78 %).
    const bool dense_ok =
      p.vec16 && p.tail > 0 && hint == RMI_PLAN_AUTO &&
      (nload == 17 || nload == 18 || (nload == 33 && key.family != kFamKvp) ||
       (key.family == kFamFloat && es == 2 && nload >= 9 && nload <= 16) ||
       (key.family == kFamKbn && ((nload >= 5 && nload <= 18) || nload == 34)));
    if (dense_ok) {
      p.dense_rows = true;
      p.short_rows = false;
      p.any_g      = false;
      p.G          = (int)nload;
    }
    // The flat kernel (row_flat_kernel): aligned 16-byte vectors whatever the row length.  It
    // is bound by its index arithmetic and its pass through LDS at about 60 % of 8 TB/s for 2-
    // to 8-byte elements (the lane-group plans read the same shapes at 70-88 %) and at 66-71 %
    // for byte rows, so it serves byte sums only, and there the rows that are no whole 32-bit
    // words, where the lane-group plans fall to 44-67 % (int8 D = 17 / 33 / 47 / 50 / 65 / 70 / 85:
    // 49 / 44 / 55 / 56 / 58 / 60 / 59 % -> 71 / 71 / 67 / 67 / 68 / 70 / 65 %; rows of whole words keep
    // their 75-80 %, and from 100 bytes on the lane groups win again).
    {
      bool flat_ok = p.vec16 && es == 1 && (key.family == kFamInt || key.family == kFamFloat) &&
                     key.red_op == RMI_RED_ADD && (row_bytes % 4) != 0 && row_bytes <= 96 &&
                     (in_misalign % 16) == 0 && acc_bytes <= 16 && hint == RMI_PLAN_AUTO;
      if (flat_ok) {
        int g = 16, r = (int)(row_bytes % 16);
        while (r != 0) {  // gcd(16, row_bytes)
          const int q = g % r;
          g = r, r = q;
        }
        const int m0   = 16 / g;  // rows after which a row starts on a 16-byte boundary again
        int chunk_rows = (int)((int64_t)kPlanFlatMaxVec * 16 / row_bytes / m0 * m0);
        // a chunk that fills less than 85 % of the workgroup's vector slots leaves too many idle
        if (chunk_rows <= 0 || (int64_t)chunk_rows * row_bytes * 100 < (int64_t)kPlanFlatChunkVec * 16 * 85)
          flat_ok = false;
        if (flat_ok) {
          int g128 = 128, r128 = (int)(row_bytes % 128);
          while (r128 != 0) {
            const int q = g128 % r128;
            g128 = r128, r128 = q;
          }
          const int m128         = 128 / g128;  // chunks of whole lines where they fill well enough
          const int aligned_rows = (int)((int64_t)kPlanFlatMaxVec * 16 / row_bytes / m128 * m128);
          if (aligned_rows > 0 && (int64_t)aligned_rows * row_bytes * 100 >= (int64_t)kPlanFlatChunkVec * 16 * 90)
            chunk_rows = aligned_rows;
          int L = 1, logL = 0;
          while (2 * L <= 64 && 2 * L * chunk_rows <= kPlanBlock && L <= nload) L *= 2, ++logL;
          p.flat_rows   = true;
          p.short_rows  = false;
          p.any_g       = false;
          p.dense_rows  = false;
          p.chunk_rows  = chunk_rows;
          p.G           = L;
          p.logG        = logL;
          p.grid_blocks = ceildiv(p.n_out, (int64_t)chunk_rows);
          if (p.grid_blocks > 0x7fffffffLL) return RMI_ERR_BAD_SHAPE;
          return RMI_OK;
        }
      }
    }
    p.logG               = (p.any_g || p.dense_rows) ? 0 : ilog2(p.G);
    const int64_t rows_w = p.dense_rows ? 1 : (int64_t)(64 / p.G) * (p.short_rows ? kPlanUnroll : 1);
    p.grid_blocks        = ceildiv(p.n_out, rows_w * (kPlanBlock / 64));
    if (p.dense_rows) {
      const int64_t step = (int64_t)kPlanDenseBundles * ((kPlanBlock * kPlanDenseSlots) / p.G);
      p.grid_blocks      = ceildiv(p.n_out, step);
      if (p.grid_blocks > (int64_t)4 * n_cu) p.grid_blocks = (int64_t)4 * n_cu;
      return RMI_OK;
    }
    if (!p.short_rows && p.vec16) {
      // Bytes in flight per CU are what the memory system is sensitive to: about
      // 80 KB sustains the most (5 workgroups when 256 lanes hold 4 loads of 16 B); the
      // default 8 resident workgroups lose 3-4 points to queueing.  A dynamic LDS
      // reservation caps the resident workgroups: as many as bring the bytes in flight
      // closest to 80 KB, at least 4.  Arg-reductions, whose accumulate step is longer,
      // want more waves to hide behind: at least 7 (86 % where 5 give 77 %).
      const int64_t wg_bytes = (int64_t)(kPlanBlock / p.G) * nload * 16;
      int64_t cap            = (kBytesInFlightPerCu + wg_bytes / 2) / wg_bytes;
      if (key.family == kFamKvp && cap < 7) cap = 7;
      if (cap < 4) cap = 4;
      p.lds_reserve = cap >= 8 ? 0 : kLdsPerCu / (int)cap - 768;
      // Rows whose length is a multiple of 16 bytes but not of a 128-byte line, or that
      // start off a line: every 128- or 256-byte piece a lane group reads straddles
      // lines, and the L1 sends a request per line and instruction (twice the requests
      // to L2, a third more misses).  Such rows are staged: the wave reads its rows as
      // one line-aligned contiguous span into LDS and the lane groups read from there.
      // (a wave's rows have to fill at least half of its staging area: below that the
      // fixed five loads and stores per lane cost more than the lines saved)
      p.stage_ok = p.tail == 0 && (row_bytes % 16) == 0 && (64 / p.G) * row_bytes >= 2048;
      if (p.stage_ok && ((row_bytes % 128) != 0 || (in_misalign % 128) != 0) &&
          (in_misalign % 16) == 0) {
        p.staged = true;
        if (p.lds_reserve < kStageBytesPerWave * (kPlanBlock / 64))
          p.lds_reserve = kStageBytesPerWave * (kPlanBlock / 64);
      }
    }
  } else if (kind == RMI_PLAN_ROW_BLOCK) {
    // a team of `threads` threads per row; a 256-thread workgroup holds several
    // teams when a team is smaller.  One wave per row is reported as ROW_WAVE.
    p.kind        = threads == 64 ? RMI_PLAN_ROW_WAVE : RMI_PLAN_ROW_BLOCK;
    p.team_kernel = true;
    p.G           = 64;
    p.logG        = 6;
    p.threads     = threads;
    p.B           = 1;
    p.chunk       = p.nvec;
    // 16-byte loads from addresses that are no multiples of four run at two thirds of the
    // rate of the others (bf16 rows of odd length, every second of which starts 2 bytes off:
    // D = 10531 ... 68709 56-63 % of 8 TB/s, even lengths 72-74 %)
    p.head_skip = head_skip;
    const int teams = threads >= kPlanBlock ? 1 : kPlanBlock / threads;
    p.grid_blocks   = ceildiv(p.n_out, teams);
    if (threads <= kPlanBlock && p.vec16 && p.grid_blocks > (int64_t)8 * n_cu) {
      // More workgroups than fit at once: the resident 256-thread workgroups per CU are
      // capped by a dynamic LDS reservation the kernel never touches.  4 keep 64-128 KB
      // in flight per CU, which measured best for rows of several batches per thread; 3
      // gain another 3 points for sums over rows of 128 KB and more (eight or more
      // batches per thread) and lose 20 on arg-reductions.  Rows read in one trip of at most
      // seven loads per thread have less in flight per workgroup and no second batch to
      // overlap their arithmetic with: 6 (as many as their registers allow) gain 7-10 points
      // (fp32 D = 1100 76 -> 85 % of 8 TB/s, fp64 D = 600 73 -> 81, bf16 D = 4786 / 10530 72 / 75
      // -> 81 / 85, int8 D = 20000 78 -> 84, arg-max D = 1100 75 -> 85), with eight or nine loads
      // per thread they lose 2.
      const bool deep = threads == kPlanBlock && key.family != kFamKvp &&
                        p.nvec >= (int64_t)8 * kPlanTeamUnroll * kPlanBlock;
      const bool one_trip = nload <= (int64_t)RMI_TEAM_OT_LOADS * threads;
      p.lds_reserve       = kLdsPerCu / (deep ? 3 : one_trip ? RMI_TEAM_WG_ONE_TRIP : 4) - 768;
    }
  } else {
    p.kind        = RMI_PLAN_ROW_SPLIT;
    p.team_kernel = true;
    p.threads     = kPlanBlock;
    p.head_skip   = head_skip;
    const int64_t quantum = (int64_t)kPlanBlock * 8;
    int64_t B             = ceildiv(slots, p.n_out * (kPlanBlock / 64));
    const int64_t maxB    = p.nvec / quantum > 1 ? p.nvec / quantum : 1;
    if (B > maxB) B = maxB;
    if (RMI_SPLIT_FINE != 0) {
      // More pieces than the wave slots ask for: the workgroups of the last round, which run
      // with the machine partly empty, are shorter (1 GB of fp32, 200 / 400 / 500 rows: 80 / 80 /
      // 79 -> 83 / 84 / 82 % of 8 TB/s).
      int64_t fine = p.nvec / split_piece;
      if (fine > kSplitMaxPieces) fine = kSplitMaxPieces;
      const bool fits = (d.flags & kFlagSmallWorkspace) == 0 ||
                        kTicketBytes + (size_t)(p.n_out * fine) * acc_bytes <= RMI_NOALLOC_SCRATCH_BYTES;
      if (fine > B && fits) B = fine;
    }
    if (B < 2) B = 2;
    if (B > 4096) B = 4096;
    p.chunk       = ceildiv(ceildiv(p.nvec, B), quantum) * quantum;
    p.B           = (int)ceildiv(p.nvec, p.chunk);
    p.grid_blocks = p.n_out * p.B;
    if (p.B < 2) {  // the row is too short to split: one block per row
      p.kind  = RMI_PLAN_ROW_BLOCK;
      p.B     = 1;
      p.chunk = p.nvec;
    } else {
      // more pieces than fit at once: four resident workgroups per CU, as for whole rows of
      // several batches per thread (1 GB of fp32, 500 / 525 / 1800 rows: 82 / 84 / 83 -> 85 / 86 / 86 %)
      if (RMI_SPLIT_WG < 8 && p.grid_blocks > (int64_t)8 * n_cu) p.lds_reserve = kLdsPerCu / RMI_SPLIT_WG - 768;
      p.ws_bytes   = kTicketBytes + (size_t)p.n_out * p.B * acc_bytes;
      p.fused_fold = (d.flags & RMI_FLAG_WORKSPACE_ZEROED) != 0 &&
                     p.n_out * ticket_lines_per_row(p.B) <= kTicketLines;
      p.passes     = p.fused_fold ? 1 : 2;
    }
  }
  if (p.grid_blocks > 0x7fffffffLL) return RMI_ERR_BAD_SHAPE;
  return RMI_OK;
}

inline void export_plan(const PlanX& p, rmi_plan& o)
{
  o.kind            = p.kind;
  o.vec_bytes       = p.vec16 ? 16 : p.elem_bytes;
  o.lanes_per_row   = p.kind == RMI_PLAN_ROW_WAVE ? p.G : 0;
  o.blocks_per_out  = p.group > 0 ? p.B * p.group : p.B;
  o.block_threads   = (p.team_kernel && p.threads > kPlanBlock) ? p.threads : kPlanBlock;
  o.passes          = p.passes;
  o.grid_blocks     = p.grid_blocks;
  o.n_outputs       = p.n_out;
  o.reduce_len      = p.len;
  o.workspace_bytes = p.ws_bytes;
}

}  // namespace rmi
