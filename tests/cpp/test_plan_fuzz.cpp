// Host-only property test of the launch-plan selector (raft_amd/csrc/rmi_plan.hpp), built
// with -fsanitize=address,undefined: random and extreme shapes, every dtype and hint, and the
// invariants the kernels and the host checks rely on (coverage of the row by the chunks,
// lane groups that hold the whole row, grid and workspace sizes, LDS reservations).
#include <cstdio>
#include <cstdlib>
#include <random>

#include "../../raft_amd/csrc/rmi_plan.hpp"

namespace {
int failures = 0;
long planned[8] = {0, 0, 0, 0, 0, 0, 0, 0};
long staged_plans = 0;
long grouped_plans = 0;
long wide_plans = 0;
long dense_plans = 0;
long flat_plans = 0;
long small_plans = 0;
long wide_team_plans = 0;
long tail_split_plans = 0;
#define REQUIRE(cond)                                                              \
  do {                                                                             \
    if (!(cond)) {                                                                 \
      if (++failures < 20)                                                         \
        std::printf("  %s:%d: %s  [dtype %d layout %d apply %d rows %lld cols %lld hint %d]\n", \
                    __FILE__, __LINE__, #cond, d.in_dtype, d.layout, d.apply,      \
                    (long long)d.n_rows, (long long)d.n_cols, d.plan_hint);        \
    }                                                                              \
  } while (0)

void check(const rmi_reduce_desc& d, int n_cu, uintptr_t in_misalign)
{
  using namespace rmi;
  PolicyKey key;
  int acc_bytes = 0;
  const int rc  = classify(d, key, acc_bytes);
  if (rc != RMI_OK) return;
  PlanX p;
  const int prc = make_plan(d, key, acc_bytes, n_cu, p, in_misalign);
  if (prc != RMI_OK) {
    REQUIRE(prc == RMI_ERR_BAD_SHAPE);
    return;
  }
  ++planned[p.kind];
  const bool row_major  = d.layout == RMI_ROW_MAJOR;
  const bool along_rows = d.apply == RMI_ALONG_ROWS;
  const int64_t contiguous = row_major ? d.n_cols : d.n_rows;
  const int64_t other      = row_major ? d.n_rows : d.n_cols;
  REQUIRE(p.strided == (row_major != along_rows));
  REQUIRE(p.n_out == (p.strided ? contiguous : other));
  REQUIRE(p.len == (p.strided ? other : contiguous));
  if (p.n_out == 0) {
    REQUIRE(p.kind == RMI_PLAN_EMPTY && p.passes == 0);
    return;
  }
  if (p.len == 0) {
    REQUIRE(p.kind == RMI_PLAN_EMPTY && p.grid_blocks >= 1);
    return;
  }
  REQUIRE(p.grid_blocks >= 1 && p.grid_blocks <= 0x7fffffffLL);
  REQUIRE(p.lds_reserve >= 0 && p.lds_reserve <= 64 * 1024);
  // partials behind the workspace's ticket words; a second launch folds them unless the
  // caller vouches for zeroed tickets and the plan splits rows (at most one ticket per row)
  REQUIRE((p.ws_bytes > 0) == (p.passes == 2 || p.fused_fold));
  REQUIRE(p.B >= 1 && p.B <= 4096);
  if (p.ws_bytes > 0)
    REQUIRE(p.ws_bytes == rmi::kTicketBytes +
                            (size_t)p.n_out * p.B * (p.group > 0 ? p.group : 1) * acc_bytes);
  REQUIRE(p.fused_fold == ((d.flags & RMI_FLAG_WORKSPACE_ZEROED) != 0 &&
                           p.kind == RMI_PLAN_ROW_SPLIT &&
                           p.n_out * rmi::ticket_lines_per_row(p.B) <= rmi::kTicketLines));
  if (p.fused_fold) REQUIRE(p.passes == 1 && p.threads == rmi::kPlanBlock);
  const int es = dtype_size(d.in_dtype);
  if (p.kind != RMI_PLAN_ROW_LANES) {
    REQUIRE(p.row_bytes == contiguous * es);
    REQUIRE(p.vec16 == (p.row_bytes >= 16 || p.group > 0 || p.small_rows));
    REQUIRE(p.nvec * p.step + p.tail == contiguous);
    REQUIRE(p.tail >= 0 && p.tail < p.step);
  }
  const int64_t nload = p.nvec + (p.tail > 0 ? 1 : 0);
  switch (p.kind) {
    case RMI_PLAN_ROW_LANES:
      REQUIRE(!p.strided && p.K >= 2 && p.K <= 16 && p.K * contiguous * es == 16);
      // asked for by name, two rows per vector, outputs narrower than 32 bits, or an input off a
      // 16-byte boundary
      REQUIRE(d.plan_hint == RMI_PLAN_ROW_LANES || p.K == 2 || dtype_size(d.out_dtype) < 4 ||
              in_misalign % 16 != 0);
      break;
    case RMI_PLAN_ROW_WAVE:
      REQUIRE(!p.strided);
      if (p.team_kernel) {
        REQUIRE(p.threads == 64 && p.B == 1 && p.chunk == p.nvec);
      } else if (p.small_rows) {
        ++small_plans;
        // rows through LDS: a chunk of whole rows per workgroup, at most 16 KB
        REQUIRE(p.row_bytes <= (es == 1 ? 15 : es == 4 ? 40 : 512) && p.row_bytes % 16 != 0);
        // rows of which four or more fill a vector come here when their outputs have 32 bits or more
        if (16 % p.row_bytes == 0) REQUIRE(dtype_size(d.out_dtype) >= 4 && 16 / p.row_bytes >= 4);
        REQUIRE(in_misalign % 16 == 0 && d.plan_hint == RMI_PLAN_AUTO);
        REQUIRE(!p.short_rows && !p.any_g && !p.dense_rows && !p.flat_rows && p.passes == 1 && p.ws_bytes == 0);
        REQUIRE(p.chunk_rows >= 32 && p.chunk_rows % 16 == 0 &&
                (int64_t)p.chunk_rows * p.row_bytes <= rmi::kPlanSmallBytes);
        REQUIRE(p.grid_blocks == (p.n_out + p.chunk_rows - 1) / p.chunk_rows);
      } else if (p.flat_rows) {
        ++flat_plans;
        // byte sums over rows that are no whole words: chunks of whole rows that start on a
        // 16-byte boundary and fit the workgroup's vector slots, a power-of-two lane group per
        // row for the fold, one workgroup per chunk
        REQUIRE(p.vec16 && !p.short_rows && !p.any_g && !p.dense_rows && !p.staged);
        REQUIRE(p.elem_bytes == 1 && p.row_bytes % 4 != 0 && p.row_bytes >= 17 && p.row_bytes <= 96);
        REQUIRE(in_misalign % 16 == 0 && p.acc_bytes <= 16);
        REQUIRE(p.chunk_rows >= 1 && ((int64_t)p.chunk_rows * p.row_bytes) % 16 == 0);
        REQUIRE((int64_t)p.chunk_rows * p.row_bytes <= (int64_t)rmi::kPlanFlatMaxVec * 16);
        REQUIRE((int64_t)p.chunk_rows * p.row_bytes * 100 >= (int64_t)rmi::kPlanFlatChunkVec * 16 * 85);
        REQUIRE(p.G >= 1 && p.G <= 64 && (1 << p.logG) == p.G);
        REQUIRE(p.G == 1 || (int64_t)p.G * p.chunk_rows <= kPlanBlock);
        REQUIRE(p.grid_blocks * p.chunk_rows >= p.n_out && (p.grid_blocks - 1) * p.chunk_rows < p.n_out);
        REQUIRE(p.passes == 1 && p.ws_bytes == 0 && p.lds_reserve == 0);
      } else if (p.dense_rows) {
        ++dense_plans;
        // one lane-load per load slot, whole adjacent rows per workgroup, rows met in LDS
        const int64_t slots = (int64_t)kPlanBlock * rmi::kPlanDenseSlots;
        REQUIRE(p.vec16 && p.tail > 0 && !p.short_rows && !p.any_g && !p.staged && p.G == nload);
        REQUIRE(p.G >= 5 && p.G <= 34 && slots / p.G >= 1);
        REQUIRE((int64_t)rmi::kPlanDenseBundles * (slots / p.G) * p.G * p.acc_bytes <= 32768);
        REQUIRE(p.grid_blocks >= 1 && p.grid_blocks <= (int64_t)4 * n_cu);
        REQUIRE(p.grid_blocks * rmi::kPlanDenseBundles * (slots / p.G) >= p.n_out ||
                p.grid_blocks == (int64_t)4 * n_cu);
        REQUIRE(p.passes == 1 && p.ws_bytes == 0 && p.lds_reserve == 0);
      } else {
        if (p.any_g) {
          // one lane per lane-load, whole rows per wave, one run of at most 64 outputs
          REQUIRE(p.short_rows && p.vec16 && p.G == nload && p.G >= 4 && p.G <= 32);
          REQUIRE((64 / p.G) * p.G >= 48);  // at least three lanes in four have a lane-load
          if (p.G >= 18) REQUIRE((64 / p.G) * p.G >= 54 && p.tail > 0);
          REQUIRE((64 / p.G) * kPlanUnroll <= 64);
        } else {
          REQUIRE(p.G >= 1 && p.G <= 64 && (p.G & (p.G - 1)) == 0 && (1 << p.logG) == p.G);
        }
        // the lanes of a row hold all of its lane-loads, kPlanUnroll apiece (one for short rows)
        REQUIRE((int64_t)p.G * (p.short_rows ? 1 : kPlanUnroll) >= nload);
        if (p.staged) {
          ++staged_plans;
          // whole vectors at 16-byte aligned addresses; the wave's rows and the lead-in of a
          // line-aligned start fit its LDS area, which the launch reserves for four waves
          REQUIRE(p.stage_ok && !p.short_rows && p.vec16 && p.tail == 0);
          REQUIRE(p.row_bytes % 16 == 0 && in_misalign % 16 == 0);
          REQUIRE((64 / p.G) * p.row_bytes + 112 + 16 <= kStageBytesPerWave);
          REQUIRE(p.lds_reserve >= 4 * kStageBytesPerWave);
          REQUIRE(p.row_bytes % 128 != 0 || in_misalign % 128 != 0);
        }
      }
      break;
    case RMI_PLAN_ROW_BLOCK:
      REQUIRE(!p.strided && p.team_kernel && p.B == 1 && p.chunk == p.nvec);
      REQUIRE(p.threads >= 64 && p.threads <= 1024 && (p.threads & (p.threads - 1)) == 0);
      if (d.plan_hint == RMI_PLAN_AUTO && p.threads >= 512) {
        // wide teams either fit at once, fill their rounds, or leave a last round that is nine
        // tenths full on rows long enough to split (shorter rows get narrower teams)
        ++wide_team_plans;
        const int64_t cap  = (int64_t)n_cu * rmi::kWavesPerCu / (p.threads / 64);
        const int64_t last = p.n_out % cap;
        REQUIRE(p.n_out <= cap || last == 0 || (last * 10 >= cap * 9 && p.nvec / rmi::kSplitPieceVecs >= 4));
      }
      break;
    case RMI_PLAN_ROW_SPLIT:
      REQUIRE(!p.strided && p.team_kernel && p.B >= 2 && p.threads == kPlanBlock);
      REQUIRE(p.chunk > 0 && (int64_t)p.B * p.chunk >= p.nvec && (int64_t)(p.B - 1) * p.chunk < p.nvec);
      REQUIRE(p.grid_blocks == p.n_out * p.B);
      // rows split for their last round: pieces of 64 KB and more, at most 32 of them
      if (d.plan_hint == RMI_PLAN_AUTO && p.n_out * 16 >= (int64_t)n_cu * rmi::kWavesPerCu) {
        ++tail_split_plans;
        REQUIRE(p.B <= rmi::kSplitMaxPieces && p.chunk >= rmi::kSplitPieceVecs);
      }
      break;
    case RMI_PLAN_COL_TILE:
      REQUIRE(p.strided);
      if (p.wide > 0) {
        ++wide_plans;
        // whole rows (or the fewest equal pieces of them) per workgroup: the slots of its
        // threads hold TY adjacent rows of TX lane-loads, more than half of them in use, in at
        // most 64 KB of LDS at the end; no more workgroups than CUs
        const int64_t slots = (int64_t)kPlanBlock * p.wide;
        // byte sums gather in 32-bit slot accumulators: terms of at most 2^14, at most 100000
        // of them per slot, and rows that fill three quarters of the slots
        const bool byte_sums = p.elem_bytes == 1 && d.reduce_op == RMI_RED_ADD &&
                               (key.family == rmi::kFamInt || key.family == rmi::kFamFloat);
        const int slot_bytes = byte_sums ? 4 : p.acc_bytes;
        REQUIRE(p.wide >= 1 && p.wide <= rmi::kColWideMaxSets && p.wide * p.step * slot_bytes <= 256);
        REQUIRE(key.family == rmi::kFamFloat || key.family == rmi::kFamKbn || key.family == rmi::kFamKvp ||
                byte_sums);
        if (byte_sums) {
          REQUIRE(p.wide == 4 && (int64_t)p.TY * p.TX * 4 >= slots * 3);
          REQUIRE(p.len <= (int64_t)100000 * p.B * p.TY && (nload % 64 != 0 || p.tail > 0));
        }
        REQUIRE(p.group == 0 && p.vec16 && nload > rmi::kColMaxLanes && p.TX <= slots);
        REQUIRE(p.gridx >= 1 && p.gridx <= n_cu && p.gridx * p.TX >= nload && (p.gridx - 1) * p.TX < nload);
        REQUIRE(p.gridx == (nload + slots - 1) / slots);
        if (p.gridx > 1) REQUIRE(nload % 64 != 0 || p.tail > 0);
        REQUIRE(p.TY >= 1 && (int64_t)p.TY * p.TX <= slots && (int64_t)(p.TY + 1) * p.TX > slots);
        REQUIRE((int64_t)p.TY * p.TX * 2 > slots);
        REQUIRE((int64_t)p.TY * p.TX * p.step * slot_bytes <= 65536);
        REQUIRE(p.B == n_cu / p.gridx && p.B >= 1 && p.grid_blocks == p.B * p.gridx && p.grid_blocks <= n_cu);
        REQUIRE(p.passes == 2);
        REQUIRE(p.len >= (int64_t)p.B * p.TY * rmi::col_wide_bundles_of(p.wide) * 16);
        REQUIRE(p.ws_bytes == rmi::kTicketBytes + (size_t)p.n_out * p.B * p.acc_bytes);
        break;
      }
      REQUIRE(p.TX >= 1 && p.TX <= 128 && p.TY == kPlanBlock / p.TX && p.TY >= 2);
      REQUIRE(p.dense == ((p.TX & (p.TX - 1)) != 0 || p.TX > 64));
      if (!p.dense) REQUIRE((1 << p.logTX) == p.TX);
      REQUIRE(p.grid_blocks == p.gridx * p.B);
      {
        const int64_t lanes = p.group > 0 ? p.group_nvec : nload;
        REQUIRE(p.gridx * p.TX >= lanes && (p.gridx - 1) * p.TX < lanes);
        // at least three lanes in five carry data
        REQUIRE(lanes * p.TY * 5 >= p.gridx * kPlanBlock * 3 || lanes < 4);
      }
      if (p.group > 0) {
        ++grouped_plans;
        // rows shorter than a 16-byte vector, or longer ones 1 or 2 bytes off whole words whose
        // group fits a workgroup's lanes, in groups that are whole vectors at aligned
        // addresses, enough of them, no index-dependent reduction
        REQUIRE(key.family != rmi::kFamKvp && in_misalign % 16 == 0);
        REQUIRE(p.row_bytes < 16 || (p.row_bytes % 4 != 0 && p.row_bytes <= rmi::kGroupMaxRowBytes &&
                                     p.group_nvec <= rmi::kColMaxLanes));
        REQUIRE(p.group >= 2 && p.group <= 16 && (p.group * p.row_bytes) % 16 == 0);
        REQUIRE(p.group_nvec * 16 == p.group * p.row_bytes && (p.row_bytes >= 16 || p.group_nvec <= 15));
        REQUIRE(p.group_len == p.len / p.group && p.group_len >= rmi::kGroupMinLen);
        REQUIRE(p.passes == 2);
      }
      break;
    default: REQUIRE(false);
  }
  // rows read from their first whole 32-bit word on: team kernel, 1- and 2-byte elements, no
  // element indices
  if (p.head_skip)
    REQUIRE(p.team_kernel && p.vec16 && es < 4 && key.family != rmi::kFamKvp &&
            (p.row_bytes % 4 != 0 || in_misalign % 4 != 0) && (es == 2 || p.nvec >= 512));
  rmi_plan out{};
  export_plan(p, out);
  REQUIRE(out.n_outputs == p.n_out && out.reduce_len == p.len && out.workspace_bytes == p.ws_bytes);
}
}  // namespace

int main()
{
  std::mt19937_64 g(20240607);
  auto pick = [&](std::initializer_list<int64_t> v) {
    return *(v.begin() + (size_t)(g() % v.size()));
  };
  long cases = 0;
  for (int it = 0; it < 400000; ++it) {
    rmi_reduce_desc d{};
    d.in_dtype  = (int)(g() % 8);
    d.layout    = (int)(g() % 2);
    d.apply     = (int)(g() % 2);
    d.plan_hint = (int)(g() % 7);
    d.flags     = (int)(g() % 2) * RMI_FLAG_WORKSPACE_ZEROED;
    const int kind = (int)(g() % 4);
    if (kind == 0) {  // sums
      d.out_dtype = d.in_dtype >= RMI_F16 ? RMI_F32 : (g() % 2 ? RMI_I64 : RMI_F32);
      d.reduce_op = RMI_RED_ADD;
    } else if (kind == 1) {  // min / max
      d.out_dtype = d.in_dtype >= RMI_F16 ? RMI_F64 : RMI_I64;
      d.reduce_op = g() % 2 ? RMI_RED_MAX : RMI_RED_MIN;
    } else {  // arg reductions
      d.main_op   = RMI_MAIN_KVP;
      d.reduce_op = g() % 2 ? RMI_RED_ARGMAX : RMI_RED_ARGMIN;
      d.out_dtype = d.in_dtype == RMI_F64 ? (g() % 2 ? RMI_KVP_I32_F64 : RMI_KVP_I64_F64)
                                          : (g() % 2 ? RMI_KVP_I32_F32 : RMI_KVP_I64_F32);
    }
    // log-uniform extents with the edge values mixed in
    auto extent = [&]() -> int64_t {
      if (g() % 8 == 0) return pick({0, 1, 2, 3, 7, 9, 15, 16, 17, 25, 33, 35, 63, 64, 65, 66, 67, 69, 100, 129, 130, 255, 256, 257, 260, 270, 1023, 1024, 1025, 4095, 4096, 4097});
      const int bits = (int)(g() % 34);
      return (int64_t)(g() & ((1ull << bits) - 1)) + (g() % 2);
    };
    d.n_rows = extent();
    d.n_cols = extent();
    // keep the element count within what one GPU could hold (2^38), larger ones are
    // rejected or planned just the same but are not interesting
    if ((long double)d.n_rows * (long double)d.n_cols > 274877906944.0L) d.n_cols = d.n_cols % 4096;
    const uintptr_t mis = (uintptr_t)pick({0, 0, 0, 16, 32, 64, 112, 4, 8, 2, 1});
    for (int n_cu : {256, 1, 304})
      check(d, n_cu, mis);
    ++cases;
  }
  // byte rows of 17 to 100 elements, the shapes the flat row plan is chosen from
  for (int cols = 17; cols <= 100; ++cols)
    for (int dt : {RMI_I8, RMI_U8})
      for (int64_t rows : {(int64_t)1, (int64_t)15, (int64_t)16, (int64_t)1000, (int64_t)1 << 20, (int64_t)33554431})
        for (uintptr_t mis : {(uintptr_t)0, (uintptr_t)16, (uintptr_t)3}) {
          rmi_reduce_desc d{};
          d.in_dtype  = dt;
          d.out_dtype = rows % 2 ? RMI_I64 : RMI_F32;
          d.main_op   = cols % 3 == 0 ? RMI_MAIN_SQ : RMI_MAIN_IDENTITY;
          d.reduce_op = RMI_RED_ADD;
          d.n_rows    = rows;
          d.n_cols    = cols;
          check(d, 256, mis);
          ++cases;
        }
  // few long rows: every row count from 500 to 2100 at three row lengths
  for (int64_t rows = 500; rows <= 2100; ++rows)
    for (int64_t cols : {(int64_t)20000, (int64_t)70001, (int64_t)524288})
      for (int dt : {RMI_F32, RMI_BF16}) {
        rmi_reduce_desc d{};
        d.in_dtype  = dt;
        d.out_dtype = RMI_F32;
        d.reduce_op = RMI_RED_ADD;
        d.n_rows    = rows;
        d.n_cols    = cols;
        d.flags     = rows % 2 ? RMI_FLAG_WORKSPACE_ZEROED : 0;
        check(d, 256, rows % 3 == 0 ? 2 : 0);
        ++cases;
      }
  // the extremes the header promises to reject
  {
    rmi_reduce_desc d{};
    d.in_dtype = RMI_F32, d.out_dtype = RMI_F32;
    d.n_rows = ((int64_t)1 << 41), d.n_cols = 1;
    rmi::PolicyKey key;
    int acc = 0;
    rmi::PlanX p;
    if (rmi::classify(d, key, acc) == RMI_OK && rmi::make_plan(d, key, acc, 256, p) != RMI_ERR_BAD_SHAPE) {
      std::printf("  2^41 rows accepted\n");
      ++failures;
    }
  }
  std::printf("plans checked: lanes %ld wave %ld block %ld split %ld col %ld (whole rows %ld) empty %ld, dense rows %ld, flat rows %ld\n",
              planned[RMI_PLAN_ROW_LANES], planned[RMI_PLAN_ROW_WAVE], planned[RMI_PLAN_ROW_BLOCK],
              planned[RMI_PLAN_ROW_SPLIT], planned[RMI_PLAN_COL_TILE], wide_plans, planned[RMI_PLAN_EMPTY],
              dense_plans, flat_plans);
  for (int k = RMI_PLAN_ROW_LANES; k <= RMI_PLAN_EMPTY; ++k)
    if (planned[k] < 1000) {
      std::printf("  plan kind %d was hardly exercised\n", k);
      ++failures;
    }
  if (grouped_plans < 1000) {
    std::printf("  grouped column plans were hardly exercised (%ld)\n", grouped_plans);
    ++failures;
  }
  if (wide_plans < 1000) {
    std::printf("  whole-row column plans were hardly exercised (%ld)\n", wide_plans);
    ++failures;
  }
  if (wide_team_plans < 500 || tail_split_plans < 500) {
    std::printf("  plans of few long rows were hardly exercised (%ld wide teams, %ld splits)\n", wide_team_plans,
                tail_split_plans);
    ++failures;
  }
  if (small_plans < 1000) {
    std::printf("  plans of rows through LDS were hardly exercised (%ld)\n", small_plans);
    ++failures;
  }
  if (dense_plans < 500) {
    std::printf("  dense row plans were hardly exercised (%ld)\n", dense_plans);
    ++failures;
  }
  if (flat_plans < 1000) {
    std::printf("  flat row plans were hardly exercised (%ld)\n", flat_plans);
    ++failures;
  }
  if (staged_plans < 1000) {
    std::printf("  staged plans were hardly exercised (%ld)\n", staged_plans);
    ++failures;
  }
  std::printf("%ld descriptors, %d failed\n", cases, failures);
  return failures == 0 ? 0 : 1;
}
