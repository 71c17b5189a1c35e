// rmi_cov / rmi_cov_workspace_bytes (include/rmi_reduce.h): shape checks, the split of the
// work into column-block pairs and slabs of rows, and the launches.
#include "rmi_cov.hpp"

namespace rmi {
int cu_count();  // rmi_api.hip

namespace {

// Workgroups per CU when one pair of column blocks covers the matrix (D <= 64, the
// shape that is bound by HBM as much as by the matrix cores): the kernels hold more than
// 256 registers, so a CU holds one workgroup at a time and a second one per CU would only
// queue behind the first.  Otherwise the number of queued workgroups per CU (diagonal pairs
// issue 10 matrix instructions per wave-load, the others 16: small units even the CUs out).
#ifndef RMI_COV_WG_PER_CU
#define RMI_COV_WG_PER_CU 1
#endif
constexpr int kWgPerCuOnePair = RMI_COV_WG_PER_CU;
constexpr int kWgPerCuPairs   = 8;

struct CovPlan {
  int nb       = 0;
  int npairs   = 0;
  int S        = 1;
  int total    = 0;
  int grid     = 0;
  bool vec     = false;  // row-major: rows are whole quads of columns
  size_t ws_bytes = 0;
};

int make_cov_plan(int dtype, int layout, int64_t N, int64_t D, CovPlan& p)
{
  if (dtype != RMI_F32 && dtype != RMI_F64)
    return dtype >= 0 && dtype < RMI_DTYPE_COUNT_ ? RMI_ERR_UNSUPPORTED : RMI_ERR_BAD_ENUM;
  if (layout != RMI_ROW_MAJOR && layout != RMI_COL_MAJOR) return RMI_ERR_BAD_ENUM;
  if (N < 0 || D < 0) return RMI_ERR_BAD_SHAPE;
  const int64_t nb = (D + cov::kBlockCols - 1) / cov::kBlockCols;
  if (nb > 8192) return RMI_ERR_BAD_SHAPE;  // 512k columns: the result alone would be 1 TB
  p.nb     = (int)nb;
  p.npairs = (int)(nb * (nb + 1) / 2);
  p.vec    = D % 4 == 0;
  const int es          = dtype == RMI_F32 ? 4 : 8;
  const int step_rows   = dtype == RMI_F32 ? cov::kBf16UnitRows
                                           : (layout == RMI_ROW_MAJOR ? cov::kRowUnitRows : cov::kColUnitRows);
  const int64_t steps   = N / step_rows > 0 ? N / step_rows : 1;
  const int n_cu        = cu_count();
  int64_t S             = p.npairs <= 1 ? (int64_t)kWgPerCuOnePair * n_cu
                                        : ((int64_t)kWgPerCuPairs * n_cu) / p.npairs;
  // every wave gets eight units or more
  const int64_t maxS = (steps + 8 * cov::kWaves - 1) / (8 * cov::kWaves);
  if (S > maxS) S = maxS;
  if (S < 1) S = 1;
  p.S        = (int)S;
  p.total    = p.S * p.npairs;
  p.grid     = (p.total + 7) / 8 * 8;
  p.ws_bytes = (size_t)p.total * cov::kTilesPerPair * cov::kTile * es;
  return RMI_OK;
}

bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// Matrices of at most 32 columns are contracted as matrices of f D <= 64 columns and N / f rows:
// every load and every matrix instruction then does useful work, where a 64-column block with
// masked columns reads 20M x 32 floats at 55 % of the rate of 10M x 64 and 45M x 3 at 5 % (20M x
// 32: 572 -> 383 us, 40M x 16: 934 -> 386 us, fp64 10M x 32: 874 -> 525 us; 45M x 3: 1359 us as it
// was).  Row-major, f rows sit side by side; col-major, the first f pieces of N / f rows of every
// column; the N % f rows left over are added by cov_blocks_kernel.  It costs one more small
// launch, so matrices below 4M elements stay as they are (32768 x 32: 14 us against 17.6).
// Returns f, or 1.
int fold_factor(int layout, int64_t N, int64_t D)
{
  if (D < 1 || D > cov::kBlockCols / 2 || N * D < ((int64_t)1 << 22)) return 1;
  const int f0 = (int)(cov::kBlockCols / D);
  if (layout != RMI_ROW_MAJOR) return f0;
  // row-major: rows of whole quads of columns are read as vectors, which is worth up to a
  // quarter fewer rows side by side (45M x 3 as 21 rows of 63 columns: 156 us, as 20 of 60: see
  // the measurements)
  for (int f = f0; f >= 1 && f * 4 >= f0 * 3; --f)
    if ((f * D) % 4 == 0) return f;
  return f0;
}
constexpr size_t kWideBytes = (size_t)cov::kBlockCols * cov::kBlockCols * sizeof(double);

template <class T>
int launch(const CovPlan& pl, int layout, int64_t N_in, int64_t D_in, int sample, bool center, T* data,
           const T* mu, T* covar, void* ws, hipStream_t st)
{
  // `pl` is the plan of the matrix as it is contracted: N / f rows of 64 columns when folded
  const int fold  = fold_factor(layout, N_in, D_in);
  const int64_t N = N_in / fold, D = D_in * fold;
  cov::GramArgs g{};
  g.mu_div = layout == RMI_ROW_MAJOR ? 1 : fold;
  g.mu_mod = fold > 1 ? (int)D_in : 0;
  g.col_ld = N_in;
  g.col_f  = fold;
  g.data    = data;
  g.mu      = mu;
  g.partial = ws;
  g.N       = N;
  g.D       = D;
  g.nb      = pl.nb;
  g.npairs  = pl.npairs;
  g.S       = pl.S;
  g.total   = pl.total;
  bool write_back = center && mu != nullptr;
  if (write_back && pl.npairs > 1) {
    // several workgroups read every column block: centre first, then contract what is left
    const int64_t total = N * D;
    const int64_t lead  = layout == RMI_ROW_MAJOR ? D : N;
    int64_t blocks      = (total + cov::kThreads - 1) / cov::kThreads;
    const int64_t cap   = (int64_t)cu_count() * 16;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL((cov::center_kernel<T>), dim3((unsigned)blocks), dim3(cov::kThreads), 0, st,
                       data, mu, total, lead, layout == RMI_ROW_MAJOR ? 1 : 0);
    g.mu       = nullptr;
    write_back = false;
  }
  const dim3 grid((unsigned)pl.grid);
  const dim3 block(cov::kThreads);
  const bool one = pl.npairs == 1;
  // fp32, exactly one whole block of columns: the kernels without column masks
  constexpr bool kF32 = std::is_same_v<T, float>;
  const bool full     = kF32 && D == cov::kBlockCols;
  if (write_back) {  // one column block: the same pass leaves x - mu behind
    if (layout != RMI_ROW_MAJOR) {
      if (full)
        hipLaunchKernelGGL((cov::gram_cols_kernel<T, true, true, kF32>), grid, block, 0, st, g);
      else
        hipLaunchKernelGGL((cov::gram_cols_kernel<T, true, true>), grid, block, 0, st, g);
    } else if (full)
      hipLaunchKernelGGL((cov::gram_rows_kernel<T, true, true, true, kF32>), grid, block, 0, st, g);
    else if (pl.vec)
      hipLaunchKernelGGL((cov::gram_rows_kernel<T, true, true, true>), grid, block, 0, st, g);
    else
      hipLaunchKernelGGL((cov::gram_rows_kernel<T, false, true, true>), grid, block, 0, st, g);
  } else if (layout == RMI_ROW_MAJOR) {
    if (full)
      hipLaunchKernelGGL((cov::gram_rows_kernel<T, true, true, false, kF32>), grid, block, 0, st, g);
    else if (pl.vec && one)
      hipLaunchKernelGGL((cov::gram_rows_kernel<T, true, true>), grid, block, 0, st, g);
    else if (pl.vec)
      hipLaunchKernelGGL((cov::gram_rows_kernel<T, true, false>), grid, block, 0, st, g);
    else if (one)
      hipLaunchKernelGGL((cov::gram_rows_kernel<T, false, true>), grid, block, 0, st, g);
    else
      hipLaunchKernelGGL((cov::gram_rows_kernel<T, false, false>), grid, block, 0, st, g);
  } else if (full) {
    hipLaunchKernelGGL((cov::gram_cols_kernel<T, true, false, kF32>), grid, block, 0, st, g);
  } else if (one) {
    hipLaunchKernelGGL((cov::gram_cols_kernel<T, true>), grid, block, 0, st, g);
  } else {
    hipLaunchKernelGGL((cov::gram_cols_kernel<T, false>), grid, block, 0, st, g);
  }
  cov::FoldArgs f{};
  f.partial  = ws;
  f.out      = covar;
  f.D        = D;
  f.nb       = pl.nb;
  f.npairs   = pl.npairs;
  f.S        = pl.S;
  f.permuted = layout == RMI_ROW_MAJOR ? 1 : 0;
  // the reference's scalar: Type(1) / Type(N - 1 | N), handed to the GEMM in Type
  f.alpha = N_in == 0 ? 0.0 : (double)(T(1) / (sample ? T(N_in - 1) : T(N_in)));  // no rows: zeros, as a GEMM with k = 0
  // folded: the 64 x 64 sums go to the workspace behind the partials, then their diagonal blocks
  // are added up into the D x D result
  double* wide = fold > 1 ? reinterpret_cast<double*>(static_cast<char*>(ws) + pl.ws_bytes) : nullptr;
  f.wide       = wide;
  hipLaunchKernelGGL((cov::cov_fold_kernel<T>),
                     dim3((unsigned)(pl.npairs * cov::kTilesPerPair * (cov::kTile / cov::kFoldElems))),
                     dim3(cov::kFoldElems * cov::kFoldSplit), 0, st, f);
  if (fold > 1) {
    const int cells = (int)(D_in * D_in);
    // the rows that the contraction leaves over, still as they were given: the last N % fold
    // rows of the matrix (row-major) or of every column (col-major)
    const int left       = (int)(N_in - N * fold);
    const bool rm        = layout == RMI_ROW_MAJOR;
    T* tail              = rm ? data + N * fold * D_in : data + N * fold;
    const int64_t rs     = rm ? D_in : 1;
    const int64_t cs     = rm ? 1 : N_in;
    hipLaunchKernelGGL((cov::cov_blocks_kernel<T>), dim3((unsigned)((cells + cov::kThreads - 1) / cov::kThreads)),
                       dim3(cov::kThreads), 0, st, wide, covar, (int)D_in, fold, rm ? 1 : 0, tail, mu, left, rs,
                       cs, f.alpha);
    if (left > 0 && center && mu != nullptr)  // ... and centred like the others afterwards
      hipLaunchKernelGGL((cov::center_tail_kernel<T>), dim3(1), dim3(cov::kThreads), 0, st, tail, mu, left,
                         (int)D_in, rs, cs);
  }
  return hipGetLastError() == hipSuccess ? RMI_OK : RMI_ERR_LAUNCH;
}

}  // namespace
}  // namespace rmi

extern "C" {

size_t rmi_cov_workspace_bytes(int dtype, int layout, int64_t n_rows, int64_t n_cols)
{
  rmi::CovPlan pl;
  const int fold = rmi::fold_factor(layout, n_rows, n_cols);
  if (rmi::make_cov_plan(dtype, layout, n_rows / fold, n_cols * fold, pl) != RMI_OK) return 0;
  return n_cols > 0 ? pl.ws_bytes + (fold > 1 ? rmi::kWideBytes : 0) : 0;
}

int rmi_cov(int dtype,
            int layout,
            int64_t n_rows,
            int64_t n_cols,
            int sample,
            int flags,
            void* data,
            const void* mu,
            void* covar,
            void* workspace,
            size_t workspace_bytes,
            void* stream)
{
  using namespace rmi;
  if ((flags & ~RMI_COV_CENTER_DATA) != 0) return RMI_ERR_BAD_ENUM;
  CovPlan pl;
  const int fold = fold_factor(layout, n_rows, n_cols);
  const int rc   = make_cov_plan(dtype, layout, n_rows / fold, n_cols * fold, pl);
  if (rc != RMI_OK) return rc;
  if (n_cols == 0) return RMI_OK;
  if (covar == nullptr) return RMI_ERR_NULL;
  if (n_rows > 0 && data == nullptr) return RMI_ERR_NULL;
  const size_t es = dtype == RMI_F32 ? 4 : 8;
  if (!aligned(data, es) || !aligned(mu, es) || !aligned(covar, es)) return RMI_ERR_ALIGNMENT;
  if (workspace == nullptr || workspace_bytes < pl.ws_bytes + (fold > 1 ? kWideBytes : 0) ||
      !aligned(workspace, 16))
    return RMI_ERR_WORKSPACE;
  hipStream_t st    = static_cast<hipStream_t>(stream);
  const bool center = (flags & RMI_COV_CENTER_DATA) != 0;
  if (dtype == RMI_F32)
    return launch<float>(pl, layout, n_rows, n_cols, sample, center, static_cast<float*>(data),
                         static_cast<const float*>(mu), static_cast<float*>(covar), workspace, st);
  return launch<double>(pl, layout, n_rows, n_cols, sample, center, static_cast<double*>(data),
                        static_cast<const double*>(mu), static_cast<double*>(covar), workspace, st);
}

}  // extern "C"
