/*
 * rmi_reduce.h — C ABI of the MI355X (gfx950) dense-reduction library.
 *
 * Plain C: pointers, sizes and POD descriptors only.  Every entry point is
 * stream-ordered, never synchronises the stream, never allocates device
 * memory, never throws, and returns an rmi_status code.  Device pointers are
 * ordinary HIP device addresses; `stream` is a hipStream_t passed as void*
 * (NULL = the null stream).
 *
 * Each declaration names the interface of NVIDIA/raft (paths relative to
 * cpp/include/raft) that it stands in for.  The reference has no FFI layer of
 * its own for this path: its boundary is the header-template API, and the C++
 * headers shipped beside this library keep those templates and lower them to
 * the calls below.
 */
#ifndef RMI_REDUCE_H_
#define RMI_REDUCE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RMI_ABI_VERSION 3

#if defined(__GNUC__) || defined(__clang__)
#define RMI_API __attribute__((visibility("default")))
#else
#define RMI_API
#endif

/* ---- status ----------------------------------------------------------- */
typedef enum rmi_status {
  RMI_OK                 = 0,
  RMI_ERR_NULL           = 1, /* a required pointer is NULL                       */
  RMI_ERR_BAD_ENUM       = 2, /* an enum field holds an unknown value             */
  RMI_ERR_BAD_SHAPE      = 3, /* negative extent, or extent too large             */
  RMI_ERR_UNSUPPORTED    = 4, /* dtype / functor combination has no kernel        */
  RMI_ERR_WORKSPACE      = 5, /* workspace missing, too small or misaligned       */
  RMI_ERR_ALIGNMENT      = 6, /* in/out pointer not aligned to its element size   */
  RMI_ERR_LAUNCH         = 7, /* HIP reported an error at launch                  */
  RMI_ERR_NO_DEVICE      = 8, /* no usable gfx950 device / code object            */
  RMI_ERR_SCRATCH_LIMIT  = 9  /* rmi_reduce_noalloc: the plan needs more scratch
                                 than RMI_NOALLOC_SCRATCH_BYTES                   */
} rmi_status;

/* ---- element types ---------------------------------------------------- */
/* KVP types are raft::KeyValuePair<Key,Value> (core/kvp.hpp:20-62): key
 * first, then value, natural alignment: {i32,f32} = 8 B, {i32,f64} = 16 B
 * (4 B padding after the key), {i64,f32} = 16 B (4 B tail padding),
 * {i64,f64} = 16 B. */
typedef enum rmi_dtype {
  RMI_I8 = 0,
  RMI_U8 = 1,
  RMI_I32 = 2,
  RMI_I64 = 3,
  RMI_F16 = 4,
  RMI_BF16 = 5,
  RMI_F32 = 6,
  RMI_F64 = 7,
  RMI_KVP_I32_F32 = 8,
  RMI_KVP_I32_F64 = 9,
  RMI_KVP_I64_F32 = 10,
  RMI_KVP_I64_F64 = 11,
  RMI_DTYPE_COUNT_ = 12
} rmi_dtype;

/* ---- layout / axis ---------------------------------------------------- */
/* raft::row_major / raft::col_major (core/mdspan_types.hpp:14-37) */
typedef enum rmi_layout { RMI_ROW_MAJOR = 0, RMI_COL_MAJOR = 1 } rmi_layout;
/* raft::Apply (linalg/linalg_types.hpp): ALONG_ROWS gives one output per row,
 * ALONG_COLUMNS one output per column. */
typedef enum rmi_apply { RMI_ALONG_ROWS = 0, RMI_ALONG_COLUMNS = 1 } rmi_apply;

/* ---- functor vocabulary (core/operators.hpp:27-203,253-370) ------------ */
/* main_op(value, index_along_reduced_axis) */
typedef enum rmi_main_op {
  RMI_MAIN_IDENTITY = 0, /* identity_op, cast_op<Out>                      */
  RMI_MAIN_SQ       = 1, /* sq_op                                          */
  RMI_MAIN_ABS      = 2, /* abs_op                                         */
  RMI_MAIN_NZ       = 3, /* nz_op: x != 0 ? 1 : 0                          */
  RMI_MAIN_KVP      = 4  /* (value, idx) -> KeyValuePair{idx, value}; the  */
                         /* only main_op allowed with ARGMIN / ARGMAX      */
} rmi_main_op;

typedef enum rmi_reduce_op {
  RMI_RED_ADD    = 0, /* add_op (compensated: linalg/reduce.cuh:25-27)     */
  RMI_RED_MAX    = 1, /* max_op (NaN-ignoring, core/math.hpp:375-397)      */
  RMI_RED_MIN    = 2, /* min_op                                            */
  RMI_RED_ARGMAX = 3, /* argmax_op (core/operators.hpp:196-203)            */
  RMI_RED_ARGMIN = 4  /* argmin_op (core/operators.hpp:187-194)            */
} rmi_reduce_op;

/* final_op(acc) applied once per output, in the output's arithmetic type
 * (f32 for f16/bf16/f32 outputs, f64 for f64, i64 for integers). */
typedef enum rmi_final_op {
  RMI_FIN_IDENTITY  = 0,
  RMI_FIN_SQRT      = 1, /* sqrt_op                                         */
  RMI_FIN_ABS       = 2, /* abs_op                                          */
  RMI_FIN_SQ        = 3, /* sq_op                                           */
  RMI_FIN_MUL_CONST = 4, /* mul_const_op<Out>(final_scalar)                 */
  RMI_FIN_DIV_CONST = 5, /* div_const_op<Out>(final_scalar)                 */
  RMI_FIN_ADD_CONST = 6, /* add_const_op<Out>(final_scalar)                 */
  RMI_FIN_SUB_CONST = 7, /* sub_const_op<Out>(final_scalar)                 */
  /* acc, aux[k] -> |acc*final_scalar - aux[k]^2*final_scalar2|, and its
   * square root: the epilogue of stats::vars / stats::stddev
   * (stats/detail/stddev.cuh:46-59,91-101), fused into the reduction. */
  RMI_FIN_VAR_FROM_SUMSQ    = 8,
  RMI_FIN_STDDEV_FROM_SUMSQ = 9,
  RMI_FIN_KEY = 10 /* key_op: KVP accumulator -> its key (integer output);
                      matrix::argmax/argmin write the key only
                      (matrix/detail/math.cuh:310)                         */
} rmi_final_op;

/* ---- scalar carrier for `init` ---------------------------------------- */
typedef struct rmi_scalar {
  double  f;   /* floating outputs: init value; KVP outputs: init.value      */
  int64_t i;   /* integer outputs: init value;  KVP outputs: init.key        */
} rmi_scalar;

/* ---- the reduction descriptor ------------------------------------------
 * Stands in for the template arguments and value arguments of
 *   raft::linalg::reduce            (linalg/reduce.cuh:55-76,140-180)
 *   raft::linalg::coalescedReduction (linalg/coalesced_reduction.cuh:55-70)
 *   raft::linalg::stridedReduction   (linalg/strided_reduction.cuh:57-78)
 * Semantics, for every output k and r running over the reduced axis:
 *   acc_k   = reduce_op-fold over r of main_op(in[k,r], r)
 *   acc_k   = reduce_op(init, acc_k)                  (init applied once)
 *   if inplace: acc_k = reduce_op(out_old[k], acc_k)
 *   out[k]  = final_op(acc_k)
 */
typedef struct rmi_reduce_desc {
  int32_t in_dtype;    /* rmi_dtype of the matrix                             */
  int32_t out_dtype;   /* rmi_dtype of the output vector                      */
  int32_t layout;      /* rmi_layout                                          */
  int32_t apply;       /* rmi_apply                                           */
  int64_t n_rows;      /* data.extent(0)                                      */
  int64_t n_cols;      /* data.extent(1)                                      */
  int32_t main_op;     /* rmi_main_op                                         */
  int32_t reduce_op;   /* rmi_reduce_op                                       */
  int32_t final_op;    /* rmi_final_op                                        */
  int32_t inplace;     /* 0 / 1                                               */
  rmi_scalar init;     /* must be reduce_op's neutral element                 */
  double final_scalar; /* constant of *_CONST; `ratio` of VAR/STDDEV          */
  double final_scalar2;/* `ratio_mean` of VAR/STDDEV                          */
  const void* final_aux; /* device vector (out_dtype, one per output) read by
                            VAR/STDDEV (the mean); NULL otherwise            */
  int32_t plan_hint;   /* rmi_plan_kind to force, or 0 = choose by shape      */
  int32_t flags;       /* RMI_FLAG_* bits; unknown bits are refused           */
} rmi_reduce_desc;

/* The caller promises that the first RMI_WORKSPACE_TICKET_BYTES bytes of the workspace passed
 * with this descriptor were zero when the workspace was first handed to this library and
 * have only been written by this library since.  Rows split over several workgroups are
 * then reduced in ONE launch: every workgroup takes a ticket for its row (counters in that
 * area, one per 16 workgroups of a row plus one per row, each on a 128-byte line of its
 * own), the last one to arrive folds the row's partials in index order (results stay
 * bitwise repeatable and equal to the two-launch plan's) and every counter wraps back to
 * zero, so the area is zero again when the call has run.  Without the flag the workspace
 * needs no initialisation and such rows take a second, folding launch.
 * The hand-off between the workgroups of that one launch is written for gfx942 / gfx950
 * (write-through stores acknowledged by the memory side, device-scope atomics) and is
 * outside the HIP memory model; the library refuses to build for other targets.  Ticket
 * words are state: see rmi_workspace_reset for what leaves them non-zero and how to recover. */
#define RMI_FLAG_WORKSPACE_ZEROED 1
#define RMI_WORKSPACE_TICKET_BYTES 65536

/* ---- launch plans ------------------------------------------------------ */
typedef enum rmi_plan_kind {
  RMI_PLAN_AUTO       = 0,
  RMI_PLAN_ROW_LANES  = 1, /* several whole rows per lane-load (rows <= 8 B..16 B)  */
  RMI_PLAN_ROW_WAVE   = 2, /* 1..64 lanes of one wavefront per row                  */
  RMI_PLAN_ROW_BLOCK  = 3, /* a team of 128..1024 threads per row, LDS combine       */
  RMI_PLAN_ROW_SPLIT  = 4, /* several blocks per row + second pass over partials    */
  RMI_PLAN_COL_TILE   = 5, /* column reduction: column-contiguous lanes, row ranges
                              per block, LDS combine, second pass over partials
                              (rows of 2 KB..20 KB: whole adjacent rows per block)  */
  RMI_PLAN_EMPTY      = 6  /* nothing to read: outputs get final_op(init) only      */
} rmi_plan_kind;

typedef struct rmi_plan {
  int32_t kind;            /* rmi_plan_kind actually chosen                   */
  int32_t vec_bytes;       /* bytes per lane-load (16, or the element size)   */
  int32_t lanes_per_row;   /* ROW_WAVE: lanes that share one row (1..64; a    */
                           /* power of two, or the row's own lane-load count) */
  int32_t blocks_per_out;  /* ROW_SPLIT / COL_TILE: partials per output (for  */
                           /* an input that starts on a 16-byte boundary)     */
  int32_t block_threads;   /* threads per workgroup                           */
  int32_t passes;          /* kernel launches (1 or 2)                        */
  int64_t grid_blocks;     /* workgroups of the first launch                  */
  int64_t n_outputs;       /* outputs produced                                */
  int64_t reduce_len;      /* elements folded into each output                */
  size_t  workspace_bytes; /* device workspace the plan needs (0 if none)     */
} rmi_plan;

/* ---- entry points ------------------------------------------------------ */

/* ABI version of the loaded library (== RMI_ABI_VERSION it was built with). */
RMI_API int rmi_abi_version(void);

/* Human-readable text for a status code; never NULL. */
RMI_API const char* rmi_status_string(int status);

/* sizeof one element of an rmi_dtype, 0 for an unknown value. */
RMI_API size_t rmi_dtype_size(int dtype);

/* Plan chosen for `desc` on the current device (CU count is queried once and
 * cached; with no device visible a 256-CU MI355X is assumed, so this call
 * works on a host without a GPU).  Replaces the hard-coded Thin/Medium/Thick
 * heuristics of linalg/detail/coalesced_reduction-inl.cuh:640-670 and the
 * launch shapes of linalg/detail/strided_reduction.cuh:148-188. */
RMI_API int rmi_plan_query(const rmi_reduce_desc* desc, rmi_plan* plan);

/* Bytes of device workspace rmi_reduce needs for `desc` (0 for single-pass
 * plans), whatever the alignment of the input pointer (a plan can depend on
 * it; the larger need is reported).  Replaces the internal rmm::device_uvector of
 * linalg/detail/coalesced_reduction-inl.cuh:560. */
RMI_API size_t rmi_reduce_workspace_bytes(const rmi_reduce_desc* desc);

/* The reduction itself: replaces detail::reduce (linalg/detail/reduce.cuh:25-49),
 * detail::coalescedReduction (linalg/detail/coalesced_reduction-inl.cuh:640-670)
 * and detail::stridedReduction (linalg/detail/strided_reduction.cuh:129-196).
 * `in`: n_rows*n_cols elements, contiguous in `layout`.  `out`: one element per
 * output.  `workspace`: at least rmi_reduce_workspace_bytes(desc) bytes, 16-byte
 * aligned, may be NULL when that is 0; its contents need no initialisation (unless
 * desc->flags says RMI_FLAG_WORKSPACE_ZEROED) and, past the first
 * RMI_WORKSPACE_TICKET_BYTES bytes, are undefined afterwards.  Calls that share a
 * workspace must be ordered on one stream. */
RMI_API int rmi_reduce(const rmi_reduce_desc* desc,
               const void* in,
               void* out,
               void* workspace,
               size_t workspace_bytes,
               void* stream);

/* rmi_reduce for callers that cannot allocate device memory and have no workspace to
 * pass: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  It has no counterpart in the reference (whose Thick plan allocates an
 * rmm::device_uvector inside the call, linalg/detail/coalesced_reduction-inl.cuh:560).
 * Same descriptor, same kernels, same results bit for bit as rmi_reduce; the partials of
 * two-pass plans go to a buffer of RMI_NOALLOC_SCRATCH_BYTES bytes that the library keeps
 * in every GPU it runs on for the life of the process (a static device array; its address
 * is looked up once per device, at the first call made with that device current: make
 * that first call outside stream capture).  The call itself allocates and frees nothing.
 * A descriptor whose plan needs more scratch (rmi_reduce_workspace_bytes(desc) >
 * RMI_NOALLOC_SCRATCH_BYTES) is refused with RMI_ERR_SCRATCH_LIMIT and nothing is
 * launched.  All calls on one GPU share that GPU's buffer: calls that may run at the same
 * time (different streams, or branches of one graph) race on it; order them on one stream.
 * The buffer's ticket words (see RMI_FLAG_WORKSPACE_ZEROED, which this entry point always
 * applies) are zero when the library is loaded and every launch leaves them zero; nothing
 * else in it has to start at zero: every partial is written before it is read. */
#define RMI_NOALLOC_SCRATCH_BYTES ((size_t)4 << 20)
RMI_API int rmi_reduce_noalloc(const rmi_reduce_desc* desc,
                               const void* in,
                               void* out,
                               void* stream);

/* Zeroes the ticket words of a workspace (its first RMI_WORKSPACE_TICKET_BYTES bytes, or all
 * of it when it is shorter) with a small kernel on `stream`: what a caller runs once on a
 * fresh workspace before it passes RMI_FLAG_WORKSPACE_ZEROED, and again to recover one whose
 * ticket words may have been left non-zero (a launch that was aborted or failed, calls that
 * overlapped on two streams, a stray write).  Counters left non-zero are not detected: the
 * rows they belong to are never folded and their outputs keep their old contents, on every
 * later call, while the calls still return RMI_OK.  A kernel, not a memset, so the call may be
 * recorded into a HIP graph.  No counterpart in the reference (its Thick plan takes a second
 * launch, linalg/detail/coalesced_reduction-inl.cuh:595-625). */
RMI_API int rmi_workspace_reset(void* workspace, size_t workspace_bytes, void* stream);

/* The same for the static buffer of rmi_reduce_noalloc on the current device. */
RMI_API int rmi_noalloc_reset(void* stream);

/* Whole-array map + reduce to one scalar: replaces detail::mapThenReduceImpl
 * (linalg/detail/map_then_reduce.cuh:72-95) behind mapThenSumReduce /
 * mapThenReduce / mapReduce / map_reduce (linalg/map_then_reduce.cuh:37-80,
 * linalg/map_reduce.cuh:37-103).  *out = reduce_op(neutral, fold of
 * main_op(in[i], i)), i < len.  Deterministic (no atomics).  Uses the
 * descriptor fields in_dtype, out_dtype, main_op, reduce_op, final_op, init
 * (= neutral), final_scalar; n_rows/n_cols/layout/apply are ignored. */
RMI_API size_t rmi_map_reduce_workspace_bytes(const rmi_reduce_desc* desc, int64_t len);
RMI_API int rmi_map_reduce(const rmi_reduce_desc* desc,
                   int64_t len,
                   const void* in,
                   void* out,
                   void* workspace,
                   size_t workspace_bytes,
                   void* stream);

/* Row normalisation fused with its norm: out[i, :] = in[i, :] / norm_i with
 * norm_i = final_op(reduce_op(init, fold over j of main_op(in[i, j]))); rows whose
 * norm is <= eps are left untouched (a NaN norm is not: that row is written as NaN, as in
 * the reference).  Replaces detail::coalesced_normalize
 * (linalg/detail/normalize.cuh:36-197) behind raft::linalg::row_normalize
 * (linalg/normalize.cuh:48-110).  Uses the descriptor fields in_dtype (also the
 * output's type: F16, BF16, F32 or F64), n_rows, n_cols, main_op (IDENTITY, SQ, ABS),
 * reduce_op (ADD, MAX, MIN), final_op (IDENTITY or SQRT) and init.f; the matrix is
 * row-major.  F32 / F64 rows are divided element by element in their own arithmetic;
 * F16 / BF16 rows are multiplied in f32 by one reciprocal of the norm, then rounded.
 * `out` may be `in`.  Needs no workspace. */
RMI_API int rmi_row_normalize(const rmi_reduce_desc* desc,
                              const void* in,
                              void* out,
                              double eps,
                              void* stream);

/* Mean and variance of every column of an [n_rows, n_cols] matrix in one pass over
 * the data: mean[j] = sum_i x[i, j] / n_rows, var[j] = sum_i (x[i, j] - mean[j])^2 /
 * max(1, sample ? n_rows - 1 : n_rows).  Replaces detail::meanvar
 * (stats/detail/meanvar.cuh:187-236) behind raft::stats::meanvar
 * (stats/meanvar.cuh:38-49 pointer form, :74-98 mdspan form).  `dtype` is F32, F64,
 * F16 or BF16 (data, mean and var share it), `layout` an rmi_layout.  The arithmetic is
 * f64 throughout; results are rounded once to `dtype`.  An empty column set is a no-op; n_rows == 0 writes zeros.  The workspace
 * follows the rules of rmi_reduce. */
RMI_API size_t rmi_meanvar_workspace_bytes(int dtype, int layout, int64_t n_rows, int64_t n_cols);
RMI_API int rmi_meanvar(int dtype,
                        int layout,
                        int64_t n_rows,
                        int64_t n_cols,
                        int sample,
                        const void* data,
                        void* mean,
                        void* var,
                        void* workspace,
                        size_t workspace_bytes,
                        void* stream);

/* Covariance matrix of the columns of an [n_rows, n_cols] matrix around a given mean
 * vector: covar[i][j] = sum_n (x[n,i] - mu[i]) * (x[n,j] - mu[j]) / (sample ? n_rows - 1 :
 * n_rows).  Replaces detail::cov (stats/detail/cov.cuh:38-66: meanCenter in place, then a
 * cuBLAS GEMM X^T X scaled by alpha) behind raft::stats::cov (stats/cov.cuh:38-50 pointer
 * form, :77-106 mdspan form).  `dtype` is F32 or F64 (data, mu and covar share it), `layout`
 * the rmi_layout of `data`; `covar` is [n_cols][n_cols] and symmetric, so its layout does not
 * matter.  The contraction runs on the matrix cores: F64 data with fp64 products and sums;
 * F32 data split exactly into three bf16 terms per value, six of the nine cross terms
 * multiplied (the three left out are below 2^-23 of the product, one fp32 rounding) and
 * summed in fp32.  Partial sums of row slabs are added in f64.  (An infinite F32 input gives
 * NaN where an fp32 product would give an infinity; subnormal terms of the split may be
 * flushed.)  `mu` may be NULL: the data is taken
 * as centred already.  With RMI_COV_CENTER_DATA in `flags` the call leaves x - mu in `data`,
 * which is what the reference documents ("this will get mean-centered at the end!") and its
 * callers rely on; without it `data` is only read and the matrix is moved once instead of
 * read and written.  n_rows == 0 writes zeros.  The workspace follows the rules of
 * rmi_reduce (rmi_cov_workspace_bytes bytes, 16-byte aligned, no initialisation needed). */
#define RMI_COV_CENTER_DATA 1
RMI_API size_t rmi_cov_workspace_bytes(int dtype, int layout, int64_t n_rows, int64_t n_cols);
RMI_API int rmi_cov(int dtype,
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
                    void* stream);

#ifdef __cplusplus
} /* extern "C" */
#endif
#endif /* RMI_REDUCE_H_ */
