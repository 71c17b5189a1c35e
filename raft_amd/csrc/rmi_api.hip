// C ABI of the reduction library (declared in include/rmi_reduce.h):
// validation, plan selection, policy lookup, launch.
#include <atomic>
#include <cstring>

#include "rmi_launch.hpp"

// Scratch of rmi_reduce_noalloc: partials of two-pass plans, for callers that can neither
// allocate nor pass a workspace.  One copy per GPU, at its own address, for the life of the
// process.  In host code this name is only a handle for hipGetSymbolAddress, never a device
// address: kernels get the looked-up pointer as an argument.
static __device__ __align__(256) unsigned char scratch[RMI_NOALLOC_SCRATCH_BYTES];

namespace rmi {

// Zero fill of a few KB on a stream: ticket words are cleared by a kernel so that the call
// can be recorded into a HIP graph (memset nodes have replayed wrongly on this platform).
__global__ __launch_bounds__(256) void zero_words_kernel(u32* p, size_t words)
{
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < words; i += (size_t)gridDim.x * 256)
    p[i] = 0;
}

// CU count of the current device, queried once per process.  Without a
// visible device the MI355X figure is assumed so that planning works on a
// build host.
int cu_count()
{
  static std::atomic<int> cached{0};
  int n = cached.load(std::memory_order_relaxed);
  if (n > 0) return n;
  int dev = 0;
  hipDeviceProp_t prop;
  if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess &&
      prop.multiProcessorCount > 0) {
    n = prop.multiProcessorCount;
  } else {
    (void)hipGetLastError();
    n = 256;
  }
  cached.store(n, std::memory_order_relaxed);
  return n;
}

namespace {

// Device address of `scratch` on the current device, looked up once per device.
constexpr int kMaxDevices = 64;
std::atomic<void*> scratch_ptr[kMaxDevices];

int scratch_of_current_device(void** out)
{
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();
    return RMI_ERR_NO_DEVICE;
  }
  void* p = scratch_ptr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) {
      (void)hipGetLastError();
      return RMI_ERR_NO_DEVICE;
    }
    scratch_ptr[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return RMI_OK;
}

run_fn lookup(const PolicyKey& k)
{
  switch (k.in_dtype) {
    case RMI_I8: return lookup_i8(k);
    case RMI_U8: return lookup_u8(k);
    case RMI_I32: return lookup_i32(k);
    case RMI_I64: return lookup_i64(k);
    case RMI_F16: return lookup_f16(k);
    case RMI_BF16: return lookup_bf16(k);
    case RMI_F32: return lookup_f32(k);
    case RMI_F64: return lookup_f64(k);
    default: return nullptr;
  }
}

bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// A planned reduction: the launch plan, the accumulator policy's key and its launcher.
struct Planned {
  PlanX pl;
  PolicyKey key;
  run_fn fn = nullptr;
};

// What a plan depends on: every descriptor field but the values that only the epilogue
// reads (init, the final scalars, the address behind final_aux), and the input's position
// within a 128-byte line (it decides whether rows are staged through LDS).
struct PlanKey {
  int32_t in_dtype, out_dtype, layout, apply;
  int64_t n_rows, n_cols;
  int32_t main_op, reduce_op, final_op, inplace, plan_hint, flags;
  int32_t has_aux, misalign;
  bool operator==(const PlanKey& o) const { return memcmp(this, &o, sizeof(PlanKey)) == 0; }
};
static_assert(sizeof(PlanKey) == 16 + 16 + 24 + 8, "no padding: keys are compared bytewise");

PlanKey plan_key(const rmi_reduce_desc& d, uintptr_t misalign)
{
  PlanKey k;
  k.in_dtype = d.in_dtype, k.out_dtype = d.out_dtype, k.layout = d.layout, k.apply = d.apply;
  k.n_rows = d.n_rows, k.n_cols = d.n_cols;
  k.main_op = d.main_op, k.reduce_op = d.reduce_op, k.final_op = d.final_op;
  k.inplace = d.inplace ? 1 : 0, k.plan_hint = d.plan_hint, k.flags = d.flags;
  k.has_aux  = d.final_aux != nullptr;
  k.misalign = (int32_t)misalign;
  return k;
}

int plan_uncached(const rmi_reduce_desc& d, uintptr_t misalign, Planned& p,
                  bool own_descriptor = false)
{
  if (!own_descriptor && (d.flags & kFlagSmallWorkspace) != 0) return RMI_ERR_BAD_ENUM;
  int acc_bytes = 8;
  int rc        = classify(d, p.key, acc_bytes);
  if (rc != RMI_OK) return rc;
  p.fn = lookup(p.key);
  if (p.fn == nullptr) return RMI_ERR_UNSUPPORTED;
  return make_plan(d, p.key, acc_bytes, cu_count(), p.pl, misalign);
}

// `in` is the input pointer when the plan is made for a launch, nullptr for queries.  A
// caller that repeats a call (a serving loop, a solver's iteration) repeats its descriptor:
// the last few plans of every host thread are kept, so such a call goes from its arguments
// to the launch without validating and planning again.  Only successful plans are kept.
int plan_for(const rmi_reduce_desc* desc, const Planned*& out, const void* in = nullptr,
             bool own_descriptor = false)
{
  if (desc == nullptr) return RMI_ERR_NULL;
  if (!own_descriptor && (desc->flags & kFlagSmallWorkspace) != 0) return RMI_ERR_BAD_ENUM;
  constexpr int kSlots = 8;
  struct Slot {
    PlanKey k;
    Planned p;
    bool used = false;
  };
  thread_local Slot slots[kSlots];
  thread_local int next = 0;
  const uintptr_t misalign = reinterpret_cast<uintptr_t>(in) % 128;
  const PlanKey k          = plan_key(*desc, misalign);
  for (int i = 0; i < kSlots; ++i) {
    if (slots[i].used && slots[i].k == k) {
      out = &slots[i].p;
      return RMI_OK;
    }
  }
  Slot& s = slots[next];
  s.used  = false;
  const int rc = plan_uncached(*desc, misalign, s.p, own_descriptor);
  if (rc != RMI_OK) return rc;
  s.k    = k;
  s.used = true;
  next   = (next + 1) % kSlots;
  out    = &s.p;
  return RMI_OK;
}

// Launches the planned reduction: pointer checks, epilogue set-up, kernel launch.
int reduce_planned(const rmi_reduce_desc& d,
                   const Planned& planned,
                   const void* in,
                   void* out,
                   void* ws,
                   size_t ws_bytes,
                   void* stream)
{
  const PlanX& pl      = planned.pl;
  const PolicyKey& key = planned.key;
  if (pl.n_out == 0) return RMI_OK;
  if (out == nullptr) return RMI_ERR_NULL;
  if (pl.len > 0 && in == nullptr) return RMI_ERR_NULL;
  if (!aligned(in, dtype_size(d.in_dtype))) return RMI_ERR_ALIGNMENT;
  const int out_es = dtype_size(d.out_dtype);
  // a KVP with a 4-byte key and value is 4-byte aligned by the C rules
  const size_t out_align = d.out_dtype == RMI_KVP_I32_F32 ? 4 : (out_es > 8 ? 8 : out_es);
  if (!aligned(out, out_align)) return RMI_ERR_ALIGNMENT;
  if (d.final_aux != nullptr && !aligned(d.final_aux, out_align)) return RMI_ERR_ALIGNMENT;
  if (pl.ws_bytes > 0) {
    if (ws == nullptr || ws_bytes < pl.ws_bytes) return RMI_ERR_WORKSPACE;
    if (!aligned(ws, 16)) return RMI_ERR_WORKSPACE;
  }

  Problem pr{};
  pr.in            = in;
  pr.ws            = ws;
  pr.epi.out       = out;
  pr.epi.aux       = d.final_aux;
  pr.epi.init_f    = d.init.f;
  pr.epi.init_i    = d.init.i;
  pr.epi.s1        = d.final_scalar;
  pr.epi.s2        = d.final_scalar2;
  pr.epi.out_dtype = d.out_dtype;
  pr.epi.final_op  = d.final_op;
  pr.epi.inplace   = d.inplace ? 1 : 0;
  const bool natural_out =
    key.family == kFamKvp
      ? false
      : (key.family == kFamInt ? true : (d.out_dtype == RMI_F32 || d.out_dtype == RMI_F64));
  const bool simple_final =
    d.final_op == RMI_FIN_IDENTITY ||
    (key.family != kFamInt && (d.final_op == RMI_FIN_SQRT || d.final_op == RMI_FIN_MUL_CONST));
  pr.epi.plain         = (!d.inplace && simple_final && natural_out) ? 1 : 0;
  pr.epi.out_aligned16 = aligned(out, 16) ? 1 : 0;
  return planned.fn(pl, pr, static_cast<hipStream_t>(stream));
}

int reduce_impl(const rmi_reduce_desc& d,
                const void* in,
                void* out,
                void* ws,
                size_t ws_bytes,
                void* stream)
{
  const Planned* p = nullptr;
  const int rc     = plan_for(&d, p, in);
  if (rc != RMI_OK) return rc;
  return reduce_planned(d, *p, in, out, ws, ws_bytes, stream);
}

// map_reduce is a one-row reduction over the contiguous dimension.
rmi_reduce_desc as_single_row(const rmi_reduce_desc& d, int64_t len)
{
  rmi_reduce_desc r = d;
  r.layout          = RMI_ROW_MAJOR;
  r.apply           = RMI_ALONG_ROWS;
  r.n_rows          = 1;
  r.n_cols          = len;
  r.inplace         = 0;
  r.final_aux       = nullptr;
  if (r.final_op == RMI_FIN_VAR_FROM_SUMSQ || r.final_op == RMI_FIN_STDDEV_FROM_SUMSQ)
    r.final_op = -1;  // rejected by classify
  return r;
}

// meanvar: one output pair per column, whatever the layout.
int meanvar_plan(int dtype, int layout, int64_t n_rows, int64_t n_cols, PlanX& pl, run_fn& fn,
                 uintptr_t in_misalign = 0)
{
  if (dtype < 0 || dtype >= RMI_DTYPE_COUNT_) return RMI_ERR_BAD_ENUM;
  if (layout != RMI_ROW_MAJOR && layout != RMI_COL_MAJOR) return RMI_ERR_BAD_ENUM;
  if (n_rows < 0 || n_cols < 0) return RMI_ERR_BAD_SHAPE;
  if (dtype == RMI_F32) fn = lookup_meanvar_f32();
  else if (dtype == RMI_F64) fn = lookup_meanvar_f64();
  else if (dtype == RMI_F16) fn = lookup_meanvar_f16();
  else if (dtype == RMI_BF16) fn = lookup_meanvar_bf16();
  else return RMI_ERR_UNSUPPORTED;
  rmi_reduce_desc d{};
  d.in_dtype  = dtype;
  d.out_dtype = dtype;
  d.layout    = layout;
  d.apply     = RMI_ALONG_COLUMNS;
  d.n_rows    = n_rows;
  d.n_cols    = n_cols;
  d.plan_hint = RMI_PLAN_AUTO;
  PolicyKey key;
  key.in_dtype = dtype;
  key.family   = kFamMeanVar;
  return make_plan(d, key, (int)sizeof(mv_t), cu_count(), pl, in_misalign);
}

}  // namespace
}  // namespace rmi

extern "C" {

int rmi_abi_version(void) { return RMI_ABI_VERSION; }

const char* rmi_status_string(int status)
{
  switch (status) {
    case RMI_OK: return "ok";
    case RMI_ERR_NULL: return "a required pointer is null";
    case RMI_ERR_BAD_ENUM: return "descriptor holds an unknown enum value";
    case RMI_ERR_BAD_SHAPE: return "extent is negative or too large";
    case RMI_ERR_UNSUPPORTED: return "no kernel for this dtype / functor combination";
    case RMI_ERR_WORKSPACE: return "workspace is missing, too small or misaligned";
    case RMI_ERR_ALIGNMENT: return "pointer is not aligned to its element type";
    case RMI_ERR_LAUNCH: return "HIP reported an error at kernel launch";
    case RMI_ERR_NO_DEVICE: return "no usable gfx950 device";
    case RMI_ERR_SCRATCH_LIMIT:
      return "the plan needs more scratch than the library's static buffer holds "
             "(RMI_NOALLOC_SCRATCH_BYTES); use rmi_reduce with a workspace";
    default: return "unknown status";
  }
}

size_t rmi_dtype_size(int dtype) { return (size_t)rmi::dtype_size(dtype); }

int rmi_plan_query(const rmi_reduce_desc* desc, rmi_plan* plan)
{
  if (plan == nullptr) return RMI_ERR_NULL;
  const rmi::Planned* p = nullptr;
  const int rc          = rmi::plan_for(desc, p);
  if (rc != RMI_OK) return rc;
  rmi::export_plan(p->pl, *plan);
  return RMI_OK;
}

// The plan, and with it the workspace, can depend on where the input starts (rows read in
// groups need a 16-byte aligned start): a query answers for the larger of the two.
size_t rmi_reduce_workspace_bytes(const rmi_reduce_desc* desc)
{
  if (desc == nullptr) return 0;
  rmi::Planned pa, pu;
  if (rmi::plan_uncached(*desc, 0, pa) != RMI_OK) return 0;
  if (rmi::plan_uncached(*desc, 1, pu) != RMI_OK) return 0;
  return pa.pl.ws_bytes > pu.pl.ws_bytes ? pa.pl.ws_bytes : pu.pl.ws_bytes;
}

int rmi_reduce(const rmi_reduce_desc* desc,
               const void* in,
               void* out,
               void* workspace,
               size_t workspace_bytes,
               void* stream)
{
  if (desc == nullptr) return RMI_ERR_NULL;
  return rmi::reduce_impl(*desc, in, out, workspace, workspace_bytes, stream);
}

int rmi_reduce_noalloc(const rmi_reduce_desc* desc, const void* in, void* out, void* stream)
{
  if (desc == nullptr) return RMI_ERR_NULL;
  // the buffer's ticket words are zero from load time on and every launch leaves them zero
  rmi_reduce_desc d = *desc;
  if ((d.flags & rmi::kFlagSmallWorkspace) != 0) return RMI_ERR_BAD_ENUM;
  d.flags |= RMI_FLAG_WORKSPACE_ZEROED | rmi::kFlagSmallWorkspace;
  const rmi::Planned* p = nullptr;
  int rc                = rmi::plan_for(&d, p, in, true);
  if (rc != RMI_OK) return rc;
  if (p->pl.ws_bytes > RMI_NOALLOC_SCRATCH_BYTES) return RMI_ERR_SCRATCH_LIMIT;
  // looked up at every device's first call, whether or not this plan needs scratch, so
  // that "the first call" is the only one that does more than launch
  void* ws = nullptr;
  rc       = rmi::scratch_of_current_device(&ws);
  if (rc != RMI_OK) return rc;
  return rmi::reduce_planned(d, *p, in, out, ws, RMI_NOALLOC_SCRATCH_BYTES, stream);
}

int rmi_workspace_reset(void* workspace, size_t workspace_bytes, void* stream)
{
  if (workspace == nullptr) return workspace_bytes == 0 ? RMI_OK : RMI_ERR_NULL;
  if (!rmi::aligned(workspace, 16)) return RMI_ERR_WORKSPACE;
  const size_t bytes = workspace_bytes < RMI_WORKSPACE_TICKET_BYTES ? workspace_bytes
                                                                    : (size_t)RMI_WORKSPACE_TICKET_BYTES;
  const size_t words = bytes / 4;
  if (words == 0) return RMI_OK;
  hipLaunchKernelGGL(rmi::zero_words_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<rmi::u32*>(workspace), words);
  return hipGetLastError() == hipSuccess ? RMI_OK : RMI_ERR_LAUNCH;
}

int rmi_noalloc_reset(void* stream)
{
  void* ws     = nullptr;
  const int rc = rmi::scratch_of_current_device(&ws);
  if (rc != RMI_OK) return rc;
  return rmi_workspace_reset(ws, RMI_NOALLOC_SCRATCH_BYTES, stream);
}

size_t rmi_map_reduce_workspace_bytes(const rmi_reduce_desc* desc, int64_t len)
{
  if (desc == nullptr || len < 0) return 0;
  const rmi_reduce_desc r = rmi::as_single_row(*desc, len);
  return rmi_reduce_workspace_bytes(&r);
}

int rmi_map_reduce(const rmi_reduce_desc* desc,
                   int64_t len,
                   const void* in,
                   void* out,
                   void* workspace,
                   size_t workspace_bytes,
                   void* stream)
{
  if (desc == nullptr) return RMI_ERR_NULL;
  if (len < 0) return RMI_ERR_BAD_SHAPE;
  const rmi_reduce_desc r = rmi::as_single_row(*desc, len);
  return rmi::reduce_impl(r, in, out, workspace, workspace_bytes, stream);
}

int rmi_row_normalize(const rmi_reduce_desc* desc,
                      const void* in,
                      void* out,
                      double eps,
                      void* stream)
{
  using namespace rmi;
  if (desc == nullptr) return RMI_ERR_NULL;
  const rmi_reduce_desc& d = *desc;
  if (d.n_rows < 0 || d.n_cols < 0) return RMI_ERR_BAD_SHAPE;
  if (d.final_op != RMI_FIN_IDENTITY && d.final_op != RMI_FIN_SQRT) return RMI_ERR_UNSUPPORTED;
  norm_fn fn = nullptr;
  switch (d.in_dtype) {
    case RMI_F16: fn = lookup_norm_f16(d.main_op, d.reduce_op); break;
    case RMI_BF16: fn = lookup_norm_bf16(d.main_op, d.reduce_op); break;
    case RMI_F32: fn = lookup_norm_f32(d.main_op, d.reduce_op); break;
    case RMI_F64: fn = lookup_norm_f64(d.main_op, d.reduce_op); break;
    default: return d.in_dtype >= 0 && d.in_dtype < RMI_DTYPE_COUNT_ ? RMI_ERR_UNSUPPORTED
                                                                     : RMI_ERR_BAD_ENUM;
  }
  if (fn == nullptr) return RMI_ERR_UNSUPPORTED;
  if (d.n_rows == 0 || d.n_cols == 0) return RMI_OK;
  if (in == nullptr || out == nullptr) return RMI_ERR_NULL;
  const int es = dtype_size(d.in_dtype);
  if (!aligned(in, es) || !aligned(out, es)) return RMI_ERR_ALIGNMENT;
  NormArgs a{};
  a.in        = in;
  a.out       = out;
  a.n_rows    = d.n_rows;
  a.len       = d.n_cols;
  a.row_bytes = d.n_cols * es;
  a.final_op  = d.final_op;
  a.init      = d.init.f;
  a.eps       = eps;
  const NormPlan small = make_small_norm_plan(d.n_rows, d.n_cols, es, in, out);
  if (small.kind == 4) return fn(small, a, static_cast<hipStream_t>(stream));
  const NormPlan flat = make_flat_norm_plan(d.n_rows, d.n_cols, es, in, out);
  if (flat.kind == 3) {
    const int rc = fn(flat, a, static_cast<hipStream_t>(stream));
    if (rc != RMI_OK || flat.flat_rows == d.n_rows) return rc;
    // the last few rows, which do not end on a 16-byte boundary, go the ordinary way
    a.in     = static_cast<const char*>(in) + flat.flat_rows * a.row_bytes;
    a.out    = static_cast<char*>(out) + flat.flat_rows * a.row_bytes;
    a.n_rows = d.n_rows - flat.flat_rows;
  }
  const NormPlan pl = make_norm_plan(a.n_rows, d.n_cols, es);
  return fn(pl, a, static_cast<hipStream_t>(stream));
}

size_t rmi_meanvar_workspace_bytes(int dtype, int layout, int64_t n_rows, int64_t n_cols)
{
  rmi::PlanX pl, pu;
  rmi::run_fn fn = nullptr;
  if (rmi::meanvar_plan(dtype, layout, n_rows, n_cols, pl, fn) != RMI_OK) return 0;
  if (rmi::meanvar_plan(dtype, layout, n_rows, n_cols, pu, fn, 1) != RMI_OK) return 0;
  return pl.ws_bytes > pu.ws_bytes ? pl.ws_bytes : pu.ws_bytes;
}

int rmi_meanvar(int dtype,
                int layout,
                int64_t n_rows,
                int64_t n_cols,
                int sample,
                const void* data,
                void* mean,
                void* var,
                void* workspace,
                size_t workspace_bytes,
                void* stream)
{
  using namespace rmi;
  PlanX pl;
  run_fn fn    = nullptr;
  const int rc = meanvar_plan(dtype, layout, n_rows, n_cols, pl, fn,
                              reinterpret_cast<uintptr_t>(data) % 128);
  if (rc != RMI_OK) return rc;
  if (pl.n_out == 0) return RMI_OK;
  if (mean == nullptr || var == nullptr) return RMI_ERR_NULL;
  if (pl.len > 0 && data == nullptr) return RMI_ERR_NULL;
  const int es = dtype_size(dtype);
  if (!aligned(data, es) || !aligned(mean, es) || !aligned(var, es)) return RMI_ERR_ALIGNMENT;
  if (pl.ws_bytes > 0) {
    if (workspace == nullptr || workspace_bytes < pl.ws_bytes) return RMI_ERR_WORKSPACE;
    if (!aligned(workspace, 16)) return RMI_ERR_WORKSPACE;
  }
  Problem pr{};
  pr.in            = data;
  pr.ws            = workspace;
  pr.epi.out       = mean;
  pr.epi.aux       = var;
  pr.epi.s1        = sample ? 1.0 : 0.0;
  pr.epi.out_dtype = dtype;
  return fn(pl, pr, static_cast<hipStream_t>(stream));
}

}  // extern "C"
