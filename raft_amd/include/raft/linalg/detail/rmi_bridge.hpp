// Lowering of the template API to the C ABI of the reduction library
// (include/rmi_reduce.h): element types and functor types become tags in an
// rmi_reduce_desc, status codes come back as the reference's exception types.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <limits>
#include <type_traits>

#include <raft/core/error.hpp>
#include <raft/core/kvp.hpp>
#include <raft/core/operators.hpp>
#include <raft/core/resources.hpp>
#include <raft/linalg/detail/rmi_scratch.hpp>

#include "rmi_reduce.h"

#if defined(__HIPCC__)
#include <raft/linalg/detail/rmi_generic.hpp>
#endif

namespace raft {

// bfloat16 storage (1 sign, 8 exponent, 7 mantissa bits) for inputs and outputs
// of that type; arithmetic on it happens on the device only.
struct bfloat16_t {
  std::uint16_t bits;
};

namespace detail::rmi {

template <typename T>
inline constexpr bool always_false = false;

// ---- element types ------------------------------------------------------------
template <typename T, typename = void>
struct dtype_of {
  static constexpr int value = -1;
};
#define RAFT_RMI_DTYPE(T, TAG)          \
  template <>                           \
  struct dtype_of<T> {                  \
    static constexpr int value = TAG;   \
  }
RAFT_RMI_DTYPE(std::int8_t, RMI_I8);
RAFT_RMI_DTYPE(std::uint8_t, RMI_U8);
RAFT_RMI_DTYPE(std::int32_t, RMI_I32);
RAFT_RMI_DTYPE(std::int64_t, RMI_I64);
RAFT_RMI_DTYPE(long long, RMI_I64);
RAFT_RMI_DTYPE(__half, RMI_F16);
RAFT_RMI_DTYPE(bfloat16_t, RMI_BF16);
RAFT_RMI_DTYPE(float, RMI_F32);
RAFT_RMI_DTYPE(double, RMI_F64);
#undef RAFT_RMI_DTYPE
template <typename K, typename V>
struct dtype_of<KeyValuePair<K, V>,
                std::enable_if_t<std::is_integral_v<K> && std::is_signed_v<K> &&
                                 (sizeof(K) == 4 || sizeof(K) == 8) &&
                                 (std::is_same_v<V, float> || std::is_same_v<V, double>)>> {
  static constexpr int value =
    sizeof(K) == 4 ? (std::is_same_v<V, float> ? RMI_KVP_I32_F32 : RMI_KVP_I32_F64)
                   : (std::is_same_v<V, float> ? RMI_KVP_I64_F32 : RMI_KVP_I64_F64);
};

template <typename T>
constexpr int dtype()
{
  static_assert(dtype_of<std::remove_cv_t<T>>::value >= 0,
                "element type not supported by the reduction library "
                "(int8, uint8, int32, int64, __half, bfloat16_t, float, double, "
                "KeyValuePair<int32|int64, float|double>)");
  return dtype_of<std::remove_cv_t<T>>::value;
}

template <typename T>
struct is_kvp : std::false_type {};
template <typename K, typename V>
struct is_kvp<KeyValuePair<K, V>> : std::true_type {};

// ---- functor types -> tags -------------------------------------------------------
// Specialise these for a functor type of your own if it computes exactly what one
// of the tags means (e.g. a local "value -> {idx, value}" functor is RMI_MAIN_KVP).
template <typename F>
struct main_tag {
  static constexpr int value = -1;
};
template <>
struct main_tag<identity_op> {
  static constexpr int value = RMI_MAIN_IDENTITY;
};
// cast_op<T> is the identity to the library (which widens every element into an f64 or
// int64 accumulator anyway) only where the cast keeps the value: to a floating type, or
// between integers without narrowing.  A cast that truncates (cast_op<int> on float data)
// has no tag; see cast_keeps_value below.
template <typename T>
struct main_tag<cast_op<T>> {
  static constexpr int value = RMI_MAIN_IDENTITY;
};
template <typename F, typename In>
struct cast_keeps_value : std::true_type {};
template <typename T, typename In>
struct cast_keeps_value<cast_op<T>, In>
  : std::bool_constant<std::is_floating_point_v<T> || std::is_same_v<T, __half> ||
                       (std::is_integral_v<T> && std::is_integral_v<In> && sizeof(T) >= sizeof(In))> {};
template <>
struct main_tag<sq_op> {
  static constexpr int value = RMI_MAIN_SQ;
};
template <>
struct main_tag<abs_op> {
  static constexpr int value = RMI_MAIN_ABS;
};
template <>
struct main_tag<nz_op> {
  static constexpr int value = RMI_MAIN_NZ;
};
template <typename I>
struct main_tag<value_to_kvp_op<I>> {
  static constexpr int value = RMI_MAIN_KVP;
};

template <typename F>
struct reduce_tag {
  static constexpr int value = -1;
};
template <>
struct reduce_tag<add_op> {
  static constexpr int value = RMI_RED_ADD;
};
template <>
struct reduce_tag<max_op> {
  static constexpr int value = RMI_RED_MAX;
};
template <>
struct reduce_tag<min_op> {
  static constexpr int value = RMI_RED_MIN;
};
template <>
struct reduce_tag<argmax_op> {
  static constexpr int value = RMI_RED_ARGMAX;
};
template <>
struct reduce_tag<argmin_op> {
  static constexpr int value = RMI_RED_ARGMIN;
};

template <typename F>
struct final_tag {
  static constexpr int value = -1;
  static double scalar(const F&) { return 0.0; }
};
#define RAFT_RMI_FINAL(F, TAG)                      \
  template <>                                       \
  struct final_tag<F> {                             \
    static constexpr int value = TAG;               \
    static double scalar(const F&) { return 0.0; }  \
  }
RAFT_RMI_FINAL(identity_op, RMI_FIN_IDENTITY);
RAFT_RMI_FINAL(sqrt_op, RMI_FIN_SQRT);
RAFT_RMI_FINAL(abs_op, RMI_FIN_ABS);
RAFT_RMI_FINAL(sq_op, RMI_FIN_SQ);
RAFT_RMI_FINAL(key_op, RMI_FIN_KEY);
#undef RAFT_RMI_FINAL
template <typename T>
struct final_tag<cast_op<T>> {
  static constexpr int value = RMI_FIN_IDENTITY;
  static double scalar(const cast_op<T>&) { return 0.0; }
};
#define RAFT_RMI_FINAL_CONST(OP, TAG)                                               \
  template <typename T>                                                             \
  struct final_tag<plug_const_op<T, OP>> {                                          \
    static constexpr int value = TAG;                                               \
    static double scalar(const plug_const_op<T, OP>& f) { return to_double(f.c); }  \
  }
template <typename T>
double to_double(const T& c)
{
  if constexpr (std::is_same_v<T, __half>) {
    return (double)__half2float(c);
  } else {
    return static_cast<double>(c);
  }
}
RAFT_RMI_FINAL_CONST(mul_op, RMI_FIN_MUL_CONST);
RAFT_RMI_FINAL_CONST(div_op, RMI_FIN_DIV_CONST);
RAFT_RMI_FINAL_CONST(add_op, RMI_FIN_ADD_CONST);
RAFT_RMI_FINAL_CONST(sub_op, RMI_FIN_SUB_CONST);
#undef RAFT_RMI_FINAL_CONST

// ---- does the library have a kernel for this combination? ----------------------------
// The rules of the library's own descriptor check, on the tags: a combination it would
// refuse at run time (a count of non-zeros into an int from float data, max of integers
// into a float, ...) is instantiated in the caller's translation unit instead, like any
// other functor the vocabulary lacks.
constexpr bool dtype_is_float(int dt)
{
  return dt == RMI_F16 || dt == RMI_BF16 || dt == RMI_F32 || dt == RMI_F64;
}
constexpr bool dtype_is_int(int dt)
{
  return dt == RMI_I8 || dt == RMI_U8 || dt == RMI_I32 || dt == RMI_I64;
}
constexpr bool dtype_is_kvp(int dt) { return dt >= RMI_KVP_I32_F32 && dt <= RMI_KVP_I64_F64; }

constexpr bool library_serves(int in_dt, int out_dt, int main_op, int red_op, int final_op)
{
  if (in_dt < 0 || out_dt < 0 || main_op < 0 || red_op < 0 || final_op < 0) return false;
  if (dtype_is_kvp(in_dt)) return false;
  const bool arg = red_op == RMI_RED_ARGMAX || red_op == RMI_RED_ARGMIN;
  if (arg) {
    if (main_op != RMI_MAIN_KVP || !dtype_is_float(in_dt)) return false;
    // (matrix::argmax names the pair type and overrides the stored type with the key's)
    if (final_op == RMI_FIN_KEY) return out_dt == RMI_I32 || out_dt == RMI_I64 || dtype_is_kvp(out_dt);
    if (final_op != RMI_FIN_IDENTITY || !dtype_is_kvp(out_dt)) return false;
    const bool out_val64 = out_dt == RMI_KVP_I32_F64 || out_dt == RMI_KVP_I64_F64;
    return out_val64 == (in_dt == RMI_F64);
  }
  if (main_op == RMI_MAIN_KVP || final_op == RMI_FIN_KEY || dtype_is_kvp(out_dt)) return false;
  if (main_op == RMI_MAIN_NZ && red_op != RMI_RED_ADD) return false;
  if (dtype_is_float(out_dt)) return !(dtype_is_int(in_dt) && red_op != RMI_RED_ADD);
  // integer output: integer arithmetic end to end
  return dtype_is_int(in_dt) && (out_dt == RMI_I32 || out_dt == RMI_I64) &&
         final_op != RMI_FIN_SQRT && final_op != RMI_FIN_VAR_FROM_SUMSQ &&
         final_op != RMI_FIN_STDDEV_FROM_SUMSQ;
}

// ---- status -> exception ----------------------------------------------------------
inline void check(int status, const char* what)
{
  if (status == RMI_OK) return;
  const std::string msg = std::string(what) + ": " + rmi_status_string(status);
  switch (status) {
    case RMI_ERR_UNSUPPORTED: throw raft::exception("exception occurred! " + msg);
    case RMI_ERR_LAUNCH:
    case RMI_ERR_NO_DEVICE: throw raft::hip_error("HIP error encountered at: " + msg);
    default: throw raft::logic_error("RAFT failure at " + msg);
  }
}

// ---- workspace ----------------------------------------------------------------------
// With a handle the workspace belongs to the handle and is reused (its ticket words are
// zero, see raft::resources::workspace, so split rows are reduced in one launch); with a
// bare stream it is a stream-ordered allocation released after the launches (what the
// reference does with rmm::device_uvector, coalesced_reduction-inl.cuh:560).
class workspace_lease {
 public:
  workspace_lease(const resources* res, hipStream_t stream, size_t bytes) : stream_(stream)
  {
    if (bytes == 0) return;
    bytes_ = bytes;
    if (res != nullptr) {
      ptr_    = res->workspace(bytes);
      zeroed_ = true;
    } else {
      ptr_   = scratch_alloc(bytes, stream);
      owned_ = true;
    }
  }
  workspace_lease(const workspace_lease&)            = delete;
  workspace_lease& operator=(const workspace_lease&) = delete;
  ~workspace_lease()
  {
    if (owned_) scratch_free(ptr_, stream_);
  }
  void* data() const { return ptr_; }
  size_t size() const { return bytes_; }
  int flags() const { return zeroed_ ? RMI_FLAG_WORKSPACE_ZEROED : 0; }

 private:
  void* ptr_     = nullptr;
  size_t bytes_  = 0;
  bool owned_    = false;
  bool zeroed_   = false;
  hipStream_t stream_;
};

// OutType(0) for every output type the library writes (__half has no
// unambiguous conversion from int on the host).
template <typename OutType>
OutType zero()
{
  if constexpr (std::is_same_v<OutType, __half>) {
    return __float2half(0.0f);
  } else if constexpr (std::is_same_v<OutType, bfloat16_t>) {
    return bfloat16_t{0};
  } else {
    return OutType(0);
  }
}

template <typename OutType>
rmi_scalar make_init(const OutType& init)
{
  rmi_scalar s{0.0, 0};
  if constexpr (is_kvp<OutType>::value) {
    s.i = static_cast<std::int64_t>(init.key);
    s.f = static_cast<double>(init.value);
  } else if constexpr (std::is_integral_v<OutType>) {
    s.i = static_cast<std::int64_t>(init);
  } else if constexpr (std::is_same_v<OutType, bfloat16_t>) {
    const std::uint32_t u = (std::uint32_t)init.bits << 16;
    float f;
    __builtin_memcpy(&f, &u, 4);
    s.f = f;
  } else {
    s.f = to_double(init);
  }
  return s;
}

// One reduction call.  `res` may be null (pointer API): the stream alone is used.
template <typename InType,
          typename OutType,
          typename MainLambda,
          typename ReduceLambda,
          typename FinalLambda>
void reduce(const resources* res,
            hipStream_t stream,
            OutType* dots,
            const InType* data,
            std::int64_t n_rows,
            std::int64_t n_cols,
            bool row_major,
            bool along_rows,
            OutType init,
            bool inplace,
            const MainLambda& main_op,
            const ReduceLambda& reduce_op,
            const FinalLambda& final_op,
            int final_override         = -1,
            double scalar1             = 0.0,
            double scalar2             = 0.0,
            const void* final_aux      = nullptr,
            int out_dtype_override     = -1)
{
  // Functor and element types the library implements go through the C ABI; anything
  // else is instantiated in this translation unit when it is compiled by hipcc.
  constexpr bool lowered =
    cast_keeps_value<MainLambda, std::remove_cv_t<InType>>::value &&
    library_serves(dtype_of<std::remove_cv_t<InType>>::value,
                   dtype_of<std::remove_cv_t<OutType>>::value, main_tag<MainLambda>::value,
                   reduce_tag<ReduceLambda>::value, final_tag<FinalLambda>::value);
  if constexpr (!lowered) {
#if defined(__HIPCC__)
    (void)res;
    generic::reduce(stream, dots, data, n_rows, n_cols, row_major, along_rows, init, inplace,
                    main_op, reduce_op, final_op);
    return;
#else
    static_assert(main_tag<MainLambda>::value >= 0,
                  "main_op is not one of the functors the reduction library implements "
                  "(identity_op, cast_op, sq_op, abs_op, nz_op, value_to_kvp_op); compile this "
                  "translation unit with hipcc to use arbitrary device functors");
    static_assert(reduce_tag<ReduceLambda>::value >= 0,
                  "reduce_op is not one of add_op, max_op, min_op, argmax_op, argmin_op; compile "
                  "this translation unit with hipcc to use arbitrary device functors");
    static_assert(final_tag<FinalLambda>::value >= 0,
                  "final_op is not one of identity_op, sqrt_op, abs_op, sq_op, key_op, "
                  "mul/div/add/sub_const_op; compile this translation unit with hipcc to use "
                  "arbitrary device functors");
    static_assert(dtype_of<std::remove_cv_t<InType>>::value >= 0 &&
                    dtype_of<std::remove_cv_t<OutType>>::value >= 0,
                  "element type not supported by the reduction library; compile this translation "
                  "unit with hipcc to reduce arbitrary trivially copyable types");
    static_assert(always_false<MainLambda>,
                  "the reduction library has no kernel for this combination of element types and "
                  "functors (floating data into an integer output, max / min of integers into a "
                  "floating output, a cast_op that narrows or truncates, nz_op with a reduce_op "
                  "other than add_op, an arg-reduction whose output is not the matching "
                  "KeyValuePair or its key); compile this translation unit with hipcc");
#endif
  } else {
  rmi_reduce_desc d{};
  d.in_dtype      = dtype_of<std::remove_cv_t<InType>>::value;
  d.out_dtype     = out_dtype_override >= 0 ? out_dtype_override
                                            : dtype_of<std::remove_cv_t<OutType>>::value;
  d.layout        = row_major ? RMI_ROW_MAJOR : RMI_COL_MAJOR;
  d.apply         = along_rows ? RMI_ALONG_ROWS : RMI_ALONG_COLUMNS;
  d.n_rows        = n_rows;
  d.n_cols        = n_cols;
  d.main_op       = main_tag<MainLambda>::value;
  d.reduce_op     = reduce_tag<ReduceLambda>::value;
  d.final_op      = final_override >= 0 ? final_override : final_tag<FinalLambda>::value;
  d.inplace       = inplace ? 1 : 0;
  d.init          = make_init(init);
  d.final_scalar  = final_override >= 0 ? scalar1 : final_tag<FinalLambda>::scalar(final_op);
  d.final_scalar2 = scalar2;
  d.final_aux     = final_aux;
  d.plan_hint     = RMI_PLAN_AUTO;
  d.flags         = 0;
  const size_t ws_bytes = rmi_reduce_workspace_bytes(&d);
  workspace_lease ws(res, stream, ws_bytes);
  d.flags = ws.flags();
  check(rmi_reduce(&d, data, dots, ws.data(), ws.size(), stream), "rmi_reduce");
  (void)main_op;
  (void)reduce_op;
  }
}

}  // namespace detail::rmi
}  // namespace raft
