// TEST INFRASTRUCTURE — NOT PART OF THE PRODUCT.
//
// CPU restatement of the dense-reduction semantics of NVIDIA/raft, used only
// as the checker by tests/, __graft_entry__.smoke() and bench.py's
// cpu_baseline leg.  Nothing under raft_amd/ may link, load or call it.
//
// Two implementations of the same contract:
//   orc_reduce        sequential, every floating quantity in fp64, integers in
//                     int64: the oracle parity tests compare against.
//   orc_reduce_typed  OpenMP, arithmetic in the output type with the reference's
//                     Kahan-Babuska-Neumaier compensation for sums: the "OpenMP
//                     host implementation of the identical semantics" that
//                     bench.py times as the CPU baseline.
//
// Reference lines restated (paths relative to the reference's cpp/):
//   fold / init / inplace / final_op, 4 layout x axis combinations
//       tests/linalg/reduce.cuh:27-178 (naiveCoalescedReduction,
//       naiveStridedReduction, naiveReduction),
//       include/raft/linalg/detail/reduce.cuh:36-48
//   index passed to main_op = position along the reduced axis
//       include/raft/linalg/detail/coalesced_reduction-inl.cuh:96,
//       include/raft/linalg/detail/strided_reduction.cuh:42,103
//   functors: include/raft/core/operators.hpp:27-203 (identity, sq, abs, nz,
//       sqrt, add, min, max, argmin_op :187-194, argmax_op :196-203,
//       *_const_op :280-316)
//   KeyValuePair layout: include/raft/core/kvp.hpp:20-62
//   NaN-ignoring device max/min: include/raft/core/math.hpp:375-397,517-533
//   compensated sum: include/raft/linalg/detail/coalesced_reduction-inl.cuh:37-46
//   norms: include/raft/linalg/detail/norm.cuh:23-61
//   mean: include/raft/stats/detail/mean.cuh:19-40
//   stddev / vars epilogue: include/raft/stats/detail/stddev.cuh:46-59,91-101
//   map-then-reduce: include/raft/linalg/detail/map_then_reduce.cuh:47-95
//   arg-reduce, key-only output, init (0, -/+inf):
//       include/raft/matrix/detail/math.cuh:292-352
//   row normalisation: include/raft/linalg/detail/normalize.cuh:36-57,
//       include/raft/linalg/normalize.cuh:91-107
//   one-pass mean and variance: include/raft/stats/detail/meanvar.cuh:16-99
//   covariance: include/raft/stats/detail/cov.cuh:38-66 (mean-centre, then alpha * X^T X)
//
// Pinned by (tests/test_oracle.py): the closed-form fixtures of
// tests/linalg/reduce.cu:108-177, tests/matrix/argmax.cu:71-75,
// tests/matrix/argmin.cu:71-75, tests/util/reduction.cu:167-181,
// tests/core/operators_host.cpp:134-172, tests/stats/sum.cu:50-98,
// tests/stats/stddev.cu:139-150, tests/linalg/map_then_reduce.cu:140-169, and
// by numpy closed forms on random inputs (orc_meanvar: numpy's two-pass mean / var
// and the statistical tolerances of tests/stats/meanvar.cu:27-33; orc_cov: the 3 x 2
// known answer of tests/stats/cov.cu:88-100 and numpy.cov with both ddof in both layouts).  The summation ORDER of the
// reference's device kernels (CUB block reductions, float atomics) is not
// recoverable from its sources and is not pinned by its own tests either; both
// implementations here fix an order of their own.
#include <math.h>
#include <stdint.h>
#include <string.h>

#include <algorithm>
#include <limits>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

#include "rmi_reduce.h"

#define ORC_API extern "C" __attribute__((visibility("default")))

namespace {

// ---- storage types --------------------------------------------------------
struct f16 {
  uint16_t b;
};
struct bf16 {
  uint16_t b;
};

inline float half_to_float(uint16_t h)
{
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp        = (h >> 10) & 0x1f;
  uint32_t man        = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else {  // subnormal: normalise
      int e = -1;
      do {
        man <<= 1;
        ++e;
      } while (!(man & 0x400u));
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

inline uint16_t float_to_half(float f)
{
  uint32_t x;
  memcpy(&x, &f, 4);
  const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  x &= 0x7fffffffu;
  if (x >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (x > 0x7f800000u ? 0x200u : 0));
  if (x >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);  // rounds to inf
  if (x < 0x33000001u) return sign;                          // rounds to zero
  int exp       = (int)(x >> 23) - 127;
  uint32_t man  = (x & 0x7fffffu) | 0x800000u;
  int shift     = exp < -14 ? (13 + (-14 - exp)) : 13;
  uint32_t half = man >> shift;
  uint32_t rem  = man & ((1u << shift) - 1);
  uint32_t mid  = 1u << (shift - 1);
  if (rem > mid || (rem == mid && (half & 1))) ++half;
  if (exp < -14) return (uint16_t)(sign | half);
  return (uint16_t)(sign | (uint16_t)(((uint32_t)(exp + 15) << 10) + (half - 0x400u)));
}

inline float bf16_to_float(uint16_t b)
{
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}
inline uint16_t float_to_bf16(float f)
{
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

template <class T>
struct Elem {
  static double f64(T x) { return (double)x; }
  static int64_t i64(T x) { return (int64_t)x; }
};
template <>
struct Elem<f16> {
  static double f64(f16 x) { return (double)half_to_float(x.b); }
  static int64_t i64(f16) { return 0; }
};
template <>
struct Elem<bf16> {
  static double f64(bf16 x) { return (double)bf16_to_float(x.b); }
  static int64_t i64(bf16) { return 0; }
};

inline bool dt_is_float(int dt) { return dt >= RMI_F16 && dt <= RMI_F64; }
inline bool dt_is_int(int dt) { return dt >= RMI_I8 && dt <= RMI_I64; }
inline bool dt_is_kvp(int dt) { return dt >= RMI_KVP_I32_F32 && dt <= RMI_KVP_I64_F64; }

// Geometry of one reduction: output k, step r  ->  element index.
// linalg/detail/reduce.cuh:36-48 and tests/linalg/reduce.cuh:39-41,104-106.
struct Geometry {
  int64_t n_out, len, out_stride, red_stride;
};
inline Geometry geometry(const rmi_reduce_desc& d)
{
  const bool rm = d.layout == RMI_ROW_MAJOR, rows = d.apply == RMI_ALONG_ROWS;
  Geometry g;
  if (rows) {
    g.n_out = d.n_rows;
    g.len   = d.n_cols;
  } else {
    g.n_out = d.n_cols;
    g.len   = d.n_rows;
  }
  // element (i, j) lives at i*n_cols + j (row-major) or i + j*n_rows (col-major)
  const int64_t row_step = rm ? d.n_cols : 1, col_step = rm ? 1 : d.n_rows;
  g.out_stride = rows ? row_step : col_step;
  g.red_stride = rows ? col_step : row_step;
  return g;
}

// core/operators.hpp: identity_op, sq_op, abs_op, nz_op
inline double main_f(int op, double x)
{
  switch (op) {
    case RMI_MAIN_SQ: return x * x;
    case RMI_MAIN_ABS: return fabs(x);
    case RMI_MAIN_NZ: return x != 0.0 ? 1.0 : 0.0;
    default: return x;
  }
}
inline int64_t main_i(int op, int64_t x)
{
  switch (op) {
    case RMI_MAIN_SQ: return x * x;
    case RMI_MAIN_ABS: return x < 0 ? -x : x;
    case RMI_MAIN_NZ: return x != 0 ? 1 : 0;
    default: return x;
  }
}
// add_op / max_op / min_op; floating max/min ignore NaN like the device
// overloads of raft::max / raft::min (core/math.hpp:375-397,517-533).
inline double red_f(int op, double a, double b)
{
  switch (op) {
    case RMI_RED_MAX: return fmax(a, b);
    case RMI_RED_MIN: return fmin(a, b);
    default: return a + b;
  }
}
inline int64_t red_i(int op, int64_t a, int64_t b)
{
  switch (op) {
    case RMI_RED_MAX: return std::max(a, b);
    case RMI_RED_MIN: return std::min(a, b);
    default: return a + b;
  }
}
// sqrt_op, abs_op, sq_op, *_const_op; stddev.cuh:54-58 / :95-100 for VAR / STDDEV
inline double final_f(const rmi_reduce_desc& d, double x, double aux)
{
  switch (d.final_op) {
    case RMI_FIN_SQRT: return sqrt(x);
    case RMI_FIN_ABS: return fabs(x);
    case RMI_FIN_SQ: return x * x;
    case RMI_FIN_MUL_CONST: return x * d.final_scalar;
    case RMI_FIN_DIV_CONST: return x / d.final_scalar;
    case RMI_FIN_ADD_CONST: return x + d.final_scalar;
    case RMI_FIN_SUB_CONST: return x - d.final_scalar;
    case RMI_FIN_VAR_FROM_SUMSQ: return fabs(x * d.final_scalar - aux * aux * d.final_scalar2);
    case RMI_FIN_STDDEV_FROM_SUMSQ:
      return sqrt(fabs(x * d.final_scalar - aux * aux * d.final_scalar2));
    default: return x;
  }
}
inline int64_t final_i(const rmi_reduce_desc& d, int64_t x)
{
  const int64_t c = (int64_t)d.final_scalar;
  switch (d.final_op) {
    case RMI_FIN_ABS: return x < 0 ? -x : x;
    case RMI_FIN_SQ: return x * x;
    case RMI_FIN_MUL_CONST: return x * c;
    case RMI_FIN_DIV_CONST: return c != 0 ? x / c : 0;
    case RMI_FIN_ADD_CONST: return x + c;
    case RMI_FIN_SUB_CONST: return x - c;
    default: return x;
  }
}

// argmax_op / argmin_op, core/operators.hpp:187-203
struct Kvp {
  int64_t key;
  double value;
};
inline Kvp arg_op(bool is_max, Kvp a, Kvp b)
{
  const bool better = is_max ? (b.value > a.value) : (b.value < a.value);
  if (better || ((a.value == b.value) && (b.key < a.key))) return b;
  return a;
}

template <class T>
int reduce_seq(const rmi_reduce_desc& d,
               const T* in,
               const double* old_f,
               const int64_t* old_i,
               const double* aux_f,
               double* out_f,
               int64_t* out_i)
{
  const Geometry g = geometry(d);
  const bool arg   = d.reduce_op == RMI_RED_ARGMAX || d.reduce_op == RMI_RED_ARGMIN;
  if (arg) {
    if (d.main_op != RMI_MAIN_KVP) return RMI_ERR_UNSUPPORTED;
    const bool is_max = d.reduce_op == RMI_RED_ARGMAX;
    for (int64_t k = 0; k < g.n_out; ++k) {
      Kvp acc{d.init.i, d.init.f};
      for (int64_t r = 0; r < g.len; ++r) {
        const T x = in[k * g.out_stride + r * g.red_stride];
        acc       = arg_op(is_max, acc, Kvp{r, Elem<T>::f64(x)});
      }
      if (d.inplace) acc = arg_op(is_max, Kvp{old_i[k], old_f[k]}, acc);
      out_i[k] = acc.key;
      if (out_f) out_f[k] = acc.value;
    }
    return RMI_OK;
  }
  if (dt_is_float(d.out_dtype)) {
    for (int64_t k = 0; k < g.n_out; ++k) {
      double acc = d.init.f;
      for (int64_t r = 0; r < g.len; ++r)
        acc = red_f(d.reduce_op, acc,
                    main_f(d.main_op, Elem<T>::f64(in[k * g.out_stride + r * g.red_stride])));
      if (d.inplace) acc = red_f(d.reduce_op, old_f[k], acc);
      out_f[k] = final_f(d, acc, aux_f ? aux_f[k] : 0.0);
    }
    return RMI_OK;
  }
  if (dt_is_int(d.out_dtype)) {
    for (int64_t k = 0; k < g.n_out; ++k) {
      int64_t acc = d.init.i;
      for (int64_t r = 0; r < g.len; ++r)
        acc = red_i(d.reduce_op, acc,
                    main_i(d.main_op, Elem<T>::i64(in[k * g.out_stride + r * g.red_stride])));
      if (d.inplace) acc = red_i(d.reduce_op, old_i[k], acc);
      out_i[k] = final_i(d, acc);
    }
    return RMI_OK;
  }
  return RMI_ERR_UNSUPPORTED;
}

// ---------------------------------------------------------------------------
// Typed OpenMP implementation (CPU baseline).
// ---------------------------------------------------------------------------
template <class T>
struct OutArith {
  using type = T;
};
template <>
struct OutArith<f16> {
  using type = float;  // the reference's half functors compute in float
};
template <>
struct OutArith<bf16> {
  using type = float;
};

template <class A, class T>
inline A widen(T x)
{
  return (A)x;
}
template <>
inline float widen<float, f16>(f16 x)
{
  return half_to_float(x.b);
}
template <>
inline float widen<float, bf16>(bf16 x)
{
  return bf16_to_float(x.b);
}
template <>
inline double widen<double, f16>(f16 x)
{
  return (double)half_to_float(x.b);
}
template <>
inline double widen<double, bf16>(bf16 x)
{
  return (double)bf16_to_float(x.b);
}
template <>
inline int64_t widen<int64_t, f16>(f16)
{
  return 0;
}
template <>
inline int64_t widen<int64_t, bf16>(bf16)
{
  return 0;
}
template <>
inline int32_t widen<int32_t, f16>(f16)
{
  return 0;
}
template <>
inline int32_t widen<int32_t, bf16>(bf16)
{
  return 0;
}

template <class A>
inline A t_abs(A x)
{
  if constexpr (std::is_floating_point_v<A>) {
    return std::fabs(x);
  } else {
    return x < 0 ? -x : x;
  }
}
template <int MAIN, class A>
inline A t_main(A x)
{
  if constexpr (MAIN == RMI_MAIN_SQ) return x * x;
  if constexpr (MAIN == RMI_MAIN_ABS) return t_abs(x);
  if constexpr (MAIN == RMI_MAIN_NZ) return x != A(0) ? A(1) : A(0);
  return x;
}
template <class A>
inline A t_max(A a, A b)
{
  if constexpr (std::is_floating_point_v<A>) {
    return std::fmax(a, b);
  } else {
    return a > b ? a : b;
  }
}
template <class A>
inline A t_min(A a, A b)
{
  if constexpr (std::is_floating_point_v<A>) {
    return std::fmin(a, b);
  } else {
    return a < b ? a : b;
  }
}

// Accumulator in arithmetic type A; sums carry the reference's
// Kahan-Babuska-Neumaier compensation term (coalesced_reduction-inl.cuh:37-46),
// a no-op for integers.
template <int RED, class A>
struct TAcc {
  A s;
  A c;
  explicit TAcc(A init) : s(init), c(A(0)) {}
  inline void push(A x)
  {
    if constexpr (RED == RMI_RED_ADD) {
      if constexpr (std::is_floating_point_v<A>) {
        const A t = s + x;
        if (std::fabs(s) >= std::fabs(x)) {
          c += (s - t) + x;
        } else {
          c += (x - t) + s;
        }
        s = t;
      } else {
        s += x;
      }
    } else if constexpr (RED == RMI_RED_MAX) {
      s = t_max(s, x);
    } else {
      s = t_min(s, x);
    }
  }
  inline void merge(const TAcc& o)
  {
    push(o.s);
    if constexpr (RED == RMI_RED_ADD) c += o.c;
  }
  inline A value() const { return RED == RMI_RED_ADD ? (A)(s + c) : s; }
};

template <class A>
inline A t_final(const rmi_reduce_desc& d, A x, A aux)
{
  const A c1 = (A)d.final_scalar, c2 = (A)d.final_scalar2;
  switch (d.final_op) {
    case RMI_FIN_SQRT:
      if constexpr (std::is_floating_point_v<A>) return std::sqrt(x);
      return x;
    case RMI_FIN_ABS: return t_abs(x);
    case RMI_FIN_SQ: return x * x;
    case RMI_FIN_MUL_CONST: return x * c1;
    case RMI_FIN_DIV_CONST: return c1 != A(0) || std::is_floating_point_v<A> ? x / c1 : A(0);
    case RMI_FIN_ADD_CONST: return x + c1;
    case RMI_FIN_SUB_CONST: return x - c1;
    case RMI_FIN_VAR_FROM_SUMSQ: return t_abs((A)(x * c1 - aux * aux * c2));
    case RMI_FIN_STDDEV_FROM_SUMSQ:
      if constexpr (std::is_floating_point_v<A>) return std::sqrt(t_abs((A)(x * c1 - aux * aux * c2)));
      return x;
    default: return x;
  }
}

template <class O, class A>
inline O narrow(A x)
{
  return (O)x;
}
template <>
inline f16 narrow<f16, float>(float x)
{
  return f16{float_to_half(x)};
}
template <>
inline bf16 narrow<bf16, float>(float x)
{
  return bf16{float_to_bf16(x)};
}

template <class T, class O, int MAIN, int RED>
void typed_core(const rmi_reduce_desc& d, const T* in, O* out, const O* aux, int threads)
{
  using A          = typename OutArith<O>::type;
  const Geometry g = geometry(d);
  A init;
  if constexpr (std::is_floating_point_v<A>) {
    init = (A)d.init.f;
  } else {
    init = (A)d.init.i;
  }
  auto finish = [&](int64_t k, TAcc<RED, A> acc) {
    if (d.inplace) {
      TAcc<RED, A> o(widen<A>(out[k]));
      o.merge(acc);
      acc = o;
    }
    const A a = aux ? widen<A>(aux[k]) : A(0);
    out[k]    = narrow<O>(t_final<A>(d, acc.value(), a));
  };
  if (g.red_stride == 1) {
    // contiguous rows: one thread per block of outputs, static schedule
#pragma omp parallel for schedule(static) num_threads(threads)
    for (int64_t k = 0; k < g.n_out; ++k) {
      TAcc<RED, A> acc(init);
      const T* p = in + k * g.out_stride;
      for (int64_t r = 0; r < g.len; ++r)
        acc.push(t_main<MAIN>(widen<A>(p[r])));
      finish(k, acc);
    }
    return;
  }
  // strided: every thread folds a contiguous range of rows into its own
  // vector of accumulators; the vectors are merged in thread order.
  int nt = threads;
  if ((int64_t)nt > g.len) nt = (int)std::max<int64_t>(1, g.len);
  std::vector<std::vector<TAcc<RED, A>>> part(nt);
#pragma omp parallel num_threads(nt)
  {
#ifdef _OPENMP
    const int t = omp_get_thread_num();
#else
    const int t = 0;
#endif
    const int64_t r0 = g.len * t / nt, r1 = g.len * (t + 1) / nt;
    std::vector<TAcc<RED, A>> acc((size_t)g.n_out,
                                  TAcc<RED, A>(RED == RMI_RED_ADD ? A(0) : init));
    for (int64_t r = r0; r < r1; ++r) {
      const T* p = in + r * g.red_stride;
      for (int64_t k = 0; k < g.n_out; ++k)
        acc[k].push(t_main<MAIN>(widen<A>(p[k * g.out_stride])));
    }
    part[t] = std::move(acc);
  }
  for (int64_t k = 0; k < g.n_out; ++k) {
    TAcc<RED, A> acc(init);
    for (int t = 0; t < nt; ++t)
      acc.merge(part[t][k]);
    finish(k, acc);
  }
}

template <class T, class O>
int typed_ops(const rmi_reduce_desc& d, const T* in, O* out, const O* aux, int threads)
{
#define ORC_CASE(M, R)                                          \
  if (d.main_op == M && d.reduce_op == R) {                     \
    typed_core<T, O, M, R>(d, in, out, aux, threads);           \
    return RMI_OK;                                              \
  }
  ORC_CASE(RMI_MAIN_IDENTITY, RMI_RED_ADD)
  ORC_CASE(RMI_MAIN_SQ, RMI_RED_ADD)
  ORC_CASE(RMI_MAIN_ABS, RMI_RED_ADD)
  ORC_CASE(RMI_MAIN_NZ, RMI_RED_ADD)
  ORC_CASE(RMI_MAIN_IDENTITY, RMI_RED_MAX)
  ORC_CASE(RMI_MAIN_ABS, RMI_RED_MAX)
  ORC_CASE(RMI_MAIN_SQ, RMI_RED_MAX)
  ORC_CASE(RMI_MAIN_IDENTITY, RMI_RED_MIN)
  ORC_CASE(RMI_MAIN_ABS, RMI_RED_MIN)
  ORC_CASE(RMI_MAIN_SQ, RMI_RED_MIN)
#undef ORC_CASE
  return RMI_ERR_UNSUPPORTED;
}

// Row arg-reduce with {key, value} or key-only output (contiguous rows only,
// like the reference: matrix/detail/math.cuh:292-352 and the coalesced-only
// KVP cases of tests/linalg/reduce.cu:365-366).
template <class T, class V, class K>
int typed_arg(const rmi_reduce_desc& d, const T* in, void* out, int threads)
{
  const Geometry g = geometry(d);
  if (g.red_stride != 1) return RMI_ERR_UNSUPPORTED;
  const bool is_max   = d.reduce_op == RMI_RED_ARGMAX;
  const bool key_only = d.final_op == RMI_FIN_KEY;
  struct Pair {
    K key;
    V value;
  };
#pragma omp parallel for schedule(static) num_threads(threads)
  for (int64_t k = 0; k < g.n_out; ++k) {
    K bk       = (K)d.init.i;
    V bv       = (V)d.init.f;
    const T* p = in + k * g.out_stride;
    for (int64_t r = 0; r < g.len; ++r) {
      const V x         = widen<V>(p[r]);
      const bool better = is_max ? (x > bv) : (x < bv);
      if (better || (x == bv && (K)r < bk)) {
        bv = x;
        bk = (K)r;
      }
    }
    if (key_only) {
      static_cast<K*>(out)[k] = bk;
    } else {
      Pair* o = static_cast<Pair*>(out);
      if (d.inplace) {
        const V ov = o[k].value;
        const K ok = o[k].key;
        // red(old, acc): acc wins if better, or equal with the smaller key
        const bool better = is_max ? (bv > ov) : (bv < ov);
        if (!(better || (bv == ov && bk < ok))) {
          bv = ov;
          bk = ok;
        }
      }
      o[k].key   = bk;
      o[k].value = bv;
    }
  }
  return RMI_OK;
}

template <class T>
int typed_in(const rmi_reduce_desc& d, const T* in, void* out, const void* aux, int threads)
{
  const bool arg = d.reduce_op == RMI_RED_ARGMAX || d.reduce_op == RMI_RED_ARGMIN;
  if (arg) {
    if constexpr (std::is_same_v<T, float> || std::is_same_v<T, f16> || std::is_same_v<T, bf16>) {
      if (d.out_dtype == RMI_KVP_I32_F32 || (d.final_op == RMI_FIN_KEY && d.out_dtype == RMI_I32))
        return typed_arg<T, float, int32_t>(d, in, out, threads);
      if (d.out_dtype == RMI_KVP_I64_F32 || (d.final_op == RMI_FIN_KEY && d.out_dtype == RMI_I64))
        return typed_arg<T, float, int64_t>(d, in, out, threads);
    }
    if constexpr (std::is_same_v<T, double>) {
      if (d.out_dtype == RMI_KVP_I32_F64 || (d.final_op == RMI_FIN_KEY && d.out_dtype == RMI_I32))
        return typed_arg<T, double, int32_t>(d, in, out, threads);
      if (d.out_dtype == RMI_KVP_I64_F64 || (d.final_op == RMI_FIN_KEY && d.out_dtype == RMI_I64))
        return typed_arg<T, double, int64_t>(d, in, out, threads);
    }
    return RMI_ERR_UNSUPPORTED;
  }
  switch (d.out_dtype) {
    case RMI_F32: return typed_ops<T, float>(d, in, (float*)out, (const float*)aux, threads);
    case RMI_F64: return typed_ops<T, double>(d, in, (double*)out, (const double*)aux, threads);
    case RMI_F16: return typed_ops<T, f16>(d, in, (f16*)out, (const f16*)aux, threads);
    case RMI_BF16: return typed_ops<T, bf16>(d, in, (bf16*)out, (const bf16*)aux, threads);
    case RMI_I64:
      if constexpr (std::is_integral_v<T>)
        return typed_ops<T, int64_t>(d, in, (int64_t*)out, (const int64_t*)aux, threads);
      return RMI_ERR_UNSUPPORTED;
    case RMI_I32:
      if constexpr (std::is_integral_v<T>)
        return typed_ops<T, int32_t>(d, in, (int32_t*)out, (const int32_t*)aux, threads);
      return RMI_ERR_UNSUPPORTED;
    default: return RMI_ERR_UNSUPPORTED;
  }
}

}  // namespace

// Sequential fp64 / int64 oracle.
//   floating outputs : out_f[k] (old_f[k] read when inplace, aux_f[k] = mean for VAR/STDDEV)
//   integer outputs  : out_i[k] (old_i[k] when inplace)
//   arg reductions   : out_i[k] = key, out_f[k] = value (out_f may be NULL);
//                      old_i / old_f when inplace
ORC_API int orc_reduce(const rmi_reduce_desc* d,
                       const void* in,
                       const double* old_f,
                       const int64_t* old_i,
                       const double* aux_f,
                       double* out_f,
                       int64_t* out_i)
{
  if (!d) return RMI_ERR_NULL;
  switch (d->in_dtype) {
    case RMI_I8: return reduce_seq(*d, (const int8_t*)in, old_f, old_i, aux_f, out_f, out_i);
    case RMI_U8: return reduce_seq(*d, (const uint8_t*)in, old_f, old_i, aux_f, out_f, out_i);
    case RMI_I32: return reduce_seq(*d, (const int32_t*)in, old_f, old_i, aux_f, out_f, out_i);
    case RMI_I64: return reduce_seq(*d, (const int64_t*)in, old_f, old_i, aux_f, out_f, out_i);
    case RMI_F16: return reduce_seq(*d, (const f16*)in, old_f, old_i, aux_f, out_f, out_i);
    case RMI_BF16: return reduce_seq(*d, (const bf16*)in, old_f, old_i, aux_f, out_f, out_i);
    case RMI_F32: return reduce_seq(*d, (const float*)in, old_f, old_i, aux_f, out_f, out_i);
    case RMI_F64: return reduce_seq(*d, (const double*)in, old_f, old_i, aux_f, out_f, out_i);
    default: return RMI_ERR_UNSUPPORTED;
  }
}

// OpenMP implementation in the output's own arithmetic; `out` and `aux` are
// host arrays of d->out_dtype.  threads <= 0 uses omp_get_max_threads().
ORC_API int orc_reduce_typed(const rmi_reduce_desc* d,
                             const void* in,
                             void* out,
                             const void* aux,
                             int threads)
{
  if (!d) return RMI_ERR_NULL;
#ifdef _OPENMP
  if (threads <= 0) threads = omp_get_max_threads();
#else
  threads = 1;
#endif
  switch (d->in_dtype) {
    case RMI_I8: return typed_in(*d, (const int8_t*)in, out, aux, threads);
    case RMI_U8: return typed_in(*d, (const uint8_t*)in, out, aux, threads);
    case RMI_I32: return typed_in(*d, (const int32_t*)in, out, aux, threads);
    case RMI_I64: return typed_in(*d, (const int64_t*)in, out, aux, threads);
    case RMI_F16: return typed_in(*d, (const f16*)in, out, aux, threads);
    case RMI_BF16: return typed_in(*d, (const bf16*)in, out, aux, threads);
    case RMI_F32: return typed_in(*d, (const float*)in, out, aux, threads);
    case RMI_F64: return typed_in(*d, (const double*)in, out, aux, threads);
    default: return RMI_ERR_UNSUPPORTED;
  }
}

// Row normalisation in fp64: out[i, :] = in[i, :] / norm_i, rows with norm_i <= eps
// untouched (cpp/include/raft/linalg/detail/normalize.cuh:36-57); a row whose norm is NaN
// fails that test and is written (as NaN), like in the reference.  `out` holds the
// previous contents on entry, as doubles.
template <class T>
static int normalize_seq(const rmi_reduce_desc& d, const T* in, double* out, double eps)
{
  for (int64_t i = 0; i < d.n_rows; ++i) {
    double acc = d.init.f;
    for (int64_t j = 0; j < d.n_cols; ++j)
      acc = red_f(d.reduce_op, acc, main_f(d.main_op, Elem<T>::f64(in[i * d.n_cols + j])));
    const double norm = d.final_op == RMI_FIN_SQRT ? sqrt(acc) : acc;
    if (norm <= eps) continue;  // normalize.cuh:52,120: a NaN norm is not skipped
    for (int64_t j = 0; j < d.n_cols; ++j)
      out[i * d.n_cols + j] = Elem<T>::f64(in[i * d.n_cols + j]) / norm;
  }
  return RMI_OK;
}

ORC_API int orc_row_normalize(const rmi_reduce_desc* d, const void* in, double* out, double eps)
{
  if (!d) return RMI_ERR_NULL;
  switch (d->in_dtype) {
    case RMI_F16: return normalize_seq(*d, (const f16*)in, out, eps);
    case RMI_BF16: return normalize_seq(*d, (const bf16*)in, out, eps);
    case RMI_F32: return normalize_seq(*d, (const float*)in, out, eps);
    case RMI_F64: return normalize_seq(*d, (const double*)in, out, eps);
    default: return RMI_ERR_UNSUPPORTED;
  }
}

// Mean and variance of every column in one pass, fp64: the reference's mean_var
// monoid (cpp/include/raft/stats/detail/meanvar.cuh:16-99) applied element by element
// in row order.  Merging a state {w, m, s} with the singleton {1, x, 0} by its
// operator+= (:60-74): cw = w + 1; d = m - x; s += cw * (d * w/cw) * (d * 1/cw);
// m = m * w/cw + x * 1/cw.  var = s / max(1, sample ? w - 1 : w) (:88-98).
inline double as_double(float x) { return (double)x; }
inline double as_double(double x) { return x; }
inline double as_double(f16 x) { return (double)half_to_float(x.b); }
inline double as_double(bf16 x) { return (double)bf16_to_float(x.b); }

template <class T>
static int meanvar_seq(int layout, int64_t n_rows, int64_t n_cols, int sample, const T* in,
                       double* mean, double* var)
{
  for (int64_t j = 0; j < n_cols; ++j) {
    double w = 0.0, m = 0.0, s = 0.0;
    for (int64_t i = 0; i < n_rows; ++i) {
      const double x  = as_double(layout == RMI_ROW_MAJOR ? in[i * n_cols + j] : in[j * n_rows + i]);
      const double cw = w + 1.0;
      const double fa = w / cw, fb = 1.0 / cw;
      const double d  = m - x;
      s += cw * (d * fa) * (d * fb);
      m = m * fa + x * fb;
      w = cw;
    }
    mean[j] = m;
    var[j]  = s / std::max(1.0, sample ? w - 1.0 : w);
  }
  return RMI_OK;
}

ORC_API int orc_meanvar(int dtype, int layout, int64_t n_rows, int64_t n_cols, int sample,
                        const void* in, double* mean, double* var)
{
  if (layout != RMI_ROW_MAJOR && layout != RMI_COL_MAJOR) return RMI_ERR_BAD_ENUM;
  switch (dtype) {
    case RMI_F32: return meanvar_seq(layout, n_rows, n_cols, sample, (const float*)in, mean, var);
    case RMI_F64: return meanvar_seq(layout, n_rows, n_cols, sample, (const double*)in, mean, var);
    case RMI_F16: return meanvar_seq(layout, n_rows, n_cols, sample, (const f16*)in, mean, var);
    case RMI_BF16: return meanvar_seq(layout, n_rows, n_cols, sample, (const bf16*)in, mean, var);
    default: return RMI_ERR_UNSUPPORTED;
  }
}

// Covariance around a given mean vector, as the reference computes it
// (cpp/include/raft/stats/detail/cov.cuh:49-60): the data is mean-centred in its own type
// (meanCenter, stats/detail/mean_center.cuh: data[n][j] - mu[j] rounded to Type), then
// covar = alpha * X^T X with alpha = Type(1) / Type(sample ? N - 1 : N).  The products and
// sums of the GEMM are restated in fp64 (the reference's order inside cuBLAS is not
// recoverable); `centered`, when given, receives the centred data in the input's type, which
// is what the reference leaves in `data`.  covar is [D][D], symmetric.
template <class T>
static int cov_seq(int layout, int64_t N, int64_t D, int sample, const T* in, const T* mu,
                   double* covar, T* centered)
{
  std::vector<T> c((size_t)N * D);  // centred, row-major [N][D]
  for (int64_t n = 0; n < N; ++n)
    for (int64_t j = 0; j < D; ++j) {
      const T x = layout == RMI_ROW_MAJOR ? in[n * D + j] : in[j * N + n];
      const T d = mu != nullptr ? (T)(x - mu[j]) : x;
      c[n * D + j] = d;
      if (centered != nullptr) centered[layout == RMI_ROW_MAJOR ? n * D + j : j * N + n] = d;
    }
  const double alpha = N == 0 ? 0.0 : (double)(T(1) / (sample ? T(N - 1) : T(N)));
#pragma omp parallel for schedule(dynamic, 1)
  for (int64_t i = 0; i < D; ++i)
    for (int64_t j = i; j < D; ++j) {
      double s = 0.0;
      for (int64_t n = 0; n < N; ++n)
        s += (double)c[n * D + i] * (double)c[n * D + j];
      covar[i * D + j] = covar[j * D + i] = s * alpha;
    }
  return RMI_OK;
}

ORC_API int orc_cov(int dtype, int layout, int64_t n_rows, int64_t n_cols, int sample,
                    const void* in, const void* mu, double* covar, void* centered)
{
  if (layout != RMI_ROW_MAJOR && layout != RMI_COL_MAJOR) return RMI_ERR_BAD_ENUM;
  switch (dtype) {
    case RMI_F32:
      return cov_seq(layout, n_rows, n_cols, sample, (const float*)in, (const float*)mu, covar,
                     (float*)centered);
    case RMI_F64:
      return cov_seq(layout, n_rows, n_cols, sample, (const double*)in, (const double*)mu, covar,
                     (double*)centered);
    default: return RMI_ERR_UNSUPPORTED;
  }
}

ORC_API int orc_max_threads(void)
{
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

// Storage conversions, exposed so tests can build f16 / bf16 inputs and read
// such outputs without a second implementation of the rounding rules.
ORC_API void orc_f32_to_bf16(const float* src, uint16_t* dst, int64_t n)
{
  for (int64_t i = 0; i < n; ++i)
    dst[i] = float_to_bf16(src[i]);
}
ORC_API void orc_bf16_to_f32(const uint16_t* src, float* dst, int64_t n)
{
  for (int64_t i = 0; i < n; ++i)
    dst[i] = bf16_to_float(src[i]);
}
ORC_API void orc_f32_to_f16(const float* src, uint16_t* dst, int64_t n)
{
  for (int64_t i = 0; i < n; ++i)
    dst[i] = float_to_half(src[i]);
}
ORC_API void orc_f16_to_f32(const uint16_t* src, float* dst, int64_t n)
{
  for (int64_t i = 0; i < n; ++i)
    dst[i] = half_to_float(src[i]);
}
