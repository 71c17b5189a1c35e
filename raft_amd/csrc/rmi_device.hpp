// Device-side building blocks for the gfx950 reduction kernels: 16-byte
// lane loads, element unpacking, accumulator policies (what main_op /
// reduce_op mean for one input type), wave64 cross-lane reductions and the
// per-output epilogue (init, inplace merge, final_op, store).
//
// Everything here is wave64 / CDNA4 specific by design: DPP row operations
// for lane distances below 16, ds_bpermute for 16 and 32.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "rmi_reduce.h"

namespace rmi {

using u32   = uint32_t;
using u64   = uint64_t;
using i64   = int64_t;
using u32x4 = u32 __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;

// Tag type for bfloat16 storage (1 sign, 8 exponent, 7 mantissa bits).
struct bf16_t {
  uint16_t bits;
};
// IEEE binary16 storage.
using f16_t = _Float16;

// ---------------------------------------------------------------------------
// Loads
// ---------------------------------------------------------------------------
// 16 bytes at any byte address: gfx950 runs global memory in unaligned access
// mode, so one global_load_dwordx4 serves aligned and unaligned addresses alike.
typedef u32x4 u32x4_unaligned __attribute__((aligned(1)));

__device__ __forceinline__ u32x4 load16(const void* p)
{
  // One global_load_dwordx4 per lane; streamed once, so mark it non-temporal.
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4_unaligned*>(p));
}

__device__ __forceinline__ float as_f32(u32 w) { return __uint_as_float(w); }
__device__ __forceinline__ u32 as_u32(float f) { return __float_as_uint(f); }

// Per input type: elements per 16-byte vector, the "natural" register type an
// element is widened to on unpack, and how to pull element J out of a vector.
template <class T>
struct In;

template <>
struct In<float> {
  static constexpr int VEC = 4;
  using nat                = float;
  template <int J>
  static __device__ __forceinline__ nat get(const u32x4& v)
  {
    return as_f32(v[J]);
  }
  static __device__ __forceinline__ nat ld(const float* p) { return __builtin_nontemporal_load(p); }
};

template <>
struct In<double> {
  static constexpr int VEC = 2;
  using nat                = double;
  template <int J>
  static __device__ __forceinline__ nat get(const u32x4& v)
  {
    typedef double f64x2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(f64x2, v)[J];
  }
  static __device__ __forceinline__ nat ld(const double* p)
  {
    return __builtin_nontemporal_load(p);
  }
};

template <>
struct In<f16_t> {
  static constexpr int VEC = 8;
  using nat                = float;
  static __device__ __forceinline__ nat cvt(uint16_t h)
  {
    f16_t x;
    __builtin_memcpy(&x, &h, 2);
    return (float)x;
  }
  template <int J>
  static __device__ __forceinline__ nat get(const u32x4& v)
  {
    u32 w = v[J / 2];
    return cvt((J & 1) ? (uint16_t)(w >> 16) : (uint16_t)(w & 0xffffu));
  }
  static __device__ __forceinline__ nat ld(const f16_t* p) { return (float)*p; }
};

template <>
struct In<bf16_t> {
  static constexpr int VEC = 8;
  using nat                = float;
  template <int J>
  static __device__ __forceinline__ nat get(const u32x4& v)
  {
    u32 w = v[J / 2];
    // bf16 -> f32 is a 16-bit left shift of the storage bits.
    return (J & 1) ? as_f32(w & 0xffff0000u) : as_f32(w << 16);
  }
  static __device__ __forceinline__ nat ld(const bf16_t* p) { return as_f32((u32)p->bits << 16); }
};

template <>
struct In<int8_t> {
  static constexpr int VEC = 16;
  using nat                = int32_t;
  template <int J>
  static __device__ __forceinline__ nat get(const u32x4& v)
  {
    return __builtin_amdgcn_sbfe((int)v[J / 4], 8 * (J & 3), 8);
  }
  static __device__ __forceinline__ nat ld(const int8_t* p) { return (int32_t)*p; }
};

template <>
struct In<uint8_t> {
  static constexpr int VEC = 16;
  using nat                = int32_t;
  template <int J>
  static __device__ __forceinline__ nat get(const u32x4& v)
  {
    return (int32_t)__builtin_amdgcn_ubfe(v[J / 4], 8 * (J & 3), 8);
  }
  static __device__ __forceinline__ nat ld(const uint8_t* p) { return (int32_t)*p; }
};

template <>
struct In<int32_t> {
  static constexpr int VEC = 4;
  using nat                = int32_t;
  template <int J>
  static __device__ __forceinline__ nat get(const u32x4& v)
  {
    return (int32_t)v[J];
  }
  static __device__ __forceinline__ nat ld(const int32_t* p) { return *p; }
};

template <>
struct In<int64_t> {
  static constexpr int VEC = 2;
  using nat                = int64_t;
  template <int J>
  static __device__ __forceinline__ nat get(const u32x4& v)
  {
    typedef int64_t i64x2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(i64x2, v)[J];
  }
  static __device__ __forceinline__ nat ld(const int64_t* p) { return *p; }
};

// ---------------------------------------------------------------------------
// Cross-lane exchange
// ---------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ u32 dpp_word(u32 v)
{
  return (u32)__builtin_amdgcn_update_dpp((int)v, (int)v, CTRL, 0xF, 0xF, false);
}

// Exchange a 4- or 8-byte scalar with another lane; SEL picks the pattern:
//   0: lane^1   (quad_perm [1,0,3,2])
//   1: lane^2   (quad_perm [2,3,0,1])
//   2: 7-lane within each 8 lanes (row_half_mirror)
//   3: 15-lane within each 16 lanes (row_mirror)
//   4: lane^16  (ds_bpermute)
//   5: lane^32  (ds_bpermute)
// After steps 0 and 1 all four lanes of a quad hold the same value, so the two
// mirror steps pair each lane with a lane of the *other* quad / half-row,
// which is all a commutative all-reduce needs.
template <int SEL>
__device__ __forceinline__ u32 xchg_word(u32 v)
{
  if constexpr (SEL == 0) return dpp_word<0xB1>(v);
  if constexpr (SEL == 1) return dpp_word<0x4E>(v);
  if constexpr (SEL == 2) return dpp_word<0x141>(v);
  if constexpr (SEL == 3) return dpp_word<0x140>(v);
  if constexpr (SEL == 4) return (u32)__shfl_xor((int)v, 16, kWave);
  if constexpr (SEL == 5) return (u32)__shfl_xor((int)v, 32, kWave);
  return v;
}

template <int SEL, class T>
__device__ __forceinline__ T xchg(T v)
{
  static_assert(sizeof(T) == 4 || sizeof(T) == 8, "xchg moves 4- or 8-byte scalars");
  if constexpr (sizeof(T) == 4) {
    u32 w;
    __builtin_memcpy(&w, &v, 4);
    w = xchg_word<SEL>(w);
    T r;
    __builtin_memcpy(&r, &w, 4);
    return r;
  } else {
    u64 w;
    __builtin_memcpy(&w, &v, 8);
    u32 lo = xchg_word<SEL>((u32)w);
    u32 hi = xchg_word<SEL>((u32)(w >> 32));
    w      = ((u64)hi << 32) | lo;
    T r;
    __builtin_memcpy(&r, &w, 8);
    return r;
  }
}

// ---------------------------------------------------------------------------
// Accumulator policies
// ---------------------------------------------------------------------------
// A policy P provides
//   in_t, acc_t, VEC
//   neutral()                      identity element of the fold
//   push(acc, nat x, idx)          acc = reduce_op(acc, main_op(x, idx))
//   push_vec(acc, u32x4 v, idx0)   the same for the VEC elements of a vector
//   push_cols(acc[VEC], v, idx)    element j goes to acc[j] (column plans)
//   merge(acc, other)              acc = reduce_op(acc, other)
//   exchange<SEL>(acc)             acc of the partner lane
//   from_scalar(f, i), from_out(p, dtype, k), result/store: see Epilogue.
// merge must be exactly commutative (bitwise) for results to be independent of the
// lane a result is read from (PolMeanVar is commutative up to rounding only: its
// results are valid from any lane but not bitwise equal across lanes).

enum : int { kClsFloat = 0, kClsInt = 1, kClsKvp = 2, kClsMeanVar = 3 };
enum : int { kTailEach = 0, kTailZero = 1, kTailDup = 2 };

template <int MAIN>
__device__ __forceinline__ double main_f64(double d)
{
  if constexpr (MAIN == RMI_MAIN_SQ) return d * d;
  if constexpr (MAIN == RMI_MAIN_ABS) return fabs(d);
  if constexpr (MAIN == RMI_MAIN_NZ) return d != 0.0 ? 1.0 : 0.0;
  return d;
}

template <int MAIN>
__device__ __forceinline__ i64 main_i64(i64 x)
{
  if constexpr (MAIN == RMI_MAIN_SQ) return x * x;
  if constexpr (MAIN == RMI_MAIN_ABS) return x < 0 ? -x : x;
  if constexpr (MAIN == RMI_MAIN_NZ) return x != 0 ? 1 : 0;
  return x;
}

template <int MAIN>
__device__ __forceinline__ int32_t main_i32(int32_t x)
{
  if constexpr (MAIN == RMI_MAIN_SQ) return x * x;
  if constexpr (MAIN == RMI_MAIN_ABS) return x < 0 ? -x : x;
  if constexpr (MAIN == RMI_MAIN_NZ) return x != 0 ? 1 : 0;
  return x;
}

template <int N, class F>
__device__ __forceinline__ void static_for(F&& f)
{
  if constexpr (N > 0) {
    static_for<N - 1>(f);
    f(std::integral_constant<int, N - 1>{});
  }
}

// ---- floating accumulators: plain double ---------------------------------
// Inputs of at most 32 bits (f16, bf16, f32, and integers up to 32 bits feeding
// a floating output) are summed in f64: every product and partial sum of such
// inputs carries >= 29 spare mantissa bits, which serves the purpose of the
// reference's per-thread Kahan-Babuska-Neumaier compensation
// (linalg/detail/coalesced_reduction-inl.cuh:37-46) at a third of the ALU cost.
template <class InT, int MAIN, int RED>
struct PolI;

template <class InT, int MAIN, int RED>
struct PolF {
  using in_t               = InT;
  using nat                = typename In<InT>::nat;
  using acc_t              = double;
  static constexpr int VEC = In<InT>::VEC;
  static constexpr int CLS = kClsFloat;
  static constexpr int kMain = MAIN;
  static constexpr int kRed  = RED;
  // How the overlapping last vector of a row (its first VEC - tail elements were already
  // counted) is folded: kTailZero: those elements are zeroed and the vector is pushed whole
  // (sums: every main op maps 0 to 0); kTailDup: the vector is pushed whole as it is (min,
  // max and arg-reductions do not change when an element is seen twice); kTailEach: element
  // by element.
  static constexpr int kTail = RED == RMI_RED_ADD ? kTailZero : kTailDup;

  static __device__ __forceinline__ acc_t neutral()
  {
    if constexpr (RED == RMI_RED_MAX) return -__builtin_inf();
    if constexpr (RED == RMI_RED_MIN) return __builtin_inf();
    return 0.0;
  }
  static __device__ __forceinline__ double red(double a, double b)
  {
    if constexpr (RED == RMI_RED_MAX) return fmax(a, b);
    if constexpr (RED == RMI_RED_MIN) return fmin(a, b);
    return a + b;
  }
  static __device__ __forceinline__ void push(acc_t& a, nat x, i64)
  {
    a = red(a, main_f64<MAIN>((double)x));
  }
  // Sums of bytes into a floating output: the terms are small integers, so a vector is folded
  // in 32-bit integer arithmetic (the dot-product instructions of PolI) and column terms gather
  // in 32-bit accumulators; both are exact, and so is every f64 sum of them below 2^53.
  static constexpr bool kBytes     = sizeof(InT) == 1 && RED == RMI_RED_ADD;
  static constexpr bool kColNarrow = kBytes;
  static constexpr int kColFlush   = 128;
  static __device__ __forceinline__ void push_cols_narrow(int32_t (&a)[VEC], const u32x4& v)
  {
    static_for<VEC>([&](auto j) { a[j] += main_i32<MAIN>((int32_t)In<InT>::template get<j>(v)); });
  }
  static __device__ __forceinline__ void push_vec(acc_t& a, const u32x4& v, i64)
  {
    if constexpr (kBytes) {
      a += (double)PolI<InT, MAIN, RMI_RED_ADD>::vec_i32(v);
      return;
    }
    // Pairwise tree inside the vector (fixed order, so results do not depend
    // on the launch plan's scheduling), then one dependent step into `a`.
    double t[VEC];
    static_for<VEC>([&](auto j) { t[j] = main_f64<MAIN>((double)In<InT>::template get<j>(v)); });
#pragma unroll
    for (int w = VEC / 2; w >= 1; w /= 2) {
#pragma unroll
      for (int j = 0; j < w; ++j)
        t[j] = red(t[j], t[j + w]);
    }
    a = red(a, t[0]);
  }
  static __device__ __forceinline__ void push_cols(acc_t (&a)[VEC], const u32x4& v, i64)
  {
    static_for<VEC>(
      [&](auto j) { a[j] = red(a[j], main_f64<MAIN>((double)In<InT>::template get<j>(v))); });
  }
  static __device__ __forceinline__ void merge(acc_t& a, const acc_t& b) { a = red(a, b); }
  template <int SEL>
  static __device__ __forceinline__ acc_t exchange(const acc_t& a)
  {
    return xchg<SEL>(a);
  }
  static __device__ __forceinline__ acc_t from_f64(double f) { return f; }
  static __device__ __forceinline__ double to_f64(const acc_t& a) { return a; }
};

// ---- floating accumulators: f64 with Kahan-Babuska-Neumaier compensation ---
// Used when the input itself is f64 and the fold is a sum: restates the
// reference's compensated sum (linalg/detail/coalesced_reduction-inl.cuh:37-46)
// and, unlike it, also carries the compensation term through every cross-lane
// and cross-block merge.
struct kbn_t {
  double s;
  double c;
};

// One compensated step.  The reference picks between (s - t) + x and (x - t) + s by
// comparing magnitudes; both are the exact rounding error of s + x.  Knuth's
// branch-free two-sum yields the same exact error with two more additions and no
// compare / select, which is cheaper on the f64 pipe.
__device__ __forceinline__ double two_sum_err(double s, double x, double t)
{
  const double bp = t - s;
  return (s - (t - bp)) + (x - bp);
}

__device__ __forceinline__ void kbn_add(kbn_t& a, double x)
{
  const double t = a.s + x;
  a.c += two_sum_err(a.s, x, t);
  a.s = t;
}

template <class InT, int MAIN>
struct PolKbn {
  using in_t               = InT;
  using nat                = typename In<InT>::nat;
  using acc_t              = kbn_t;
  static constexpr int VEC = In<InT>::VEC;
  static constexpr int CLS = kClsFloat;
  static constexpr int kMain = MAIN;
  static constexpr int kRed  = RMI_RED_ADD;
  static constexpr int kTail = kTailZero;

  static __device__ __forceinline__ acc_t neutral() { return kbn_t{0.0, 0.0}; }
  static __device__ __forceinline__ void push(acc_t& a, nat x, i64)
  {
    kbn_add(a, main_f64<MAIN>((double)x));
  }
  static __device__ __forceinline__ void push_vec(acc_t& a, const u32x4& v, i64)
  {
    static_for<VEC>([&](auto j) { push(a, In<InT>::template get<j>(v), 0); });
  }
  static __device__ __forceinline__ void push_cols(acc_t (&a)[VEC], const u32x4& v, i64)
  {
    static_for<VEC>([&](auto j) { push(a[j], In<InT>::template get<j>(v), 0); });
  }
  static __device__ __forceinline__ void merge(acc_t& a, const acc_t& b)
  {
    const double t = a.s + b.s;
    const double e = two_sum_err(a.s, b.s, t);
    a.c            = (a.c + b.c) + e;
    a.s            = t;
  }
  template <int SEL>
  static __device__ __forceinline__ acc_t exchange(const acc_t& a)
  {
    return kbn_t{xchg<SEL>(a.s), xchg<SEL>(a.c)};
  }
  static __device__ __forceinline__ acc_t from_f64(double f) { return kbn_t{f, 0.0}; }
  static __device__ __forceinline__ double to_f64(const acc_t& a) { return a.s + a.c; }
};

// ---- integer accumulators: int64 ------------------------------------------
template <class InT, int MAIN, int RED>
struct PolI {
  using in_t               = InT;
  using nat                = typename In<InT>::nat;
  using acc_t              = i64;
  static constexpr int VEC = In<InT>::VEC;
  static constexpr int CLS = kClsInt;
  static constexpr int kTail = RED == RMI_RED_ADD ? kTailZero : kTailDup;
  // 8-bit inputs: fold a whole vector in 32 bits first (16 terms of at most
  // 2^14 cannot overflow), then widen once.
  static constexpr bool kNarrow = sizeof(InT) == 1;

  static __device__ __forceinline__ acc_t neutral()
  {
    if constexpr (RED == RMI_RED_MAX) return INT64_MIN;
    if constexpr (RED == RMI_RED_MIN) return INT64_MAX;
    return 0;
  }
  template <class T>
  static __device__ __forceinline__ T red(T a, T b)
  {
    if constexpr (RED == RMI_RED_MAX) return a > b ? a : b;
    if constexpr (RED == RMI_RED_MIN) return a < b ? a : b;
    return a + b;
  }
  static __device__ __forceinline__ void push(acc_t& a, nat x, i64)
  {
    a = red<i64>(a, main_i64<MAIN>((i64)x));
  }
  // main_op of the four bytes of one word, folded in 32 bits (kNarrow inputs only)
  static __device__ __forceinline__ int32_t word_i32(u32 w)
  {
    if constexpr (RED == RMI_RED_ADD && std::is_same_v<InT, int8_t> &&
                  (MAIN == RMI_MAIN_IDENTITY || MAIN == RMI_MAIN_SQ)) {
      // v_dot4_i32_i8: four signed byte products per instruction.
      const int x = (int)w;
      return __builtin_amdgcn_sdot4(x, MAIN == RMI_MAIN_SQ ? x : 0x01010101, 0, false);
    } else if constexpr (RED == RMI_RED_ADD && std::is_same_v<InT, uint8_t> &&
                         (MAIN == RMI_MAIN_IDENTITY || MAIN == RMI_MAIN_ABS ||
                          MAIN == RMI_MAIN_SQ)) {
      return (int32_t)__builtin_amdgcn_udot4(w, MAIN == RMI_MAIN_SQ ? w : 0x01010101u, 0u, false);
    } else if constexpr (RED == RMI_RED_ADD && std::is_same_v<InT, int8_t> &&
                         MAIN == RMI_MAIN_ABS) {
      // |x| summed with v_sad_u8 after biasing signed bytes to unsigned.
      return (int32_t)__builtin_amdgcn_sad_u8(w ^ 0x80808080u, 0x80808080u, 0u);
    } else {
      int32_t t[4];
      static_for<4>([&](auto j) {
        if constexpr (std::is_same_v<InT, int8_t>)
          t[j] = main_i32<MAIN>(__builtin_amdgcn_sbfe((int)w, 8 * j, 8));
        else
          t[j] = main_i32<MAIN>((int32_t)__builtin_amdgcn_ubfe(w, 8 * j, 8));
      });
      return red<int32_t>(red<int32_t>(t[0], t[1]), red<int32_t>(t[2], t[3]));
    }
  }
  static __device__ __forceinline__ int32_t vec_i32(const u32x4& v)
  {
    if constexpr (RED == RMI_RED_ADD) {
      // dot products chain their accumulator: one instruction per word
      if constexpr (std::is_same_v<InT, int8_t> && (MAIN == RMI_MAIN_IDENTITY || MAIN == RMI_MAIN_SQ)) {
        int32_t s = 0;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const int x = (int)v[w];
          s = __builtin_amdgcn_sdot4(x, MAIN == RMI_MAIN_SQ ? x : 0x01010101, s, false);
        }
        return s;
      } else if constexpr (std::is_same_v<InT, uint8_t> &&
                           (MAIN == RMI_MAIN_IDENTITY || MAIN == RMI_MAIN_ABS || MAIN == RMI_MAIN_SQ)) {
        int32_t s = 0;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const u32 x = v[w];
          s = (int32_t)__builtin_amdgcn_udot4(x, MAIN == RMI_MAIN_SQ ? x : 0x01010101u, (u32)s, false);
        }
        return s;
      } else if constexpr (std::is_same_v<InT, int8_t> && MAIN == RMI_MAIN_ABS) {
        u32 s = 0;
#pragma unroll
        for (int w = 0; w < 4; ++w)
          s = __builtin_amdgcn_sad_u8(v[w] ^ 0x80808080u, 0x80808080u, s);
        return (int32_t)s;
      }
    }
    return red<int32_t>(red<int32_t>(word_i32(v[0]), word_i32(v[1])),
                        red<int32_t>(word_i32(v[2]), word_i32(v[3])));
  }
  static __device__ __forceinline__ void push_vec(acc_t& a, const u32x4& v, i64)
  {
    if constexpr (kNarrow) {
      a = red<i64>(a, (i64)vec_i32(v));
    } else {
      static_for<VEC>([&](auto j) { push(a, In<InT>::template get<j>(v), 0); });
    }
  }
  static __device__ __forceinline__ void push_cols(acc_t (&a)[VEC], const u32x4& v, i64)
  {
    static_for<VEC>([&](auto j) { push(a[j], In<InT>::template get<j>(v), 0); });
  }
  // Column sums of 8-bit elements gather in 32-bit accumulators (one add per byte where a
  // 64-bit one costs three) and are emptied into the 64-bit ones every kColFlush lane-loads
  // (2 % more instructions): a term is at most 2^14 (a squared byte), so 128 of them stay far
  // below 2^31, and matrices of a few hundred MB already pass through the emptying step.
  static constexpr bool kColNarrow = kNarrow && RED == RMI_RED_ADD;
  static constexpr int kColFlush   = 128;
  static __device__ __forceinline__ void push_cols_narrow(int32_t (&a)[VEC], const u32x4& v)
  {
    static_for<VEC>([&](auto j) { a[j] += main_i32<MAIN>((int32_t)In<InT>::template get<j>(v)); });
  }
  static __device__ __forceinline__ void merge(acc_t& a, const acc_t& b) { a = red<i64>(a, b); }
  template <int SEL>
  static __device__ __forceinline__ acc_t exchange(const acc_t& a)
  {
    return xchg<SEL>(a);
  }
};

// ---- key-value accumulators: arg-max / arg-min ------------------------------
// Rule of raft::argmax_op / argmin_op (core/operators.hpp:187-203): the
// candidate wins if its value is strictly better, or equal with a smaller key.
// NaN never compares true, so NaN never wins (same as the reference).
template <class KeyT, class ValT>
struct kvp_t {
  KeyT key;
  ValT value;
};

template <class InT, class KeyT, bool IS_MAX>
struct PolKvp {
  using in_t               = InT;
  using nat                = typename In<InT>::nat;
  using val_t              = nat;  // float for f16/bf16/f32 inputs, double for f64
  using acc_t              = kvp_t<KeyT, val_t>;
  static constexpr int VEC = In<InT>::VEC;
  static constexpr int CLS = kClsKvp;
  static constexpr int kTail = kTailDup;
  static constexpr KeyT kKeyMax = sizeof(KeyT) == 4 ? (KeyT)INT32_MAX : (KeyT)INT64_MAX;

  static __device__ __forceinline__ acc_t neutral()
  {
    return acc_t{kKeyMax, IS_MAX ? (val_t)-__builtin_inf() : (val_t)__builtin_inf()};
  }
  static __device__ __forceinline__ void take(acc_t& a, KeyT k, val_t x)
  {
    const bool better = IS_MAX ? (x > a.value) : (x < a.value);
    const bool win    = better || ((x == a.value) && (k < a.key));
    a.value           = win ? x : a.value;
    a.key             = win ? k : a.key;
  }
  static __device__ __forceinline__ void push(acc_t& a, nat x, i64 idx) { take(a, (KeyT)idx, x); }
  static __device__ __forceinline__ void push_vec(acc_t& a, const u32x4& v, i64 idx0)
  {
    const KeyT k0 = (KeyT)idx0;
    static_for<VEC>([&](auto j) { take(a, (KeyT)(k0 + j), In<InT>::template get<j>(v)); });
  }
  // A batch of vectors that a lane holds in registers is scanned from its highest index down.
  // Every candidate's key is then below the holder's, so the rule shrinks to "not worse"
  // (`>=` for arg-max): a compare and two selects per element where `take` needs seven
  // instructions, and the key that travels is the element's slot in the batch, a constant of
  // the instruction.  An element met twice (the overlapping last vector of a row) is harmless
  // as long as the last visits go down in index.  The batch's winner then enters the
  // accumulator under the full rule; a batch of NaNs only has no winner (slot -1).
  struct scan_t {
    int slot;
    val_t value;
  };
  static __device__ __forceinline__ scan_t scan_begin() { return scan_t{-1, neutral().value}; }
  template <int SLOT0>
  static __device__ __forceinline__ void scan_vec(scan_t& s, const u32x4& v)
  {
    static_for<VEC>([&](auto jj) {
      constexpr int j = VEC - 1 - decltype(jj)::value;
      const val_t x   = In<InT>::template get<j>(v);
      const bool win  = IS_MAX ? (x >= s.value) : (x <= s.value);
      s.value         = win ? x : s.value;
      s.slot          = win ? SLOT0 + j : s.slot;
    });
  }
  // `key`: the index of the element in slot s.slot.  FRESH: the accumulator is known to be the
  // neutral one, which the winner replaces.
  template <bool FRESH = false>
  static __device__ __forceinline__ void scan_end(acc_t& a, const scan_t& s, KeyT key)
  {
    const KeyT k = s.slot < 0 ? kKeyMax : key;
    if constexpr (FRESH) {
      a = acc_t{k, s.value};
    } else {
      take(a, k, s.value);
    }
  }
  static __device__ __forceinline__ void push_cols(acc_t (&a)[VEC], const u32x4& v, i64 idx)
  {
    static_for<VEC>([&](auto j) { take(a[j], (KeyT)idx, In<InT>::template get<j>(v)); });
  }
  // The same for a thread that walks DOWN the rows of its columns: every accumulator is the
  // neutral one or holds a key above `idx`.
  static __device__ __forceinline__ void push_cols_down(acc_t (&a)[VEC], const u32x4& v, i64 idx)
  {
    static_for<VEC>([&](auto j) {
      const val_t x  = In<InT>::template get<j>(v);
      const bool win = IS_MAX ? (x >= a[j].value) : (x <= a[j].value);
      a[j].value     = win ? x : a[j].value;
      a[j].key       = win ? (KeyT)idx : a[j].key;
    });
  }
  static __device__ __forceinline__ void merge(acc_t& a, const acc_t& b) { take(a, b.key, b.value); }
  template <int SEL>
  static __device__ __forceinline__ acc_t exchange(const acc_t& a)
  {
    return acc_t{xchg<SEL>(a.key), xchg<SEL>(a.value)};
  }
};

// ---- mean and variance in one pass ---------------------------------------------
// State of a set of w values: their mean is k + sd / w and their sum of squared
// deviations from the mean is sdd - sd * sd / w, where sd and sdd are the sums of
// (x - k) and (x - k)^2 and the shift k is the first value the lane saw.  With the
// shift inside the data's range the subtraction loses a few bits at most, and an
// element costs three f64 operations and no division.  Two states merge by the
// pairwise update of Chan et al. that the reference's mean_var monoid uses
// (stats/detail/meanvar.cuh:16-99), the merged state stored with k = mean, sd = 0; sets
// of up to kMvReshiftMax values together merge by moving one's sums to the other's shift.
struct mv_t {
  double w;
  double k;
  double sd;
  double sdd;
};

__device__ __forceinline__ double mv_mean(const mv_t& a)
{
  return a.w > 0.0 ? a.k + a.sd / a.w : 0.0;
}
__device__ __forceinline__ double mv_m2(const mv_t& a)
{
  return a.w > 0.0 ? fmax(a.sdd - a.sd * a.sd / a.w, 0.0) : 0.0;
}

#ifndef RMI_MV_RESHIFT
#define RMI_MV_RESHIFT 1
#endif
constexpr double kMvReshiftMax = 65536.0;  // largest merged set that keeps a member's shift

template <class InT>
struct PolMeanVar {
  using in_t               = InT;
  using nat                = typename In<InT>::nat;
  using acc_t              = mv_t;
  static constexpr int VEC = In<InT>::VEC;
  static constexpr int CLS = kClsMeanVar;
  static constexpr int kTail = kTailEach;

  static __device__ __forceinline__ acc_t neutral() { return mv_t{0.0, 0.0, 0.0, 0.0}; }
  static __device__ __forceinline__ void push(acc_t& a, nat x, i64)
  {
    const double xd = (double)x;
    a.k             = a.w == 0.0 ? xd : a.k;
    const double d  = xd - a.k;
    a.sd += d;
    a.sdd = fma(d, d, a.sdd);
    a.w += 1.0;
  }
  // One shifted step without the first-value test (the caller has set a.k).
  static __device__ __forceinline__ void step(acc_t& a, double xd)
  {
    const double d = xd - a.k;
    a.sd += d;
    a.sdd = fma(d, d, a.sdd);
  }
  static __device__ __forceinline__ void push_vec(acc_t& a, const u32x4& v, i64)
  {
    // the shift is tested once per vector, behind a branch that is taken once per lane
    if (a.w == 0.0) a.k = (double)In<InT>::template get<0>(v);
    static_for<VEC>([&](auto j) { step(a, (double)In<InT>::template get<j>(v)); });
    a.w += (double)VEC;
  }
  static __device__ __forceinline__ void push_cols(acc_t (&a)[VEC], const u32x4& v, i64)
  {
    // per-column selects: a branch here measured slower on ragged widths
    static_for<VEC>([&](auto j) { push(a[j], In<InT>::template get<j>(v), 0); });
  }
  // The column kernel's main loop, where a lane folds one vector after the other into the
  // same VEC columns: the shift is taken from the first vector before the loop, a step is
  // three operations per element, and the count is added once after the loop.
  static __device__ __forceinline__ void cols_set_shift(acc_t (&a)[VEC], const u32x4& v)
  {
    static_for<VEC>([&](auto j) { a[j].k = (double)In<InT>::template get<j>(v); });
  }
  static __device__ __forceinline__ void cols_steps(acc_t (&a)[VEC], const u32x4& v)
  {
    static_for<VEC>([&](auto j) { step(a[j], (double)In<InT>::template get<j>(v)); });
  }
  static __device__ __forceinline__ void cols_count(acc_t (&a)[VEC], double n)
  {
    static_for<VEC>([&](auto j) { a[j].w += n; });
  }
  static __device__ __forceinline__ void merge(acc_t& a, const acc_t& b)
  {
    const double cw = a.w + b.w;
    double k, sd, sdd;
    if (RMI_MV_RESHIFT != 0 && cw <= kMvReshiftMax) {
      // Small sets: b's sums are moved to a's shift, sum(x - ka) = sd_b + w_b d and
      // sum((x - ka)^2) = sdd_b + 2 d sd_b + w_b d^2 with d = kb - ka, which takes no
      // division (the pairwise update takes three: six of them per row cost more than
      // reading a row of 671 floats).  The shift stays a value of the set, so
      // (mean - k)^2 <= w var and the subtraction in mv_m2 loses at most log2(w) bits
      // of the 53.
      k                = a.w == 0.0 ? b.k : a.k;
      const double d   = b.k - k;
      const double bwd = b.w * d;
      sdd              = a.sdd + fma(d, 2.0 * b.sd + bwd, b.sdd);
      sd               = a.sd + (b.sd + bwd);
    } else {
      const double ma = mv_mean(a), mb = mv_mean(b);
      const double sa = mv_m2(a), sb = mv_m2(b);
      const double fb = cw > 0.0 ? b.w / cw : 0.0;
      const double d  = mb - ma;
      k               = ma + d * fb;
      sdd             = (sa + sb) + d * d * (a.w * fb);
      sd              = 0.0;
    }
    a.k   = k;
    a.sd  = sd;
    a.sdd = sdd;
    a.w   = cw;
  }
  template <int SEL>
  static __device__ __forceinline__ acc_t exchange(const acc_t& a)
  {
    return mv_t{xchg<SEL>(a.w), xchg<SEL>(a.k), xchg<SEL>(a.sd), xchg<SEL>(a.sdd)};
  }
};

// ---------------------------------------------------------------------------
// The last, overlapping vector of a row whose length is not a multiple of VEC:
// it ends exactly at the row's end, so its first `skip` elements were already
// folded by the previous whole vector and only elements j >= skip count.
// ---------------------------------------------------------------------------
template <class P>
__device__ __forceinline__ void push_vec_from(typename P::acc_t& a,
                                              const u32x4& v,
                                              i64 idx0,
                                              int skip)
{
  using in_t = typename P::in_t;
  static_for<P::VEC>([&](auto j) {
    if (j >= skip) P::push(a, In<in_t>::template get<j>(v), idx0 + j);
  });
}

// ---------------------------------------------------------------------------
// Wave-level all-reduce over groups of G lanes (G a power of two, 1..64).
// G is wave-uniform at run time; every lane of the wave must call this.
// ---------------------------------------------------------------------------
template <class P>
__device__ __forceinline__ void group_allreduce(typename P::acc_t& a, int G)
{
  if (G > 1) P::merge(a, P::template exchange<0>(a));
  if (G > 2) P::merge(a, P::template exchange<1>(a));
  if (G > 4) P::merge(a, P::template exchange<2>(a));
  if (G > 8) P::merge(a, P::template exchange<3>(a));
  if (G > 16) P::merge(a, P::template exchange<4>(a));
  if (G > 32) P::merge(a, P::template exchange<5>(a));
}

template <class P>
__device__ __forceinline__ void wave_allreduce(typename P::acc_t& a)
{
  P::merge(a, P::template exchange<0>(a));
  P::merge(a, P::template exchange<1>(a));
  P::merge(a, P::template exchange<2>(a));
  P::merge(a, P::template exchange<3>(a));
  P::merge(a, P::template exchange<4>(a));
  P::merge(a, P::template exchange<5>(a));
}

// ---------------------------------------------------------------------------
// Epilogue: out[k] = final_op(inplace ? red(out_old[k], red(init, acc)) : red(init, acc))
// ---------------------------------------------------------------------------
struct Epilogue {
  void* out;
  const void* aux;
  double init_f;
  i64 init_i;
  double s1;
  double s2;
  int out_dtype;
  int final_op;
  int inplace;
  // Set by the host when inplace is off, the output is stored in the accumulator's
  // own family (f32 / f64, i32 / i64) and final_op is the identity (floating
  // outputs: also sqrt or a multiplication by a constant): the common cases, kept
  // free of the general epilogue's branches.
  int plain;
  int out_aligned16;  // the output pointer is 16-byte aligned
};

__device__ __forceinline__ float bf16_to_f32(uint16_t b) { return as_f32((u32)b << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16(float f)
{
  u32 u = as_u32(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);  // quiet NaN
  u += 0x7fffu + ((u >> 16) & 1u);                                            // nearest-even
  return (uint16_t)(u >> 16);
}

// Read one output-typed element as f64 (floating outputs only).
__device__ __forceinline__ double load_out_f64(const void* p, int dtype, i64 k)
{
  switch (dtype) {
    case RMI_F64: return static_cast<const double*>(p)[k];
    case RMI_F32: return (double)static_cast<const float*>(p)[k];
    case RMI_F16: return (double)(float)static_cast<const f16_t*>(p)[k];
    case RMI_BF16: return (double)bf16_to_f32(static_cast<const uint16_t*>(p)[k]);
    default: return 0.0;
  }
}

template <class T>
__device__ __forceinline__ T apply_final_fp(const Epilogue& e, T x, i64 k)
{
  switch (e.final_op) {
    case RMI_FIN_SQRT: return sqrt(x);
    case RMI_FIN_ABS: return fabs(x);
    case RMI_FIN_SQ: return x * x;
    case RMI_FIN_MUL_CONST: return x * (T)e.s1;
    case RMI_FIN_DIV_CONST: return x / (T)e.s1;
    case RMI_FIN_ADD_CONST: return x + (T)e.s1;
    case RMI_FIN_SUB_CONST: return x - (T)e.s1;
    case RMI_FIN_VAR_FROM_SUMSQ:
    case RMI_FIN_STDDEV_FROM_SUMSQ: {
      // stats/detail/stddev.cuh:46-59: a*ratio - b*b*ratio_mean, abs, [sqrt];
      // every step rounded in the output's arithmetic type.
      const T b = (T)load_out_f64(e.aux, e.out_dtype, k);
      T t       = x * (T)e.s1 - b * b * (T)e.s2;
      t         = fabs(t);
      return e.final_op == RMI_FIN_STDDEV_FROM_SUMSQ ? sqrt(t) : t;
    }
    default: return x;
  }
}

__device__ __forceinline__ void store_fp(const Epilogue& e, i64 k, double r)
{
  if (e.out_dtype == RMI_F64) {
    static_cast<double*>(e.out)[k] = apply_final_fp<double>(e, r, k);
    return;
  }
  const float y = apply_final_fp<float>(e, (float)r, k);
  switch (e.out_dtype) {
    case RMI_F32: static_cast<float*>(e.out)[k] = y; break;
    case RMI_F16: static_cast<f16_t*>(e.out)[k] = (f16_t)y; break;
    case RMI_BF16: static_cast<uint16_t*>(e.out)[k] = f32_to_bf16(y); break;
    default: break;
  }
}

__device__ __forceinline__ i64 apply_final_int(const Epilogue& e, i64 x)
{
  const i64 c = (i64)e.s1;
  switch (e.final_op) {
    case RMI_FIN_ABS: return x < 0 ? -x : x;
    case RMI_FIN_SQ: return x * x;
    case RMI_FIN_MUL_CONST: return x * c;
    case RMI_FIN_DIV_CONST: return c != 0 ? x / c : 0;
    case RMI_FIN_ADD_CONST: return x + c;
    case RMI_FIN_SUB_CONST: return x - c;
    default: return x;
  }
}

__device__ __forceinline__ void store_int(const Epilogue& e, i64 k, i64 r)
{
  r = apply_final_int(e, r);
  if (e.out_dtype == RMI_I64) {
    static_cast<i64*>(e.out)[k] = r;
  } else {
    static_cast<int32_t*>(e.out)[k] = (int32_t)r;
  }
}

// Output-side KVP layouts (natural alignment, key first).
template <class K, class V>
struct out_kvp {
  K key;
  V value;
};

// Single outputs use ordinary stores: small or strided non-temporal stores bypass
// the L2's write combining and measured slower on every shape.
template <class T>
__device__ __forceinline__ void store_stream(T* p, T v)
{
  *p = v;
}

template <class P>
__device__ __forceinline__ void finish(const Epilogue& e, i64 k, typename P::acc_t acc)
{
  using acc_t = typename P::acc_t;
  if constexpr (P::CLS == kClsFloat) {
    acc_t a = P::from_f64(e.init_f);
    P::merge(a, acc);
    if (e.plain) {
      // identity, sqrt or a multiplication by a constant, stored as f32 or f64:
      // the epilogues of sums, L2 norms and means
      if (e.out_dtype == RMI_F32) {
        float y = (float)P::to_f64(a);
        if (e.final_op == RMI_FIN_SQRT) y = sqrt(y);
        if (e.final_op == RMI_FIN_MUL_CONST) y = y * (float)e.s1;
        store_stream(static_cast<float*>(e.out) + k, y);
      } else {
        double y = P::to_f64(a);
        if (e.final_op == RMI_FIN_SQRT) y = sqrt(y);
        if (e.final_op == RMI_FIN_MUL_CONST) y = y * e.s1;
        store_stream(static_cast<double*>(e.out) + k, y);
      }
      return;
    }
    if (e.inplace) {
      acc_t o = P::from_f64(load_out_f64(e.out, e.out_dtype, k));
      P::merge(o, a);
      a = o;
    }
    store_fp(e, k, P::to_f64(a));
  } else if constexpr (P::CLS == kClsInt) {
    acc_t a = e.init_i;
    P::merge(a, acc);
    if (e.plain) {
      if (e.out_dtype == RMI_I64) {
        store_stream(static_cast<i64*>(e.out) + k, (i64)a);
      } else {
        store_stream(static_cast<int32_t*>(e.out) + k, (int32_t)a);
      }
      return;
    }
    if (e.inplace) {
      acc_t o = e.out_dtype == RMI_I64 ? static_cast<const i64*>(e.out)[k]
                                       : (i64) static_cast<const int32_t*>(e.out)[k];
      P::merge(o, a);
      a = o;
    }
    store_int(e, k, a);
  } else if constexpr (P::CLS == kClsMeanVar) {
    // out: means, aux: variances (written here), s1: 1 for the sample variance.
    // stats/detail/meanvar.cuh:88-98: var = M2 / max(1, sample ? w - 1 : w)
    const double mean = mv_mean(acc);
    const double den  = fmax(1.0, e.s1 != 0.0 ? acc.w - 1.0 : acc.w);
    const double var  = mv_m2(acc) / den;
    void* vp          = const_cast<void*>(e.aux);
    switch (e.out_dtype) {
      case RMI_F64:
        static_cast<double*>(e.out)[k] = mean;
        static_cast<double*>(vp)[k]    = var;
        break;
      case RMI_F16:
        static_cast<f16_t*>(e.out)[k] = (f16_t)(float)mean;
        static_cast<f16_t*>(vp)[k]    = (f16_t)(float)var;
        break;
      case RMI_BF16:
        static_cast<uint16_t*>(e.out)[k] = f32_to_bf16((float)mean);
        static_cast<uint16_t*>(vp)[k]    = f32_to_bf16((float)var);
        break;
      default:
        static_cast<float*>(e.out)[k] = (float)mean;
        static_cast<float*>(vp)[k]    = (float)var;
    }
  } else {
    using key_t = decltype(acc.key);
    using val_t = decltype(acc.value);
    acc_t a{(key_t)e.init_i, (val_t)e.init_f};
    P::merge(a, acc);
    if (e.final_op == RMI_FIN_KEY) {
      // index-only output (matrix::argmax / argmin); inplace has no meaning here
      if (e.out_dtype == RMI_I64) {
        static_cast<i64*>(e.out)[k] = (i64)a.key;
      } else {
        static_cast<int32_t*>(e.out)[k] = (int32_t)a.key;
      }
      return;
    }
    auto* o = static_cast<out_kvp<key_t, val_t>*>(e.out);
    if (e.inplace) {
      acc_t old{o[k].key, o[k].value};
      P::merge(old, a);
      a = old;
    }
    o[k].key   = a.key;
    o[k].value = a.value;
  }
}

// K results for the consecutive outputs k0 .. k0+K-1 held by one lane.  Pairs of
// int64 results leave as one 16-byte store when the epilogue is plain.
template <class P, int K>
__device__ __forceinline__ void finish_run(const Epilogue& e, i64 k0, typename P::acc_t (&acc)[K])
{
  if constexpr (P::CLS == kClsInt && (K % 2 == 0)) {
    if (e.plain && e.out_dtype == RMI_I64 && e.out_aligned16) {
#pragma unroll
      for (int r = 0; r < K; r += 2) {
        i64 a = e.init_i, b = e.init_i;
        P::merge(a, acc[r]);
        P::merge(b, acc[r + 1]);
        u32x4 v;
        v[0] = (u32)(u64)a;
        v[1] = (u32)((u64)a >> 32);
        v[2] = (u32)(u64)b;
        v[3] = (u32)((u64)b >> 32);
        // whole 16-byte lane stores, contiguous across the wave: streamed past the caches
        __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(static_cast<i64*>(e.out) + k0 + r));
      }
      return;
    }
  }
  if constexpr (P::CLS == kClsFloat && (K % 2 == 0)) {
    // the same for floating results: four f32 or two f64 per 16-byte store, two f32 per
    // 8-byte store (k0 is a multiple of K, so the stores are aligned when the output is)
    if (e.plain && e.out_aligned16) {
      auto value = [&](int r) {
        typename P::acc_t a = P::from_f64(e.init_f);
        P::merge(a, acc[r]);
        return P::to_f64(a);
      };
      if (e.out_dtype == RMI_F32) {
        float y[K];
#pragma unroll
        for (int r = 0; r < K; ++r) {
          y[r] = (float)value(r);
          if (e.final_op == RMI_FIN_SQRT) y[r] = sqrt(y[r]);
          if (e.final_op == RMI_FIN_MUL_CONST) y[r] = y[r] * (float)e.s1;
        }
        float* o = static_cast<float*>(e.out) + k0;
        if constexpr (K % 4 == 0) {
#pragma unroll
          for (int r = 0; r < K; r += 4) {
            u32x4 v;
            v[0] = as_u32(y[r]), v[1] = as_u32(y[r + 1]), v[2] = as_u32(y[r + 2]), v[3] = as_u32(y[r + 3]);
            __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(o + r));
          }
        } else {
          typedef u32 u32x2 __attribute__((ext_vector_type(2)));
#pragma unroll
          for (int r = 0; r < K; r += 2) {
            u32x2 v;
            v[0] = as_u32(y[r]), v[1] = as_u32(y[r + 1]);
            __builtin_nontemporal_store(v, reinterpret_cast<u32x2*>(o + r));
          }
        }
        return;
      }
      if (e.out_dtype == RMI_F64) {
        typedef double f64x2 __attribute__((ext_vector_type(2)));
#pragma unroll
        for (int r = 0; r < K; r += 2) {
          f64x2 v;
#pragma unroll
          for (int q = 0; q < 2; ++q) {
            double y = value(r + q);
            if (e.final_op == RMI_FIN_SQRT) y = sqrt(y);
            if (e.final_op == RMI_FIN_MUL_CONST) y = y * e.s1;
            v[q] = y;
          }
          __builtin_nontemporal_store(v, reinterpret_cast<f64x2*>(static_cast<double*>(e.out) + k0 + r));
        }
        return;
      }
    }
  }
#pragma unroll
  for (int r = 0; r < K; ++r)
    finish<P>(e, k0 + r, acc[r]);
}

}  // namespace rmi
