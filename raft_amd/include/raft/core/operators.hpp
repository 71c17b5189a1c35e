// The functor vocabulary of the reduction path: main_op / reduce_op / final_op
// arguments of raft::linalg::reduce and its wrappers.  Names, call signatures
// and results follow the reference (core/operators.hpp:27-423).  Every functor
// is also callable on the host, which is how the CPU tests pin the meaning of
// the tags the library's kernels implement.
//
// The kernels live behind a C ABI, so a functor reaches them as a tag, not as
// code: raft::detail::rmi::main_tag / reduce_tag / final_tag (rmi_bridge.hpp)
// map each functor type below to its tag.  A functor type with no mapping is
// a compile-time error at the call site.
#pragma once

#include <cstddef>
#include <tuple>
#include <type_traits>
#include <utility>

#include <raft/core/detail/macros.hpp>
#include <raft/core/kvp.hpp>
#include <raft/core/math.hpp>

namespace raft {

// ---- unary ------------------------------------------------------------------
struct identity_op {
  template <typename T, typename... Ignored>
  constexpr RAFT_INLINE_FUNCTION auto operator()(const T& x, Ignored...) const
  {
    return x;
  }
};

struct void_op {
  template <typename... Ignored>
  constexpr RAFT_INLINE_FUNCTION void operator()(Ignored...) const
  {
  }
};

template <typename OutT>
struct cast_op {
  template <typename T, typename... Ignored>
  constexpr RAFT_INLINE_FUNCTION auto operator()(T x, Ignored...) const
  {
    return static_cast<OutT>(x);
  }
};

struct key_op {
  template <typename KVP, typename... Ignored>
  constexpr RAFT_INLINE_FUNCTION auto operator()(const KVP& p, Ignored...) const
  {
    return p.key;
  }
};

struct value_op {
  template <typename KVP, typename... Ignored>
  constexpr RAFT_INLINE_FUNCTION auto operator()(const KVP& p, Ignored...) const
  {
    return p.value;
  }
};

struct sqrt_op {
  template <typename T, typename... Ignored>
  RAFT_INLINE_FUNCTION auto operator()(const T& x, Ignored...) const
  {
    return raft::sqrt(x);
  }
};

struct nz_op {
  template <typename T, typename... Ignored>
  constexpr RAFT_INLINE_FUNCTION auto operator()(const T& x, Ignored...) const
  {
    return x != T(0) ? T(1) : T(0);
  }
};

struct abs_op {
  template <typename T, typename... Ignored>
  RAFT_INLINE_FUNCTION auto operator()(const T& x, Ignored...) const
  {
    return raft::abs(x);
  }
};

struct sq_op {
  template <typename T, typename... Ignored>
  constexpr RAFT_INLINE_FUNCTION auto operator()(const T& x, Ignored...) const
  {
    return x * x;
  }
};

// (value, index) -> KeyValuePair{index, value}: the main_op of a key-value
// arg-reduction.  The reference leaves this functor to its callers (e.g. the
// test-local ValueToKVP of cpp/tests/linalg/reduce.cu:346-349); it is named here
// because a functor must have a known type to be lowered to a kernel tag.
template <typename IdxT = int>
struct value_to_kvp_op {
  template <typename T, typename I>
  constexpr RAFT_INLINE_FUNCTION auto operator()(const T& value, I idx) const
  {
    return KeyValuePair<IdxT, T>(static_cast<IdxT>(idx), value);
  }
};

// ---- binary -----------------------------------------------------------------
#define RAFT_RMI_BINARY_OP(NAME, EXPR)                                             \
  struct NAME {                                                                    \
    template <typename T1, typename T2>                                            \
    constexpr RAFT_INLINE_FUNCTION auto operator()(const T1& a, const T2& b) const \
    {                                                                              \
      return EXPR;                                                                 \
    }                                                                              \
  }
RAFT_RMI_BINARY_OP(add_op, a + b);
RAFT_RMI_BINARY_OP(sub_op, a - b);
RAFT_RMI_BINARY_OP(mul_op, a* b);
RAFT_RMI_BINARY_OP(div_op, a / b);
RAFT_RMI_BINARY_OP(greater_op, a > b);
RAFT_RMI_BINARY_OP(less_op, a < b);
RAFT_RMI_BINARY_OP(greater_or_equal_op, a >= b);
RAFT_RMI_BINARY_OP(less_or_equal_op, a <= b);
RAFT_RMI_BINARY_OP(equal_op, a == b);
RAFT_RMI_BINARY_OP(notequal_op, a != b);
#undef RAFT_RMI_BINARY_OP

struct div_checkzero_op {
  template <typename T1, typename T2>
  constexpr RAFT_INLINE_FUNCTION auto operator()(const T1& a, const T2& b) const
  {
    return b == T2{0} ? T1{0} / T2{1} : a / b;
  }
};

struct min_op {
  template <typename... Args>
  RAFT_INLINE_FUNCTION auto operator()(Args&&... args) const
  {
    return raft::min(std::forward<Args>(args)...);
  }
};

struct max_op {
  template <typename... Args>
  RAFT_INLINE_FUNCTION auto operator()(Args&&... args) const
  {
    return raft::max(std::forward<Args>(args)...);
  }
};

// Arg-reductions over KeyValuePair: the candidate b replaces a when its value is
// strictly better, or equal with the smaller key (lowest index wins ties).
struct argmin_op {
  template <typename KVP>
  constexpr RAFT_INLINE_FUNCTION auto operator()(const KVP& a, const KVP& b) const
  {
    const bool take_b = (b.value < a.value) || ((a.value == b.value) && (b.key < a.key));
    return take_b ? b : a;
  }
};

struct argmax_op {
  template <typename KVP>
  constexpr RAFT_INLINE_FUNCTION auto operator()(const KVP& a, const KVP& b) const
  {
    const bool take_b = (b.value > a.value) || ((a.value == b.value) && (b.key < a.key));
    return take_b ? b : a;
  }
};

// ---- constants and composition ------------------------------------------------
template <typename ScalarT>
struct const_op {
  const ScalarT scalar;
  constexpr explicit const_op(const ScalarT& s) : scalar{s} {}
  template <typename... Args>
  constexpr RAFT_INLINE_FUNCTION auto operator()(Args...) const
  {
    return scalar;
  }
};

// A binary functor with its right-hand operand fixed.
template <typename ConstT, typename BinaryOpT>
struct plug_const_op {
  const ConstT c;
  const BinaryOpT composed_op;

  template <typename OpT = BinaryOpT,
            typename     = std::enable_if_t<std::is_default_constructible_v<OpT>>>
  constexpr explicit plug_const_op(const ConstT& s) : c{s}, composed_op{}
  {
  }
  constexpr plug_const_op(const ConstT& s, BinaryOpT o) : c{s}, composed_op{o} {}

  template <typename T>
  constexpr RAFT_INLINE_FUNCTION auto operator()(T a) const
  {
    return composed_op(a, c);
  }
};

template <typename T>
using add_const_op = plug_const_op<T, add_op>;
template <typename T>
using sub_const_op = plug_const_op<T, sub_op>;
template <typename T>
using mul_const_op = plug_const_op<T, mul_op>;
template <typename T>
using div_const_op = plug_const_op<T, div_op>;
template <typename T>
using div_checkzero_const_op = plug_const_op<T, div_checkzero_op>;
template <typename T>
using equal_const_op = plug_const_op<T, equal_op>;

// compose_op(f, g, h)(x...) == f(g(h(x...))): all arguments go to the innermost op.
template <typename... OpsT>
struct compose_op {
  const std::tuple<OpsT...> ops;

  template <typename TupleT = std::tuple<OpsT...>,
            typename        = std::enable_if_t<std::is_default_constructible_v<TupleT>>>
  constexpr compose_op()
  {
  }
  constexpr explicit compose_op(OpsT... o) : ops{o...} {}

  template <typename... Args>
  constexpr RAFT_INLINE_FUNCTION auto operator()(Args&&... args) const
  {
    return apply_from<sizeof...(OpsT)>(std::forward<Args>(args)...);
  }

 private:
  template <size_t Remaining, typename... Args>
  constexpr RAFT_INLINE_FUNCTION auto apply_from(Args&&... args) const
  {
    if constexpr (Remaining == 0) {
      return identity_op{}(std::forward<Args>(args)...);
    } else {
      return apply_from<Remaining - 1>(std::get<Remaining - 1>(ops)(std::forward<Args>(args)...));
    }
  }
};

using absdiff_op = compose_op<abs_op, sub_op>;
using sqdiff_op  = compose_op<sq_op, sub_op>;

// map_args_op<Outer, A, B>(x, y) == Outer(A(x), B(y)).
template <typename OuterOpT, typename... ArgOpsT>
struct map_args_op {
  const OuterOpT outer_op;
  const std::tuple<ArgOpsT...> arg_ops;

  template <typename T1 = OuterOpT,
            typename T2 = std::tuple<ArgOpsT...>,
            typename    = std::enable_if_t<std::is_default_constructible_v<T1> &&
                                        std::is_default_constructible_v<T2>>>
  constexpr map_args_op() : outer_op{}
  {
  }
  constexpr explicit map_args_op(OuterOpT outer, ArgOpsT... inner)
    : outer_op{outer}, arg_ops{inner...}
  {
  }

  template <typename... Args>
  constexpr RAFT_INLINE_FUNCTION auto operator()(Args&&... args) const
  {
    static_assert(sizeof...(ArgOpsT) == sizeof...(Args),
                  "The number of arguments does not match the number of mapping operators");
    return call(std::index_sequence_for<ArgOpsT...>{}, std::forward<Args>(args)...);
  }

 private:
  template <size_t... I, typename... Args>
  constexpr RAFT_INLINE_FUNCTION auto call(std::index_sequence<I...>, Args&&... args) const
  {
    return outer_op(std::get<I>(arg_ops)(std::forward<Args>(args))...);
  }
};

}  // namespace raft
