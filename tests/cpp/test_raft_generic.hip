// GPU tests of the header-template fallback: reductions whose functors or element
// types are outside the library's vocabulary (device lambdas, caller-defined functor
// structs, KeyValuePair<int, short>) are instantiated in this translation unit by
// hipcc.  Cases follow the reference's callers of that kind: the test-local ValueToKVP
// / ArgMaxOp of cpp/tests/linalg/reduce.cu:346-411 and the capturing lambda of
// stats/detail/stddev.cuh:46-47.
#include <raft/core/device_mdarray.hpp>
#include <raft/core/device_mdspan.hpp>
#include <raft/core/operators.hpp>
#include <raft/linalg/coalesced_reduction.cuh>
#include <raft/linalg/map_reduce.cuh>
#include <raft/linalg/reduce.cuh>
#include <raft/linalg/strided_reduction.cuh>
#include <raft/stats/weighted_mean.cuh>
#include <raft/util/cudart_utils.hpp>
#include <raft/util/popc.cuh>

#include <cmath>
#include <cstdint>
#include <limits>
#include <random>

#include "check.hpp"

namespace {

template <typename T>
std::vector<T> to_host(const T* d, size_t n, hipStream_t s)
{
  std::vector<T> h(n);
  raft::update_host(h.data(), d, n, s);
  RAFT_HIP_TRY(hipStreamSynchronize(s));
  return h;
}

template <typename T>
std::vector<T> uniform(size_t n, double lo, double hi, unsigned long long seed)
{
  std::mt19937_64 g(seed);
  std::uniform_real_distribution<double> d(lo, hi);
  std::vector<T> v(n);
  for (auto& x : v)
    x = (T)d(g);
  return v;
}

inline size_t at(bool row_major, size_t N, size_t D, size_t i, size_t j)
{
  return row_major ? i * D + j : i + j * N;
}

// the test-local functors of cpp/tests/linalg/reduce.cu:346-358
template <typename T, typename IdxT = int>
struct ValueToKVP {
  HDI raft::KeyValuePair<IdxT, T> operator()(T value, IdxT idx) const { return {idx, value}; }
};
template <typename T1, typename T2>
struct ArgMaxOp {
  HDI raft::KeyValuePair<T1, T2> operator()(raft::KeyValuePair<T1, T2> a,
                                            raft::KeyValuePair<T1, T2> b) const
  {
    return (a.value > b.value || (a.value == b.value && a.key <= b.key)) ? a : b;
  }
};

bool close(double a, double b, double eps)
{
  const double d = std::fabs(a - b), m = std::max(std::fabs(a), std::fabs(b));
  return d <= eps || d / m <= eps;
}

}  // namespace

// device lambdas as main_op and final_op, all four layout x axis combinations
TEST_CASE(LambdaMainAndFinal)
{
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  for (auto [rows, cols] : std::vector<std::pair<int, int>>{{11, 7}, {1234, 33}, {1234, 128},
                                                            {37, 500}, {5, 70001}, {20011, 24}}) {
    auto h = uniform<float>((size_t)rows * cols, -1.0, 1.0, 1234);
    auto d = raft::make_device_vector<float, int>(handle, rows * cols);
    raft::update_device(d.data_handle(), h.data(), h.size(), stream);
    for (int rm = 0; rm < 2; ++rm)
      for (int ar = 0; ar < 2; ++ar) {
        const int n_out = ar ? rows : cols, len = ar ? cols : rows;
        auto out = raft::make_device_vector<float, int>(handle, n_out);
        auto main_op = [] __device__(float a, int i) { return a * a + 0.001f * (float)(i % 7); };
        auto fin_op  = [] __device__(float x) { return 0.5f * x + 1.0f; };
        auto ov      = out.view();
        if (rm) {
          auto v = raft::make_device_matrix_view<const float, int, raft::row_major>(
            d.data_handle(), rows, cols);
          if (ar)
            raft::linalg::reduce<raft::Apply::ALONG_ROWS>(handle, v, ov, 0.0f, false, main_op,
                                                          raft::add_op(), fin_op);
          else
            raft::linalg::reduce<raft::Apply::ALONG_COLUMNS>(handle, v, ov, 0.0f, false, main_op,
                                                             raft::add_op(), fin_op);
        } else {
          auto v = raft::make_device_matrix_view<const float, int, raft::col_major>(
            d.data_handle(), rows, cols);
          if (ar)
            raft::linalg::reduce<raft::Apply::ALONG_ROWS>(handle, v, ov, 0.0f, false, main_op,
                                                          raft::add_op(), fin_op);
          else
            raft::linalg::reduce<raft::Apply::ALONG_COLUMNS>(handle, v, ov, 0.0f, false, main_op,
                                                             raft::add_op(), fin_op);
        }
        auto got = to_host(out.data_handle(), (size_t)n_out, stream);
        bool ok  = true;
        for (int k = 0; k < n_out; ++k) {
          double acc = 0;
          for (int r = 0; r < len; ++r) {
            const double x = h[ar ? at(rm, rows, cols, k, r) : at(rm, rows, cols, r, k)];
            acc += x * x + 0.001 * (r % 7);
          }
          ok &= close(got[k], 0.5 * acc + 1.0, 2e-4);
        }
        CHECK(ok);
      }
  }
}

// cpp/tests/linalg/reduce.cu:360-400: KeyValuePair<int, short> / <int, float> / <int, double>
// arg-max with the test's own functors, inplace = false then true
template <typename T>
void kvp_custom()
{
  using KVP = raft::KeyValuePair<int, T>;
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  for (int rows : {11, 1234})
    for (int cols : {7, 33, 128, 500}) {
      std::mt19937 g(1234);
      std::uniform_int_distribution<int> di(-3000, 3000);
      std::vector<T> h((size_t)rows * cols);
      for (auto& x : h)
        x = (T)di(g);
      auto d    = raft::make_device_matrix<T, int, raft::row_major>(handle, rows, cols);
      auto dots = raft::make_device_vector<KVP, int>(handle, rows);
      raft::update_device(d.data_handle(), h.data(), h.size(), stream);
      for (int inplace = 0; inplace < 2; ++inplace) {
        raft::linalg::reduce<raft::Apply::ALONG_ROWS>(
          handle, raft::make_const_mdspan(d.view()), dots.view(), KVP(0, std::numeric_limits<T>::lowest()),
          (bool)inplace, ValueToKVP<T, int>(), ArgMaxOp<int, T>(), raft::identity_op());
        auto got = to_host(dots.data_handle(), (size_t)rows, stream);
        bool ok  = true;
        for (int r = 0; r < rows; ++r) {
          int best = 0;
          for (int j = 1; j < cols; ++j)
            if (h[(size_t)r * cols + j] > h[(size_t)r * cols + best]) best = j;
          ok &= got[r].key == best && got[r].value == h[(size_t)r * cols + best];
        }
        CHECK(ok);
      }
    }
}
TEST_CASE(KvpShortCustomFunctors) { kvp_custom<short>(); }
TEST_CASE(KvpFloatCustomFunctors) { kvp_custom<float>(); }
TEST_CASE(KvpDoubleCustomFunctors) { kvp_custom<double>(); }

// stats/detail/stddev.cuh:46-47: a capturing lambda as main_op of a column reduction
TEST_CASE(CapturingLambdaColumns)
{
  raft::resources handle;
  auto stream    = raft::resource::get_cuda_stream(handle);
  const int rows = 50000, cols = 48;
  auto h         = uniform<float>((size_t)rows * cols, -2.0, 3.0, 7);
  auto d         = raft::make_device_matrix<float, int, raft::row_major>(handle, rows, cols);
  auto out       = raft::make_device_vector<float, int>(handle, cols);
  raft::update_device(d.data_handle(), h.data(), h.size(), stream);
  const float shift = 0.25f;
  raft::linalg::strided_reduction(
    handle, raft::make_const_mdspan(d.view()), out.view(), 0.0f, false,
    [shift] __device__(float a, int) { return (a - shift) * (a - shift); });
  auto got = to_host(out.data_handle(), (size_t)cols, stream);
  bool ok  = true;
  for (int j = 0; j < cols; ++j) {
    double acc = 0;
    for (int i = 0; i < rows; ++i) {
      const double x = (double)h[(size_t)i * cols + j] - shift;
      acc += x * x;
    }
    ok &= close(got[j], acc, 5e-4);
  }
  CHECK(ok);
}

// an element type the library has no kernel for (int16) with library functors, and a
// custom reduce_op (product) over doubles: long rows (split) and many short rows
TEST_CASE(UnknownTypesAndReduceOps)
{
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  {
    const int rows = 3, cols = 300000;
    std::mt19937 g(5);
    std::uniform_int_distribution<int> di(-100, 100);
    std::vector<std::int16_t> h((size_t)rows * cols);
    for (auto& x : h)
      x = (std::int16_t)di(g);
    auto d   = raft::make_device_matrix<std::int16_t, int, raft::row_major>(handle, rows, cols);
    auto out = raft::make_device_vector<long long, int>(handle, rows);
    raft::update_device(d.data_handle(), h.data(), h.size(), stream);
    raft::linalg::coalesced_reduction(handle, raft::make_const_mdspan(d.view()), out.view(), 0LL,
                                      false, raft::cast_op<long long>(), raft::add_op());
    auto got = to_host(out.data_handle(), (size_t)rows, stream);
    for (int r = 0; r < rows; ++r) {
      long long s = 0;
      for (int j = 0; j < cols; ++j)
        s += h[(size_t)r * cols + j];
      CHECK(got[r] == s);
    }
  }
  {
    const int rows = 4000, cols = 9;
    auto h   = uniform<double>((size_t)rows * cols, 0.9, 1.1, 11);
    auto d   = raft::make_device_matrix<double, int, raft::row_major>(handle, rows, cols);
    auto out = raft::make_device_vector<double, int>(handle, rows);
    raft::update_device(d.data_handle(), h.data(), h.size(), stream);
    raft::linalg::reduce<raft::Apply::ALONG_ROWS>(handle, raft::make_const_mdspan(d.view()),
                                                  out.view(), 1.0, false, raft::identity_op(),
                                                  raft::mul_op());
    auto got = to_host(out.data_handle(), (size_t)rows, stream);
    bool ok  = true;
    for (int r = 0; r < rows; ++r) {
      double p = 1;
      for (int j = 0; j < cols; ++j)
        p *= h[(size_t)r * cols + j];
      ok &= close(got[r], p, 1e-12);
    }
    CHECK(ok);
  }
}

// Column reductions of the template path over element types of 1, 2 and 8 bytes: rows
// shorter than one 16-byte lane load, rows that end in a partial one, wide rows; the main_op
// uses the row index, so a thread that owned a wrong column or row would show.
template <typename T>
void strided_index_cases()
{
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  for (auto [rows, cols] : std::vector<std::pair<int, int>>{
         {9, 1}, {2000, 3}, {1501, 5}, {4099, 20}, {777, 33}, {3000, 129}, {300, 1030}, {40001, 16}}) {
    std::mt19937 g(rows + cols);
    std::uniform_int_distribution<int> di(-100, 100);
    std::vector<T> h((size_t)rows * cols);
    for (auto& x : h)
      x = (T)di(g);
    auto d   = raft::make_device_matrix<T, int, raft::row_major>(handle, rows, cols);
    auto out = raft::make_device_vector<long long, int>(handle, cols);
    raft::update_device(d.data_handle(), h.data(), h.size(), stream);
    raft::linalg::strided_reduction(
      handle, raft::make_const_mdspan(d.view()), out.view(), 0LL, false,
      [] __device__(T a, int i) { return (long long)a * (long long)(1 + i % 5); }, raft::add_op());
    auto got = to_host(out.data_handle(), (size_t)cols, stream);
    bool ok  = true;
    for (int j = 0; j < cols; ++j) {
      long long s = 0;
      for (int i = 0; i < rows; ++i)
        s += (long long)h[(size_t)i * cols + j] * (1 + i % 5);
      ok &= got[j] == s;
    }
    if (!ok) std::printf("  strided %dx%d, %zu-byte elements\n", rows, cols, sizeof(T));
    CHECK(ok);
  }
}
TEST_CASE(StridedIndexInt8) { strided_index_cases<std::int8_t>(); }
TEST_CASE(StridedIndexInt16) { strided_index_cases<std::int16_t>(); }
TEST_CASE(StridedIndexDouble) { strided_index_cases<double>(); }

// arg-max along the columns with the test-local functors (the reference's own kernels
// reject KeyValuePair outputs there, linalg/strided_reduction.cuh:70-77)
TEST_CASE(KvpColumnsCustomFunctors)
{
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  using KVP   = raft::KeyValuePair<int, float>;
  for (auto [rows, cols] : std::vector<std::pair<int, int>>{{5000, 7}, {3001, 64}, {901, 130}}) {
    auto h   = uniform<float>((size_t)rows * cols, -1.0, 1.0, 99 + cols);
    auto d   = raft::make_device_matrix<float, int, raft::row_major>(handle, rows, cols);
    auto out = raft::make_device_vector<KVP, int>(handle, cols);
    raft::update_device(d.data_handle(), h.data(), h.size(), stream);
    raft::linalg::strided_reduction(handle, raft::make_const_mdspan(d.view()), out.view(),
                                    KVP{0, -std::numeric_limits<float>::infinity()}, false,
                                    ValueToKVP<float, int>{}, ArgMaxOp<int, float>{});
    auto got = to_host(out.data_handle(), (size_t)cols, stream);
    bool ok  = true;
    for (int j = 0; j < cols; ++j) {
      int best = 0;
      for (int i = 1; i < rows; ++i)
        if (h[(size_t)i * cols + j] > h[(size_t)best * cols + j]) best = i;
      ok &= got[j].key == best && got[j].value == h[(size_t)best * cols + j];
    }
    CHECK(ok);
  }
}

// util/detail/popc.cuh:30-65: a bit count over packed words as a coalesced reduction of an
// N x 1 column-major view, whose lambda masks the last word by its index
template <typename value_t, typename index_t>
void popc_caller_case(index_t n_words, index_t max_len)
{
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  std::mt19937_64 g(n_words + max_len);
  std::vector<value_t> h((size_t)n_words);
  for (auto& x : h)
    x = (value_t)g();
  auto d       = raft::make_device_vector<value_t, index_t>(handle, n_words);
  auto counter = raft::make_device_vector<index_t, index_t>(handle, 1);
  raft::update_device(d.data_handle(), h.data(), h.size(), stream);
  constexpr index_t bits  = sizeof(value_t) * 8;
  const value_t tail_len  = (value_t)(max_len % bits);
  const value_t tail_mask = tail_len ? (value_t)((value_t{1} << tail_len) - value_t{1}) : (value_t) ~value_t{0};
  auto values = raft::make_device_matrix_view<const value_t, index_t, raft::col_major>(
    d.data_handle(), n_words, 1);
  raft::linalg::coalesced_reduction(
    handle, values, counter.view(), index_t{0}, false,
    [tail_mask, n_words] __device__(value_t value, index_t index) {
      const value_t v = index == n_words - 1 ? (value_t)(value & tail_mask) : value;
      return (index_t)__popcll((unsigned long long)v);
    });
  auto got = to_host(counter.data_handle(), 1, stream);
  index_t want = 0;
  for (index_t i = 0; i < n_words; ++i) {
    const value_t v = i == n_words - 1 ? (value_t)(h[(size_t)i] & tail_mask) : h[(size_t)i];
    want += (index_t)__builtin_popcountll((unsigned long long)v);
  }
  if (got[0] != want) std::printf("  popc %lld words: %lld != %lld\n", (long long)n_words, (long long)got[0], (long long)want);
  CHECK(got[0] == want);
}
// the same through raft::popc itself (cpp/tests/util/popc.cu: bit arrays whose length is
// not a multiple of the word size)
TEST_CASE(PopcHeader)
{
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  for (std::int64_t n_bits : std::vector<std::int64_t>{1, 31, 32, 33, 1000, 65537, 10000019}) {
    const std::int64_t n_words = (n_bits + 31) / 32;
    std::mt19937 g((unsigned)n_bits);
    std::vector<std::uint32_t> h((size_t)n_words);
    for (auto& x : h) x = g();
    auto d       = raft::make_device_vector<std::uint32_t, std::int64_t>(handle, n_words);
    auto counter = raft::make_device_vector<std::int64_t, std::int64_t>(handle, 1);
    raft::update_device(d.data_handle(), h.data(), h.size(), stream);
    raft::popc(handle, raft::make_device_vector_view<const std::uint32_t, std::int64_t>(d.data_handle(), n_words),
               raft::make_host_scalar_view<const std::int64_t, std::int64_t>(&n_bits),
               raft::make_device_scalar_view<std::int64_t>(counter.data_handle()));
    auto got = to_host(counter.data_handle(), 1, stream);
    std::int64_t want = 0;
    for (std::int64_t b = 0; b < n_bits; ++b)
      want += (h[(size_t)(b / 32)] >> (b % 32)) & 1u;
    CHECK(got[0] == want);
  }
}

TEST_CASE(PopcCaller)
{
  popc_caller_case<std::uint32_t, std::int64_t>(1, 7);
  popc_caller_case<std::uint32_t, std::int64_t>(1000, 1000 * 32 - 5);
  popc_caller_case<std::uint32_t, std::int64_t>(3000001, 3000001LL * 32 - 31);
  popc_caller_case<std::uint64_t, std::int64_t>(777777, 777777LL * 64 - 1);
  popc_caller_case<std::uint8_t, std::int64_t>(100003, 100003LL * 8 - 3);
}

// linalg/detail/tsvd.cuh:213-245: the signed value of largest magnitude per column or per
// row, with the caller's own reduce lambda (sign flip of the singular vectors)
TEST_CASE(SignedAbsMaxCaller)
{
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  for (auto [N, D] : std::vector<std::pair<int, int>>{{1000, 7}, {20000, 33}, {64, 5000}, {3, 200000}}) {
    auto h   = uniform<float>((size_t)N * D, -1.0, 1.0, N + D);
    auto d   = raft::make_device_vector<float, int>(handle, N * D);
    raft::update_device(d.data_handle(), h.data(), h.size(), stream);
    auto absmax = [] __device__(float a, float b) {
      const float abs_a = a >= 0.f ? a : -a;
      const float abs_b = b >= 0.f ? b : -b;
      return abs_a >= abs_b ? a : b;
    };
    for (int along_rows = 0; along_rows < 2; ++along_rows) {
      const int n_out = along_rows ? N : D, len = along_rows ? D : N;
      auto out = raft::make_device_vector<float, int>(handle, n_out);
      if (along_rows)
        raft::linalg::reduce<true, true>(out.data_handle(), d.data_handle(), D, N, 0.f, stream, false,
                                         raft::identity_op(), absmax, raft::identity_op());
      else
        raft::linalg::reduce<true, false>(out.data_handle(), d.data_handle(), D, N, 0.f, stream, false,
                                          raft::identity_op(), absmax, raft::identity_op());
      auto got = to_host(out.data_handle(), (size_t)n_out, stream);
      bool ok  = true;
      for (int k = 0; k < n_out; ++k) {
        float best = 0.f;
        for (int r = 0; r < len; ++r) {
          const float x = along_rows ? h[(size_t)k * D + r] : h[(size_t)r * D + k];
          if (std::fabs(x) > std::fabs(best)) best = x;
        }
        ok &= got[k] == best;
      }
      if (!ok) std::printf("  signed abs-max %dx%d along_rows=%d\n", N, D, along_rows);
      CHECK(ok);
    }
  }
}

// library functors still take the C ABI path from a hipcc translation unit
TEST_CASE(VocabularyStillLowered)
{
  raft::resources handle;
  auto stream    = raft::resource::get_cuda_stream(handle);
  const int rows = 1000, cols = 128;
  auto h         = uniform<float>((size_t)rows * cols, -1.0, 1.0, 3);
  auto d         = raft::make_device_matrix<float, int, raft::row_major>(handle, rows, cols);
  auto out       = raft::make_device_vector<float, int>(handle, rows);
  raft::update_device(d.data_handle(), h.data(), h.size(), stream);
  raft::linalg::reduce<raft::Apply::ALONG_ROWS>(handle, raft::make_const_mdspan(d.view()),
                                                out.view(), 0.0f, false, raft::sq_op(),
                                                raft::add_op(), raft::sqrt_op());
  auto got = to_host(out.data_handle(), (size_t)rows, stream);
  bool ok  = true;
  for (int r = 0; r < rows; ++r) {
    double s = 0;
    for (int j = 0; j < cols; ++j)
      s += (double)h[(size_t)r * cols + j] * h[(size_t)r * cols + j];
    ok &= close(got[r], std::sqrt(s), 1e-6);
  }
  CHECK(ok);
}

// map_reduce with a device lambda: the map sees the value alone
// (linalg/detail/map_then_reduce.cuh:58-61)
TEST_CASE(MapReduceLambda)
{
  raft::resources handle;
  auto stream   = raft::resource::get_cuda_stream(handle);
  const int len = 1 << 20;
  auto h        = uniform<float>(len, -1.0, 1.0, 9);
  auto in       = raft::make_device_vector<float, int>(handle, len);
  auto out      = raft::make_device_scalar<float>(handle);
  raft::update_device(in.data_handle(), h.data(), h.size(), stream);
  auto in_c = raft::make_device_vector_view<const float, int>(in.data_handle(), len);
  raft::linalg::map_reduce(handle, in_c, out.view(), 0.0f,
                           [] __device__(float x) { return x > 0.0f ? x : 0.0f; },
                           raft::add_op());
  double want = 0;
  for (float x : h)
    want += x > 0 ? x : 0;
  CHECK(close(to_host(out.data_handle(), 1, stream)[0], want, 1e-4));
}

// cpp/tests/stats/weighted_mean.cu:24-300: weighted means along rows and columns, both
// layouts, against the naive host evaluation with the reference's tolerance (tol * N)
template <typename T>
void weighted_mean_cases(double tol)
{
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  struct Case { int M, N; bool along_rows, row_major; };
  const std::vector<Case> cases{{4, 4, true, true},      {32, 32, true, false},
                                {32, 64, false, false},  {32, 256, true, true},
                                {32, 256, false, false}, {1024, 32, true, false},
                                {1024, 64, true, true},  {1024, 128, true, false},
                                {1024, 256, true, true}, {1024, 32, false, false},
                                {1024, 64, false, true}, {1024, 128, false, false},
                                {1024, 256, false, true}, {3, 100000, true, true},
                                {100000, 5, false, true}};
  for (const auto& c : cases) {
    const int rows = c.M, cols = c.N;
    const int wlen = c.along_rows ? cols : rows, olen = c.along_rows ? rows : cols;
    auto hd = uniform<T>((size_t)rows * cols, -1.0, 1.0, 1234);
    auto hw = uniform<T>((size_t)wlen, -1.0, 1.0, 4321);
    auto dd = raft::make_device_vector<T, int>(handle, rows * cols);
    auto dw = raft::make_device_vector<T, int>(handle, wlen);
    auto mu = raft::make_device_vector<T, int>(handle, olen);
    raft::update_device(dd.data_handle(), hd.data(), hd.size(), stream);
    raft::update_device(dw.data_handle(), hw.data(), hw.size(), stream);
    auto wv = raft::make_device_vector_view<const T, int>(dw.data_handle(), wlen);
    auto run = [&](auto layout) {
      using layout_t = decltype(layout);
      auto in = raft::make_device_matrix_view<const T, int, layout_t>(dd.data_handle(), rows, cols);
      if (c.along_rows)
        raft::stats::row_weighted_mean(handle, in, wv, mu.view());
      else
        raft::stats::col_weighted_mean(handle, in, wv, mu.view());
    };
    if (c.row_major) run(raft::row_major{}); else run(raft::col_major{});
    double ws = 0;
    for (T w : hw)
      ws += (double)w;
    // the device sums the weights in T; divide by that sum as the reference does
    std::vector<double> want(olen, 0.0);
    for (int k = 0; k < olen; ++k) {
      double s = 0;
      for (int r = 0; r < wlen; ++r) {
        const size_t idx = c.along_rows ? at(c.row_major, rows, cols, k, r)
                                        : at(c.row_major, rows, cols, r, k);
        s += (double)hd[idx] * (double)hw[r];
      }
      want[k] = s / ws;
    }
    auto got = to_host(mu.data_handle(), (size_t)olen, stream);
    bool ok  = true;
    const double bound = tol * wlen / std::fabs(ws) + tol;
    for (int k = 0; k < olen; ++k)
      ok &= std::fabs((double)got[k] - want[k]) <= bound * (1.0 + std::fabs(want[k]));
    if (!ok) std::printf("  weighted mean %dx%d along_rows=%d row_major=%d\n", rows, cols, c.along_rows, c.row_major);
    CHECK(ok);
  }
}
TEST_CASE(WeightedMeanF) { weighted_mean_cases<float>(1e-6); }
TEST_CASE(WeightedMeanD) { weighted_mean_cases<double>(1e-14); }

// Combinations whose functors all have tags but which the library has no kernel for are
// instantiated here like any other functor: a count of non-zeros of float data into an int
// (nz_op + add_op), the maximum of integers into a float, and cast_op<int> on float data,
// whose truncation must not be lost (sum of the truncated values, not the truncated sum).
TEST_CASE(TagValidCombinationsWithoutALibraryKernel)
{
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  const int rows = 300, cols = 517;
  auto h = uniform<float>((size_t)rows * cols, -3.0, 3.0, 77);
  for (size_t i = 0; i < h.size(); i += 7)
    h[i] = 0.0f;
  auto in = raft::make_device_matrix<float, int, raft::row_major>(handle, rows, cols);
  raft::update_device(in.data_handle(), h.data(), h.size(), stream);
  auto in_c = raft::make_const_mdspan(in.view());
  {
    auto out = raft::make_device_vector<int, int>(handle, rows);
    raft::linalg::reduce<raft::Apply::ALONG_ROWS>(handle, in_c, out.view(), 0, false, raft::nz_op{},
                                                  raft::add_op{});
    auto got = to_host(out.data_handle(), (size_t)rows, stream);
    bool ok  = true;
    for (int r = 0; r < rows; ++r) {
      int want = 0;
      for (int c = 0; c < cols; ++c)
        want += h[(size_t)r * cols + c] != 0.0f;
      ok &= got[r] == want;
    }
    CHECK(ok);
  }
  {
    auto out = raft::make_device_vector<int, int>(handle, cols);
    raft::linalg::reduce<raft::Apply::ALONG_COLUMNS>(handle, in_c, out.view(), 0, false,
                                                     raft::cast_op<int>{}, raft::add_op{});
    auto got = to_host(out.data_handle(), (size_t)cols, stream);
    bool ok  = true;
    for (int c = 0; c < cols; ++c) {
      int want = 0;
      for (int r = 0; r < rows; ++r)
        want += (int)h[(size_t)r * cols + c];
      ok &= got[c] == want;
    }
    CHECK(ok);
  }
  {
    std::vector<int> hi((size_t)rows * cols);
    for (size_t i = 0; i < hi.size(); ++i)
      hi[i] = (int)(h[i] * 1000.0f);
    auto ini = raft::make_device_matrix<int, int, raft::row_major>(handle, rows, cols);
    raft::update_device(ini.data_handle(), hi.data(), hi.size(), stream);
    auto out = raft::make_device_vector<float, int>(handle, rows);
    raft::linalg::reduce<raft::Apply::ALONG_ROWS>(handle, raft::make_const_mdspan(ini.view()), out.view(),
                                                  -1e30f, false, raft::cast_op<float>{}, raft::max_op{});
    auto got = to_host(out.data_handle(), (size_t)rows, stream);
    bool ok  = true;
    for (int r = 0; r < rows; ++r) {
      int want = hi[(size_t)r * cols];
      for (int c = 1; c < cols; ++c)
        want = std::max(want, hi[(size_t)r * cols + c]);
      ok &= got[r] == (float)want;
    }
    CHECK(ok);
  }
}

// The weight sum stays on the device (the reference brings it to the host and synchronises,
// stats/detail/weighted_mean.cuh:38-42), so the whole call can be captured into a HIP graph:
// captured once, replayed over new data and weights, each replay against the host.
TEST_CASE(WeightedMeanUnderGraphCapture)
{
  hipStream_t s;
  RAFT_HIP_TRY(hipStreamCreate(&s));
  {
    raft::resources handle(s);
    const int rows = 1024, cols = 256;
    auto dd = raft::make_device_vector<float, int>(handle, rows * cols);
    auto dw = raft::make_device_vector<float, int>(handle, cols);
    auto mu = raft::make_device_vector<float, int>(handle, rows);
    auto in = raft::make_device_matrix_view<const float, int, raft::row_major>(dd.data_handle(), rows, cols);
    auto wv = raft::make_device_vector_view<const float, int>(dw.data_handle(), cols);
    auto upload = [&](unsigned long long seed) {
      auto hd = uniform<float>((size_t)rows * cols, -1.0, 1.0, seed);
      auto hw = uniform<float>((size_t)cols, 0.1, 1.0, seed + 1);
      RAFT_HIP_TRY(hipMemcpy(dd.data_handle(), hd.data(), hd.size() * sizeof(float), hipMemcpyHostToDevice));
      RAFT_HIP_TRY(hipMemcpy(dw.data_handle(), hw.data(), hw.size() * sizeof(float), hipMemcpyHostToDevice));
      std::vector<double> want(rows);
      double ws = 0;
      for (float w : hw)
        ws += w;
      for (int r = 0; r < rows; ++r) {
        double acc = 0;
        for (int c = 0; c < cols; ++c)
          acc += (double)hd[(size_t)r * cols + c] * hw[c];
        want[r] = acc / ws;
      }
      return want;
    };
    auto check_mu = [&](const std::vector<double>& want) {
      auto got = to_host(mu.data_handle(), (size_t)rows, s);
      bool ok  = true;
      for (int r = 0; r < rows; ++r)
        ok &= std::fabs((double)got[r] - want[r]) <= 1e-5 * (1.0 + std::fabs(want[r]));
      CHECK(ok);
    };
    // eager once: the handle allocates its scalar slot here, outside the capture
    auto want = upload(11);
    raft::stats::row_weighted_mean(handle, in, wv, mu.view());
    check_mu(want);

    hipGraph_t graph;
    hipGraphExec_t exec;
    RAFT_HIP_TRY(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal));
    raft::stats::row_weighted_mean(handle, in, wv, mu.view());
    RAFT_HIP_TRY(hipStreamEndCapture(s, &graph));
    RAFT_HIP_TRY(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
    for (int rep = 0; rep < 3; ++rep) {
      want = upload(100 + 7 * rep);
      RAFT_HIP_TRY(hipMemsetAsync(mu.data_handle(), 0, rows * sizeof(float), s));
      RAFT_HIP_TRY(hipStreamSynchronize(s));
      RAFT_HIP_TRY(hipGraphLaunch(exec, s));
      check_mu(want);
    }
    RAFT_HIP_TRY(hipGraphExecDestroy(exec));
    RAFT_HIP_TRY(hipGraphDestroy(graph));
  }
  RAFT_HIP_TRY(hipStreamDestroy(s));
}

// map over two arrays, then sum: the call shape of linalg/detail/mean_squared_error.cuh:18-24
// (sq_diff(a, b) summed over two arrays) and stats/detail/kl_divergence.cuh:62
TEST_CASE(MapReduceTwoArrays)
{
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  for (int len : {0, 1, 3, 1000, 4099, (1 << 20) + 5, (1 << 24) + 1}) {
    auto ha = uniform<float>((size_t)len, -1.0, 1.0, 31);
    auto hb = uniform<float>((size_t)len, -1.0, 1.0, 32);
    auto da = raft::make_device_vector<float, int>(handle, len + 1);
    auto db = raft::make_device_vector<float, int>(handle, len + 1);
    auto out = raft::make_device_scalar<double>(handle);
    // one element of slack in front: element-aligned, not 16-byte aligned
    raft::update_device(da.data_handle() + 1, ha.data(), ha.size(), stream);
    raft::update_device(db.data_handle() + 1, hb.data(), hb.size(), stream);
    const float weight = 0.5f;
    auto sq_diff       = [weight] __device__(float a, float b) {
      const double d = (double)a - (double)b;
      return d * d * weight;
    };
    raft::linalg::mapThenSumReduce<float, decltype(sq_diff), std::uint32_t, 256, const float*>(
      out.data_handle(), (std::uint32_t)len, sq_diff, stream, da.data_handle() + 1,
      (const float*)(db.data_handle() + 1));
    double want = 0;
    for (int i = 0; i < len; ++i) {
      const double d = (double)ha[i] - (double)hb[i];
      want += d * d * 0.5;
    }
    CHECK(close(to_host(out.data_handle(), 1, stream)[0], want, 1e-9));
    // a maximum over three arrays through mapReduce
    auto dc = raft::make_device_vector<float, int>(handle, len + 1);
    raft::update_device(dc.data_handle(), ha.data(), ha.size(), stream);
    auto outf = raft::make_device_scalar<float>(handle);
    raft::linalg::mapReduce<float>(
      outf.data_handle(), (size_t)len, -1e30f,
      [] __device__(float a, float b, float c) { return a * b + c; }, raft::max_op(), stream,
      (const float*)(da.data_handle() + 1), (const float*)(db.data_handle() + 1),
      (const float*)dc.data_handle());
    float wantf = -1e30f;
    for (int i = 0; i < len; ++i)
      wantf = std::max(wantf, ha[i] * hb[i] + ha[i]);
    CHECK(close(to_host(outf.data_handle(), 1, stream)[0], wantf, 1e-6));
  }
}

// Sums of a caller's own main_op carry a wider accumulator, as the reference's kernels carry a
// Kahan-Babuska-Neumaier compensation whenever reduce_op is raft::add_op
// (linalg/detail/coalesced_reduction-inl.cuh:255,421,568).  The data is that of the reference's
// accuracy test (cpp/tests/stats/sum.cu:54-76): along the reduced axis 3v, -v * L, +v * L repeat
// with L = 1e7 (float) / 1e12 (double), so a plain accumulation in the element type loses the
// small terms' low bits at every step and the exact sum is (len / 3) * T(3v).
template <typename T>
void compensated_lambda_sums(double large, double tol)
{
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  const T v   = (T)0.1;
  struct shape {
    int n_out, len;
  };
  // lane-group rows (power-of-two and other lane counts), split rows, few and many columns
  for (bool contiguous : {true, false})
    for (shape sh : {shape{501, 96}, shape{300, 3072}, shape{3, 3 << 19}, shape{40, 3 << 15}}) {
      std::vector<T> h((size_t)sh.n_out * sh.len);
      for (int k = 0; k < sh.n_out; ++k)
        for (int i = 0; i < sh.len; ++i) {
          const T x = i % 3 == 0 ? (T)(3.0 * (double)v)
                                 : (T)((i % 3 == 1 ? -1.0 : 1.0) * (double)v * large);
          h[contiguous ? (size_t)k * sh.len + i : (size_t)i * sh.n_out + k] = x;
        }
      auto d   = raft::make_device_vector<T, int>(handle, (int)h.size());
      auto out = raft::make_device_vector<T, int>(handle, sh.n_out);
      raft::update_device(d.data_handle(), h.data(), h.size(), stream);
      auto main_op = [] __device__(T a, int) { return a; };  // a lambda: no library kernel
      auto fin_op  = [] __device__(T x) { return x; };
      for (bool inplace : {false, true}) {
        std::vector<T> before((size_t)sh.n_out, (T)1000);
        raft::update_device(out.data_handle(), before.data(), before.size(), stream);
        if (contiguous) {
          auto view = raft::make_device_matrix_view<const T, int, raft::row_major>(
            d.data_handle(), sh.n_out, sh.len);
          raft::linalg::reduce<raft::Apply::ALONG_ROWS>(handle, view, out.view(), (T)0, inplace,
                                                        main_op, raft::add_op(), fin_op);
        } else {
          auto view = raft::make_device_matrix_view<const T, int, raft::row_major>(
            d.data_handle(), sh.len, sh.n_out);
          raft::linalg::reduce<raft::Apply::ALONG_COLUMNS>(handle, view, out.view(), (T)0, inplace,
                                                           main_op, raft::add_op(), fin_op);
        }
        const double want =
          (double)(sh.len / 3) * (double)(T)(3.0 * (double)v) + (inplace ? 1000.0 : 0.0);
        auto got = to_host(out.data_handle(), (size_t)sh.n_out, stream);
        bool ok  = true;
        for (int k = 0; k < sh.n_out; ++k)
          ok &= close(got[k], want, tol);
        if (!ok)
          std::printf("    contiguous=%d n_out=%d len=%d inplace=%d got %.17g want %.17g\n",
                      (int)contiguous, sh.n_out, sh.len, (int)inplace, (double)got[0], want);
        CHECK(ok);
      }
    }
  // map over two arrays, then sum: the same pattern split over the two operands
  const int len = 3 << 20;
  std::vector<T> ha(len), hb(len);
  for (int i = 0; i < len; ++i) {
    ha[i] = i % 3 == 0 ? (T)(3.0 * (double)v) : (T)((i % 3 == 1 ? -1.0 : 1.0) * (double)v * large);
    hb[i] = (T)0;
  }
  auto da  = raft::make_device_vector<T, int>(handle, len);
  auto db  = raft::make_device_vector<T, int>(handle, len);
  auto out = raft::make_device_scalar<T>(handle);
  raft::update_device(da.data_handle(), ha.data(), ha.size(), stream);
  raft::update_device(db.data_handle(), hb.data(), hb.size(), stream);
  raft::linalg::mapReduce<T>(
    out.data_handle(), (size_t)len, (T)0, [] __device__(T a, T b) { return a + b; },
    raft::add_op(), stream, (const T*)da.data_handle(), (const T*)db.data_handle());
  CHECK(close(to_host(out.data_handle(), 1, stream)[0],
              (double)(len / 3) * (double)(T)(3.0 * (double)v), tol));
}
TEST_CASE(CompensatedLambdaSumsF) { compensated_lambda_sums<float>(1e7, 2e-7); }
TEST_CASE(CompensatedLambdaSumsD) { compensated_lambda_sums<double>(1e12, 1e-13); }

// Column reductions with the caller's functors over rows of more than 128 lane-loads: whole
// adjacent rows per workgroup (D = 4097: one piece, D = 6001: two), partials per workgroup and a
// second pass; sums through the wide accumulator, a maximum of a lambda, and an arg-max with the
// test's own functors (ties: the lowest row wins).  Row counts are the fewest that take this
// layout plus a remainder; one more case stays just below and takes the other layout.
TEST_CASE(WideColumnsLambdas)
{
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  using KVP   = raft::KeyValuePair<int, float>;
  struct shape {
    int rows, cols;
  };
  for (shape sh : {shape{8192 + 5, 4097}, shape{4096 + 3, 6001}, shape{16384 + 9, 2049}, shape{8191, 4097}}) {
    const int rows = sh.rows, cols = sh.cols;
    auto h = uniform<float>((size_t)rows * cols, -1.0, 1.0, 1000 + cols);
    for (int j = 0; j < cols; j += 97)  // planted ties for the arg-max
      h[(size_t)(rows - 1) * cols + j] = h[(size_t)(rows / 3) * cols + j] = 2.0f;
    auto d = raft::make_device_matrix<float, int, raft::row_major>(handle, rows, cols);
    raft::update_device(d.data_handle(), h.data(), h.size(), stream);
    auto sums = raft::make_device_vector<float, int>(handle, cols);
    auto maxs = raft::make_device_vector<float, int>(handle, cols);
    auto args = raft::make_device_vector<KVP, int>(handle, cols);
    const float scale = 0.5f;
    raft::linalg::strided_reduction(
      handle, raft::make_const_mdspan(d.view()), sums.view(), 0.0f, false,
      [scale] __device__(float a, int i) { return a * scale + (i % 3 == 0 ? 0.25f : 0.0f); },
      raft::add_op(), [] __device__(float x) { return 2.0f * x; });
    raft::linalg::strided_reduction(handle, raft::make_const_mdspan(d.view()), maxs.view(), -1e30f,
                                    false, [] __device__(float a, int) { return a * a; },
                                    raft::max_op());
    raft::linalg::strided_reduction(handle, raft::make_const_mdspan(d.view()), args.view(),
                                    KVP{0, -std::numeric_limits<float>::infinity()}, false,
                                    ValueToKVP<float, int>{}, ArgMaxOp<int, float>{});
    auto got_s = to_host(sums.data_handle(), (size_t)cols, stream);
    auto got_m = to_host(maxs.data_handle(), (size_t)cols, stream);
    auto got_a = to_host(args.data_handle(), (size_t)cols, stream);
    bool ok_s = true, ok_m = true, ok_a = true;
    for (int j = 0; j < cols; ++j) {
      double acc = 0;
      float mx   = -1e30f;
      int best   = 0;
      for (int i = 0; i < rows; ++i) {
        const float x = h[(size_t)i * cols + j];
        acc += (double)(x * scale + (i % 3 == 0 ? 0.25f : 0.0f));
        mx = std::max(mx, x * x);
        if (x > h[(size_t)best * cols + j]) best = i;
      }
      ok_s &= close(got_s[j], 2.0 * acc, 1e-6);
      ok_m &= got_m[j] == mx;
      ok_a &= got_a[j].key == best && got_a[j].value == h[(size_t)best * cols + j];
    }
    if (!(ok_s && ok_m && ok_a)) std::printf("    %d x %d: sums %d max %d arg %d\n", rows, cols, ok_s, ok_m, ok_a);
    CHECK(ok_s);
    CHECK(ok_m);
    CHECK(ok_a);
  }
}

int main()
{
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess || n == 0) {
    std::printf("no GPU visible\n");
    return 2;
  }
  return t::run_all();
}
