// GPU tests of the elementwise map family (raft::linalg::map / map_offset / unaryOp /
// writeOnlyUnaryOp / binaryOp), restating cpp/tests/linalg/map.cu:28-330 (three-input
// add with a scalar for float / double / a 12-byte padded type / KeyValuePairs of 4, 8
// and 16 bytes; map_offset scaling) plus lengths and pointer offsets that exercise the
// pack tail and element-aligned (not 16-byte aligned) vector accesses.
#include <raft/core/device_mdarray.hpp>
#include <raft/core/device_mdspan.hpp>
#include <raft/core/kvp.hpp>
#include <raft/linalg/binary_op.cuh>
#include <raft/linalg/map.cuh>
#include <raft/linalg/matrix_vector_op.cuh>
#include <raft/linalg/unary_op.cuh>
#include <raft/stats/mean_center.cuh>
#include <raft/util/cudart_utils.hpp>

#include <cmath>
#include <cstdint>
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

std::vector<double> uniform(size_t n, double lo, double hi, unsigned long long seed)
{
  std::mt19937_64 g(seed);
  std::uniform_real_distribution<double> d(lo, hi);
  std::vector<double> v(n);
  for (auto& x : v)
    x = d(g);
  return v;
}

// cpp/tests/linalg/map.cu:33-47: a 12-byte element (not a power of two)
struct padded_float {
  float value_;
  int padding1;
  int padding2;
  padded_float() = default;
  constexpr __host__ __device__ padded_float(const float& x) : value_(x), padding1(0), padding2(0) {}
};
constexpr __host__ __device__ padded_float operator+(const padded_float& x, const padded_float& y)
{
  return padded_float(x.value_ + y.value_);
}

using KVP4  = raft::KeyValuePair<std::int16_t, std::int16_t>;
using KVP8  = raft::KeyValuePair<int, float>;
using KVP16 = raft::KeyValuePair<std::int64_t, double>;

template <typename T>
struct Elem {  // host-side construction / comparison per element type
  static T make(double a, double) { return (T)a; }
  static double key(const T& x) { return (double)x; }
  static double val(const T&) { return 0.0; }
};
template <>
struct Elem<padded_float> {
  static padded_float make(double a, double) { return padded_float((float)a); }
  static double key(const padded_float& x) { return x.value_; }
  static double val(const padded_float&) { return 0.0; }
};
template <typename K, typename V>
struct Elem<raft::KeyValuePair<K, V>> {
  static raft::KeyValuePair<K, V> make(double a, double b)
  {
    return raft::KeyValuePair<K, V>{(K)(a * 100.0), (V)(std::is_integral_v<V> ? b * 100.0 : b)};
  }
  static double key(const raft::KeyValuePair<K, V>& x) { return (double)x.key; }
  static double val(const raft::KeyValuePair<K, V>& x) { return (double)x.value; }
};

template <typename T>
struct Add3 {  // a + b + c + scalar, for arithmetic and padded elements
  T scalar;
  __device__ T operator()(T a, T b, T c) const { return a + b + c + scalar; }
};
template <typename K, typename V>
struct Add3<raft::KeyValuePair<K, V>> {  // cpp/tests/linalg/map.cu:98-109
  raft::KeyValuePair<K, V> scalar;
  __device__ raft::KeyValuePair<K, V> operator()(raft::KeyValuePair<K, V> a,
                                                 raft::KeyValuePair<K, V> b,
                                                 raft::KeyValuePair<K, V> c) const
  {
    return raft::KeyValuePair<K, V>{static_cast<K>(a.key + b.key + c.key + scalar.key),
                                    static_cast<V>(a.value + b.value + c.value + scalar.value)};
  }
};

template <typename T, typename IdxT>
void map3(double tol, IdxT len, int shift)
{
  raft::resources handle;
  auto stream    = raft::resource::get_cuda_stream(handle);
  const size_t n = (size_t)len;
  auto a = uniform(n, -1.0, 1.0, 1), b = uniform(n, -1.0, 1.0, 2), c = uniform(n, -1.0, 1.0, 3);
  auto a2 = uniform(n, -1.0, 1.0, 4), b2 = uniform(n, -1.0, 1.0, 5), c2 = uniform(n, -1.0, 1.0, 6);
  std::vector<T> h1(n), h2(n), h3(n);
  for (size_t i = 0; i < n; ++i) {
    h1[i] = Elem<T>::make(a[i], a2[i]);
    h2[i] = Elem<T>::make(b[i], b2[i]);
    h3[i] = Elem<T>::make(c[i], c2[i]);
  }
  const T scalar = Elem<T>::make(3.2, 0.5);
  // `shift` elements of slack in front: the views start at an element-aligned address
  auto d1 = raft::make_device_vector<T, IdxT>(handle, len + shift);
  auto d2 = raft::make_device_vector<T, IdxT>(handle, len + shift);
  auto d3 = raft::make_device_vector<T, IdxT>(handle, len + shift);
  auto d0 = raft::make_device_vector<T, IdxT>(handle, len + shift);
  raft::update_device(d1.data_handle() + shift, h1.data(), n, stream);
  raft::update_device(d2.data_handle() + shift, h2.data(), n, stream);
  raft::update_device(d3.data_handle() + shift, h3.data(), n, stream);
  auto v1 = raft::make_device_vector_view<const T, IdxT>(d1.data_handle() + shift, len);
  auto v2 = raft::make_device_vector_view<const T, IdxT>(d2.data_handle() + shift, len);
  auto v3 = raft::make_device_vector_view<const T, IdxT>(d3.data_handle() + shift, len);
  auto vo = raft::make_device_vector_view<T, IdxT>(d0.data_handle() + shift, len);
  raft::linalg::map(handle, vo, Add3<T>{scalar}, v1, v2, v3);
  auto got = to_host(d0.data_handle() + shift, n, stream);
  bool ok  = true;
  for (size_t i = 0; i < n && ok; ++i) {
    const double wk = Elem<T>::key(h1[i]) + Elem<T>::key(h2[i]) + Elem<T>::key(h3[i]) +
                      Elem<T>::key(scalar);
    const double wv = Elem<T>::val(h1[i]) + Elem<T>::val(h2[i]) + Elem<T>::val(h3[i]) +
                      Elem<T>::val(scalar);
    ok = std::fabs(Elem<T>::key(got[i]) - wk) <= tol * (1 + std::fabs(wk)) &&
         std::fabs(Elem<T>::val(got[i]) - wv) <= tol * (1 + std::fabs(wv));
    if (!ok) std::printf("  mismatch at %zu (len %zu shift %d)\n", i, n, shift);
  }
  CHECK(ok);
}

template <typename T, typename IdxT>
void map3_grid(double tol)
{
  for (IdxT len : {(IdxT)1, (IdxT)7, (IdxT)1023, (IdxT)1024, (IdxT)4099, (IdxT)(1024 * 1024),
                   (IdxT)(1024 * 1024 + 3)})
    for (int shift : {0, 1, 3})
      map3<T, IdxT>(tol, len, shift);
}

}  // namespace

TEST_CASE(MapFloatI32) { map3_grid<float, int>(1e-6); }
TEST_CASE(MapFloatSizeT) { map3_grid<float, size_t>(1e-6); }
TEST_CASE(MapDoubleI32) { map3_grid<double, int>(1e-12); }
TEST_CASE(MapDoubleSizeT) { map3_grid<double, size_t>(1e-12); }
TEST_CASE(MapPaddedFloat) { map3_grid<padded_float, int>(1e-6); }
TEST_CASE(MapKVP4) { map3_grid<KVP4, int>(0.0); }
TEST_CASE(MapKVP8) { map3_grid<KVP8, int>(1e-6); }
TEST_CASE(MapKVP16) { map3_grid<KVP16, int>(1e-12); }

// float inputs, double output (cpp/tests/linalg/map.cu:185-187): the widest type sets the pack
TEST_CASE(MapFloatToDouble)
{
  raft::resources handle;
  auto stream   = raft::resource::get_cuda_stream(handle);
  const int len = 1024 * 1024 + 5;
  auto a = uniform(len, -1.0, 1.0, 11), b = uniform(len, -1.0, 1.0, 12);
  std::vector<float> h1(a.begin(), a.end()), h2(b.begin(), b.end());
  auto d1 = raft::make_device_vector<float, int>(handle, len);
  auto d2 = raft::make_device_vector<float, int>(handle, len);
  auto d0 = raft::make_device_vector<double, int>(handle, len);
  raft::update_device(d1.data_handle(), h1.data(), h1.size(), stream);
  raft::update_device(d2.data_handle(), h2.data(), h2.size(), stream);
  raft::linalg::map(handle, raft::make_const_mdspan(d1.view()), raft::make_const_mdspan(d2.view()),
                    d0.view(), [] __device__(float x, float y) { return (double)x * (double)y; });
  auto got = to_host(d0.data_handle(), (size_t)len, stream);
  bool ok  = true;
  for (int i = 0; i < len; ++i)
    ok &= got[i] == (double)h1[i] * (double)h2[i];
  CHECK(ok);
}

// cpp/tests/linalg/map.cu:120-175 (MapOffsetTest): out[i] = i * scalar, no inputs; and
// with an input
TEST_CASE(MapOffset)
{
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  for (int len : {1, 5, 1000, 1024 * 1024 + 1}) {
    auto d0            = raft::make_device_vector<float, int>(handle, len);
    const float scalar = 2.5f;
    raft::linalg::map_offset(handle, d0.view(),
                             [scalar] __device__(int idx) { return (float)idx * scalar; });
    auto got = to_host(d0.data_handle(), (size_t)len, stream);
    bool ok  = true;
    for (int i = 0; i < len; ++i)
      ok &= got[i] == (float)i * scalar;
    CHECK(ok);
    auto d1 = raft::make_device_vector<float, int>(handle, len);
    raft::linalg::map_offset(handle, raft::make_const_mdspan(d0.view()), d1.view(),
                             [] __device__(int idx, float x) { return x + (float)(idx & 7); });
    auto got2 = to_host(d1.data_handle(), (size_t)len, stream);
    ok        = true;
    for (int i = 0; i < len; ++i)
      ok &= got2[i] == got[i] + (float)(i & 7);
    CHECK(ok);
  }
}

// unaryOp / writeOnlyUnaryOp / binaryOp (cpp/tests/linalg/unary_op.cu, binary_op.cu), and
// an in-place call (out aliases in1)
TEST_CASE(UnaryBinaryOps)
{
  raft::resources handle;
  auto stream   = raft::resource::get_cuda_stream(handle);
  const int len = 100003;
  auto a        = uniform(len, -1.0, 1.0, 21);
  std::vector<float> h(a.begin(), a.end());
  auto din  = raft::make_device_vector<float, int>(handle, len);
  auto dout = raft::make_device_vector<float, int>(handle, len);
  raft::update_device(din.data_handle(), h.data(), h.size(), stream);
  const float s = 1.5f;
  raft::linalg::unaryOp(dout.data_handle(), din.data_handle(), len,
                        [s] __device__(float x) { return x * s; }, stream);
  auto got = to_host(dout.data_handle(), (size_t)len, stream);
  bool ok  = true;
  for (int i = 0; i < len; ++i)
    ok &= got[i] == h[i] * s;
  CHECK(ok);

  raft::linalg::writeOnlyUnaryOp(dout.data_handle(), len,
                                 [s] __device__(float* out, int idx) { *out = s * (float)idx; },
                                 stream);
  got = to_host(dout.data_handle(), (size_t)len, stream);
  ok  = true;
  for (int i = 0; i < len; ++i)
    ok &= got[i] == s * (float)i;
  CHECK(ok);

  // in place: din = din + dout
  raft::linalg::binaryOp(din.data_handle(), din.data_handle(), dout.data_handle(), len,
                         [] __device__(float x, float y) { return x + y; }, stream);
  auto got2 = to_host(din.data_handle(), (size_t)len, stream);
  ok        = true;
  for (int i = 0; i < len; ++i)
    ok &= got2[i] == h[i] + got[i];
  CHECK(ok);

  // mdspan forms
  raft::linalg::unary_op(handle, raft::make_const_mdspan(dout.view()), din.view(),
                         [] __device__(float x) { return -x; });
  got2 = to_host(din.data_handle(), (size_t)len, stream);
  ok   = true;
  for (int i = 0; i < len; ++i)
    ok &= got2[i] == -got[i];
  CHECK(ok);
}

// "All inputs must be contiguous and have the same size as the output"
// (linalg/detail/map.cuh:174-180)
TEST_CASE(MapShapeMismatchThrows)
{
  raft::resources handle;
  auto a = raft::make_device_vector<float, int>(handle, 10);
  auto b = raft::make_device_vector<float, int>(handle, 11);
  bool threw = false;
  try {
    raft::linalg::map(handle, raft::make_const_mdspan(a.view()), b.view(),
                      [] __device__(float x) { return x; });
  } catch (const raft::logic_error&) {
    threw = true;
  }
  CHECK(threw);
}

// linalg::matrixVectorOp with one and two vectors: the grid of
// cpp/tests/linalg/matrix_vector_op.cu:213-218 (1024 x {32, 64}, both layouts, both
// broadcast directions, input and output pointers 0..2 elements off), the naive kernels of
// cpp/tests/linalg/matrix_vector_op.cuh:15-105 as the check, plus ragged shapes.
template <typename T, typename IdxT>
void matvec_grid(double tol)
{
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  struct Shape { IdxT rows, cols; };
  std::vector<Shape> shapes = {{1024, 32}, {1024, 64}, {2500, 250}, {1000, 33}, {7, 5}, {3, 100003},
                               {4099, 1}, {1, 777}, {300, 1028}};
  for (auto sh : shapes)
    for (int rm = 0; rm < 2; ++rm)
      for (int bcast = 0; bcast < 2; ++bcast)
        for (int in_off = 0; in_off < 3; ++in_off)
          for (int out_off = 0; out_off < 3; out_off += 2) {
            const size_t len = (size_t)sh.rows * sh.cols;
            const size_t vlen = bcast ? sh.cols : sh.rows;
            std::mt19937_64 g(len + rm * 7 + bcast * 3 + in_off);
            std::uniform_real_distribution<double> u(-1.0, 1.0);
            std::vector<T> hm(len), hv1(vlen), hv2(vlen);
            for (auto& x : hm) x = (T)u(g);
            for (auto& x : hv1) x = (T)u(g);
            for (auto& x : hv2) x = (T)u(g);
            auto dm  = raft::make_device_vector<T, size_t>(handle, len + 4);
            auto dv1 = raft::make_device_vector<T, size_t>(handle, vlen);
            auto dv2 = raft::make_device_vector<T, size_t>(handle, vlen);
            auto dout = raft::make_device_vector<T, size_t>(handle, len + 4);
            raft::update_device(dm.data_handle() + in_off, hm.data(), len, stream);
            raft::update_device(dv1.data_handle(), hv1.data(), vlen, stream);
            raft::update_device(dv2.data_handle(), hv2.data(), vlen, stream);
            const T* in = dm.data_handle() + in_off;
            T* out      = dout.data_handle() + out_off;
            auto vec_of = [&](size_t idx) {
              const size_t D = sh.cols, N = sh.rows;
              if (rm && bcast) return idx % D;
              if (!rm && !bcast) return idx % N;
              if (rm && !bcast) return idx / D;
              return idx / N;
            };
            for (int two = 0; two < 2; ++two) {
              auto add1 = [] __device__(T a, T b) { return a + b; };
              auto add2 = [] __device__(T a, T b, T c) { return a + b + c; };
              if (rm && bcast) {
                if (two) raft::linalg::matrixVectorOp<true, true>(out, in, dv1.data_handle(), dv2.data_handle(), sh.cols, sh.rows, add2, stream);
                else raft::linalg::matrixVectorOp<true, true>(out, in, dv1.data_handle(), sh.cols, sh.rows, add1, stream);
              } else if (rm && !bcast) {
                if (two) raft::linalg::matrixVectorOp<true, false>(out, in, dv1.data_handle(), dv2.data_handle(), sh.cols, sh.rows, add2, stream);
                else raft::linalg::matrixVectorOp<true, false>(out, in, dv1.data_handle(), sh.cols, sh.rows, add1, stream);
              } else if (!rm && bcast) {
                if (two) raft::linalg::matrixVectorOp<false, true>(out, in, dv1.data_handle(), dv2.data_handle(), sh.cols, sh.rows, add2, stream);
                else raft::linalg::matrixVectorOp<false, true>(out, in, dv1.data_handle(), sh.cols, sh.rows, add1, stream);
              } else {
                if (two) raft::linalg::matrixVectorOp<false, false>(out, in, dv1.data_handle(), dv2.data_handle(), sh.cols, sh.rows, add2, stream);
                else raft::linalg::matrixVectorOp<false, false>(out, in, dv1.data_handle(), sh.cols, sh.rows, add1, stream);
              }
              auto got = to_host(out, len, stream);
              bool ok  = true;
              for (size_t i = 0; i < len; ++i) {
                const size_t k = vec_of(i);
                const double want = (double)hm[i] + (double)hv1[k] + (two ? (double)hv2[k] : 0.0);
                ok &= std::fabs((double)got[i] - want) <= tol * (1.0 + std::fabs(want));
              }
              if (!ok)
                std::printf("  matvec %lldx%lld rm=%d bcast=%d in+%d out+%d vecs=%d\n", (long long)sh.rows,
                            (long long)sh.cols, rm, bcast, in_off, out_off, two + 1);
              CHECK(ok);
            }
          }
}
TEST_CASE(MatVecOpFloatI32) { matvec_grid<float, int>(1e-5); }
TEST_CASE(MatVecOpDoubleI64) { matvec_grid<double, std::int64_t>(1e-7); }

// stats::mean_center / mean_add through the mdspan API: the grid of
// cpp/tests/stats/mean_center.cu:110-122 (1024 x {32, 64, 128}, both layouts, both
// directions), in place as well
template <typename T>
void mean_center_grid(double tol)
{
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  for (int cols : {32, 64, 128, 37})
    for (int rm = 0; rm < 2; ++rm)
      for (int bcast = 0; bcast < 2; ++bcast) {
        const int rows = 1024;
        const size_t len = (size_t)rows * cols, vlen = bcast ? cols : rows;
        std::mt19937_64 g(cols + rm + bcast);
        std::normal_distribution<double> nd(-1.0, 1.0);
        std::vector<T> hm(len), hmu(vlen);
        for (auto& x : hm) x = (T)nd(g);
        for (auto& x : hmu) x = (T)nd(g);
        auto dm  = raft::make_device_vector<T, int>(handle, (int)len);
        auto dmu = raft::make_device_vector<T, int>(handle, (int)vlen);
        auto dout = raft::make_device_vector<T, int>(handle, (int)len);
        raft::update_device(dm.data_handle(), hm.data(), len, stream);
        raft::update_device(dmu.data_handle(), hmu.data(), vlen, stream);
        auto mu = raft::make_device_vector_view<const T, int>(dmu.data_handle(), (int)vlen);
        auto run = [&](auto layout, bool add) {
          using L = decltype(layout);
          auto in  = raft::make_device_matrix_view<const T, int, L>(dm.data_handle(), rows, cols);
          auto out = raft::make_device_matrix_view<T, int, L>(dout.data_handle(), rows, cols);
          if (bcast) {
            if (add) raft::stats::mean_add<raft::Apply::ALONG_ROWS>(handle, in, mu, out);
            else raft::stats::mean_center<raft::Apply::ALONG_ROWS>(handle, in, mu, out);
          } else {
            if (add) raft::stats::mean_add<raft::Apply::ALONG_COLUMNS>(handle, in, mu, out);
            else raft::stats::mean_center<raft::Apply::ALONG_COLUMNS>(handle, in, mu, out);
          }
        };
        for (int add = 0; add < 2; ++add) {
          if (rm) run(raft::row_major{}, add); else run(raft::col_major{}, add);
          auto got = to_host(dout.data_handle(), len, stream);
          bool ok  = true;
          for (size_t i = 0; i < len; ++i) {
            const size_t r = rm ? i / cols : i % rows, c = rm ? i % cols : i / rows;
            const double m = (double)hmu[bcast ? c : r];
            const double want = (double)hm[i] + (add ? m : -m);
            ok &= std::fabs((double)got[i] - want) <= tol * (1.0 + std::fabs(want));
          }
          if (!ok) std::printf("  mean_%s 1024x%d rm=%d bcast=%d\n", add ? "add" : "center", cols, rm, bcast);
          CHECK(ok);
        }
      }
}
// out == matrix (linalg/matrix_vector_op.cuh:38 allows it), on row lengths with and without
// elements after the last whole 16-byte pack
TEST_CASE(MatVecOpInPlace)
{
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  for (auto [rows, cols] : std::vector<std::pair<int, int>>{{3000, 13}, {1000, 129}, {513, 64}, {20000, 3}, {7, 4099}})
    for (int bcast = 0; bcast < 2; ++bcast) {
      const size_t len = (size_t)rows * cols, vlen = bcast ? cols : rows;
      auto hm = std::vector<float>(len);
      auto hv = std::vector<float>(vlen);
      std::mt19937 g(rows + cols);
      std::uniform_real_distribution<float> u(-1.f, 1.f);
      for (auto& x : hm) x = u(g);
      for (auto& x : hv) x = u(g);
      auto dm = raft::make_device_vector<float, int>(handle, (int)len);
      auto dv = raft::make_device_vector<float, int>(handle, (int)vlen);
      raft::update_device(dm.data_handle(), hm.data(), len, stream);
      raft::update_device(dv.data_handle(), hv.data(), vlen, stream);
      auto op = [] __device__(float a, float b) { return 2.f * a - b; };
      if (bcast)
        raft::linalg::matrixVectorOp<true, true>(dm.data_handle(), dm.data_handle(), dv.data_handle(), cols, rows, op, stream);
      else
        raft::linalg::matrixVectorOp<true, false>(dm.data_handle(), dm.data_handle(), dv.data_handle(), cols, rows, op, stream);
      auto got = to_host(dm.data_handle(), len, stream);
      bool ok  = true;
      for (size_t i = 0; i < len; ++i)
        ok &= got[i] == 2.f * hm[i] - hv[bcast ? i % cols : i / cols];
      if (!ok) std::printf("  in place %dx%d bcast=%d\n", rows, cols, bcast);
      CHECK(ok);
    }
}

TEST_CASE(MeanCenterF) { mean_center_grid<float>(1e-6); }
TEST_CASE(MeanCenterD) { mean_center_grid<double>(1e-14); }

int main()
{
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess || n == 0) {
    std::printf("no GPU visible\n");
    return 2;
  }
  return t::run_all();
}
