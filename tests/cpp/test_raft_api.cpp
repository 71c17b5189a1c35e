// GPU tests of the C++ API layer: the reference's reduction-path tests restated
// against the same names and signatures (raft::linalg::reduce, coalesced_reduction,
// strided_reduction, norm, map_reduce, raft::stats::mean / stddev / vars / sum,
// raft::matrix::argmax / argmin).  Expected values come from a sequential host
// evaluation in double precision written here (the reference compares with naive
// one-thread-per-output kernels, cpp/tests/linalg/reduce.cuh:27-178) and from the
// reference's literal fixtures.
#include <raft/core/device_mdarray.hpp>
#include <raft/core/device_mdspan.hpp>
#include <raft/core/device_resources.hpp>
#include <raft/core/operators.hpp>
#include <raft/linalg/coalesced_reduction.cuh>
#include <raft/linalg/map_reduce.cuh>
#include <raft/linalg/map_then_reduce.cuh>
#include <raft/linalg/norm.cuh>
#include <raft/linalg/normalize.cuh>
#include <raft/linalg/reduce.cuh>
#include <raft/linalg/strided_reduction.cuh>
#include <raft/matrix/argmax.cuh>
#include <raft/matrix/argmin.cuh>
#include <raft/stats/cov.cuh>
#include <raft/stats/mean.cuh>
#include <raft/stats/meanvar.cuh>
#include <raft/stats/stddev.cuh>
#include <raft/stats/sum.cuh>
#include <raft/util/cudart_utils.hpp>
#include <raft/util/itertools.hpp>

#include <chrono>
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

template <typename T>
std::vector<T> normal(size_t n, double mu, double sigma, unsigned long long seed)
{
  std::mt19937_64 g(seed);
  std::normal_distribution<double> d(mu, sigma);
  std::vector<T> v(n);
  for (auto& x : v)
    x = (T)d(g);
  return v;
}

// element (i, j) of an N x D matrix
inline size_t at(bool row_major, size_t N, size_t D, size_t i, size_t j)
{
  return row_major ? i * D + j : i + j * N;
}

// dots = final(inplace ? red(old, fold) : fold), fold in double
template <typename In, typename Main, typename Red, typename Fin>
std::vector<double> host_reduce(const std::vector<In>& data, size_t N, size_t D, bool row_major,
                                bool along_rows, double init, const std::vector<double>* old,
                                Main main_op, Red red_op, Fin fin_op)
{
  const size_t n_out = along_rows ? N : D, len = along_rows ? D : N;
  std::vector<double> out(n_out);
  for (size_t k = 0; k < n_out; ++k) {
    double acc = init;
    for (size_t r = 0; r < len; ++r) {
      const size_t idx = along_rows ? at(row_major, N, D, k, r) : at(row_major, N, D, r, k);
      acc              = red_op(acc, main_op((double)data[idx], (int)r));
    }
    if (old) acc = red_op((*old)[k], acc);
    out[k] = fin_op(acc);
  }
  return out;
}

template <typename T>
bool all_close(const std::vector<T>& got, const std::vector<double>& want, double eps)
{
  if (got.size() != want.size()) return false;
  t::CompareApprox<double> cmp(eps);
  for (size_t i = 0; i < got.size(); ++i)
    if (!cmp((double)got[i], want[i])) {
      std::printf("  mismatch at %zu: got %.9g want %.9g\n", i, (double)got[i], want[i]);
      return false;
    }
  return true;
}

// ---------------------------------------------------------------------------
// cpp/tests/linalg/reduce.cu:106-178 simpleTest
// ---------------------------------------------------------------------------
template <typename T>
void simple_max()
{
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  std::vector<T> data_h{1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12};
  const std::uint32_t rows = 3, cols = 4;
  for (int along_rows = 0; along_rows < 2; ++along_rows) {
    auto output = raft::make_device_vector<T, std::uint32_t>(handle, along_rows ? rows : cols);
    {
      auto data = raft::make_device_matrix<T, std::uint32_t, raft::row_major>(handle, rows, cols);
      raft::copy(data.data_handle(), data_h.data(), data.size(), stream);
      std::vector<T> want;
      if (along_rows) {
        raft::linalg::reduce<raft::Apply::ALONG_ROWS>(handle, raft::make_const_mdspan(data.view()),
                                                      output.view(), T(0), false,
                                                      raft::identity_op(), raft::max_op(),
                                                      raft::identity_op());
        want = {4, 8, 12};
      } else {
        raft::linalg::reduce<raft::Apply::ALONG_COLUMNS>(
          handle, raft::make_const_mdspan(data.view()), output.view(), T(0), false,
          raft::identity_op(), raft::max_op(), raft::identity_op());
        want = {9, 10, 11, 12};
      }
      CHECK(to_host(output.data_handle(), want.size(), stream) == want);
    }
    {
      auto data = raft::make_device_matrix<T, std::uint32_t, raft::col_major>(handle, rows, cols);
      raft::copy(data.data_handle(), data_h.data(), data.size(), stream);
      std::vector<T> want;
      if (along_rows) {
        raft::linalg::reduce<raft::Apply::ALONG_ROWS>(handle, raft::make_const_mdspan(data.view()),
                                                      output.view(), T(0), false,
                                                      raft::identity_op(), raft::max_op(),
                                                      raft::identity_op());
        want = {10, 11, 12};
      } else {
        raft::linalg::reduce<raft::Apply::ALONG_COLUMNS>(
          handle, raft::make_const_mdspan(data.view()), output.view(), T(0), false,
          raft::identity_op(), raft::max_op(), raft::identity_op());
        want = {3, 6, 9, 12};
      }
      CHECK(to_host(output.data_handle(), want.size(), stream) == want);
    }
  }
}

// ---------------------------------------------------------------------------
// cpp/tests/linalg/reduce.cu:180-341 fullTest: sq_op / add_op / sqrt_op, first
// inplace=false then inplace=true on the same output.
// ---------------------------------------------------------------------------
template <typename In, typename Out, typename Idx>
void reduce_full(double tol, std::vector<int> rows_list, std::vector<int> cols_list)
{
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  for (int rows : rows_list)
    for (int cols : cols_list)
      for (int rm = 0; rm < 2; ++rm)
        for (int ar = 0; ar < 2; ++ar) {
          const size_t len = (size_t)rows * cols;
          auto data_h      = uniform<In>(len, -1.0, 1.0, 1234);
          const Idx n_out  = ar ? rows : cols;
          auto data_d      = raft::make_device_vector<In, Idx>(handle, (Idx)len);
          auto dots        = raft::make_device_vector<Out, Idx>(handle, n_out);
          raft::update_device(data_d.data_handle(), data_h.data(), len, stream);
          auto sq   = [](double x, int) { return x * x; };
          auto add  = [](double a, double b) { return a + b; };
          auto sqr  = [](double x) { return std::sqrt(x); };
          auto run  = [&](bool inplace) {
            auto out_view = raft::make_device_vector_view<Out, Idx>(dots.data_handle(), n_out);
            if (rm) {
              auto v = raft::make_device_matrix_view<const In, Idx, raft::row_major>(
                data_d.data_handle(), (Idx)rows, (Idx)cols);
              if (ar) {
                raft::linalg::reduce<raft::Apply::ALONG_ROWS>(handle, v, out_view, Out(0), inplace,
                                                              raft::sq_op(), raft::add_op(),
                                                              raft::sqrt_op());
              } else {
                raft::linalg::reduce<raft::Apply::ALONG_COLUMNS>(handle, v, out_view, Out(0),
                                                                 inplace, raft::sq_op(),
                                                                 raft::add_op(), raft::sqrt_op());
              }
            } else {
              auto v = raft::make_device_matrix_view<const In, Idx, raft::col_major>(
                data_d.data_handle(), (Idx)rows, (Idx)cols);
              if (ar) {
                raft::linalg::reduce<raft::Apply::ALONG_ROWS>(handle, v, out_view, Out(0), inplace,
                                                              raft::sq_op(), raft::add_op(),
                                                              raft::sqrt_op());
              } else {
                raft::linalg::reduce<raft::Apply::ALONG_COLUMNS>(handle, v, out_view, Out(0),
                                                                 inplace, raft::sq_op(),
                                                                 raft::add_op(), raft::sqrt_op());
              }
            }
          };
          run(false);
          auto first = to_host(dots.data_handle(), (size_t)n_out, stream);
          auto want  = host_reduce(data_h, rows, cols, rm, ar, 0.0, nullptr, sq, add, sqr);
          CHECK(all_close(first, want, tol));
          run(true);
          std::vector<double> old(first.begin(), first.end());
          auto want2 = host_reduce(data_h, rows, cols, rm, ar, 0.0, &old, sq, add, sqr);
          CHECK(all_close(to_host(dots.data_handle(), (size_t)n_out, stream), want2, tol));
        }
}

// ---------------------------------------------------------------------------
// cpp/tests/linalg/reduce.cu:343-411: key-value arg-max through reduce().
// ---------------------------------------------------------------------------
template <typename T>
void reduce_kvp()
{
  using KVP = raft::KeyValuePair<int, T>;
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  for (int rows : {11, 1234})
    for (int cols : {7, 33, 128, 500}) {
      auto data_h = uniform<T>((size_t)rows * cols, -1.0, 1.0, 1234);
      // exact ties: the lowest index must win
      for (int r = 0; r < rows; r += 3) {
        const int a = (r * 7) % cols, b = (r * 13 + 5) % cols;
        data_h[(size_t)r * cols + a] = data_h[(size_t)r * cols + b] = T(2);
      }
      auto data = raft::make_device_matrix<T, int, raft::row_major>(handle, rows, cols);
      auto dots = raft::make_device_vector<KVP, int>(handle, rows);
      raft::update_device(data.data_handle(), data_h.data(), data_h.size(), stream);
      raft::linalg::reduce<raft::Apply::ALONG_ROWS>(
        handle, raft::make_const_mdspan(data.view()), dots.view(),
        KVP(0, -std::numeric_limits<T>::infinity()), false, raft::value_to_kvp_op<int>(),
        raft::argmax_op(), raft::identity_op());
      auto got = to_host(dots.data_handle(), (size_t)rows, stream);
      bool ok  = true;
      for (int r = 0; r < rows; ++r) {
        int best = 0;
        for (int j = 1; j < cols; ++j)
          if (data_h[(size_t)r * cols + j] > data_h[(size_t)r * cols + best]) best = j;
        ok &= got[r].key == best && got[r].value == data_h[(size_t)r * cols + best];
      }
      CHECK(ok);
    }
}

// ---------------------------------------------------------------------------
// cpp/tests/linalg/coalesced_reduction.cu, strided_reduction.cu
// ---------------------------------------------------------------------------
template <typename T>
void coalesced_and_strided(double tol)
{
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  auto sq     = [](double x, int) { return x * x; };
  auto add    = [](double a, double b) { return a + b; };
  auto idf    = [](double x) { return x; };
  const std::vector<std::pair<int, int>> shapes = {{10000, 3}, {10000, 17}, {10000, 32},
                                                   {10000, 270}, {10, 25000}, {1024, 64},
                                                   {1024, 256}, {9, 100000}};
  for (auto [rows, cols] : shapes) {
    auto data_h = uniform<T>((size_t)rows * cols, -1.0, 1.0, 1234);
    auto data   = raft::make_device_matrix<T, int, raft::row_major>(handle, rows, cols);
    raft::update_device(data.data_handle(), data_h.data(), data_h.size(), stream);
    auto by_row = raft::make_device_vector<T, int>(handle, rows);
    auto by_col = raft::make_device_vector<T, int>(handle, cols);
    raft::linalg::coalesced_reduction(handle, raft::make_const_mdspan(data.view()), by_row.view(),
                                      T(0), false, raft::sq_op());
    CHECK(all_close(to_host(by_row.data_handle(), (size_t)rows, stream),
                    host_reduce(data_h, rows, cols, true, true, 0.0, nullptr, sq, add, idf), tol));
    raft::linalg::strided_reduction(handle, raft::make_const_mdspan(data.view()), by_col.view(),
                                    T(0), false, raft::sq_op());
    CHECK(all_close(to_host(by_col.data_handle(), (size_t)cols, stream),
                    host_reduce(data_h, rows, cols, true, false, 0.0, nullptr, sq, add, idf), tol));
    // pointer forms on a bare stream
    raft::linalg::coalescedReduction(by_row.data_handle(), data.data_handle(), cols, rows, T(0),
                                     stream, false, raft::abs_op());
    auto absm = [](double x, int) { return std::fabs(x); };
    CHECK(all_close(to_host(by_row.data_handle(), (size_t)rows, stream),
                    host_reduce(data_h, rows, cols, true, true, 0.0, nullptr, absm, add, idf),
                    tol));
    raft::linalg::stridedReduction(by_col.data_handle(), data.data_handle(), cols, rows, T(0),
                                   stream, false, raft::abs_op());
    CHECK(all_close(to_host(by_col.data_handle(), (size_t)cols, stream),
                    host_reduce(data_h, rows, cols, true, false, 0.0, nullptr, absm, add, idf),
                    tol));
  }
}

// ---------------------------------------------------------------------------
// cpp/tests/linalg/norm.cu: L1 / L2 / Linf, rows and columns, with and without sqrt
// ---------------------------------------------------------------------------
template <typename T, typename OutT>
void norms(double tol)
{
  using namespace raft::linalg;
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  auto add    = [](double a, double b) { return a + b; };
  auto mx     = [](double a, double b) { return std::max(a, b); };
  auto idf    = [](double x) { return x; };
  auto sqr    = [](double x) { return std::sqrt(x); };
  auto sq     = [](double x, int) { return x * x; };
  auto ab     = [](double x, int) { return std::fabs(x); };
  for (auto [rows, cols] : std::vector<std::pair<int, int>>{{4, 8}, {1024, 32}, {1024, 64},
                                                            {1000, 100}, {37, 1024}}) {
    auto data_h = uniform<T>((size_t)rows * cols, -10.0, 10.0, 1234);
    auto data   = raft::make_device_matrix<T, int, raft::row_major>(handle, rows, cols);
    raft::update_device(data.data_handle(), data_h.data(), data_h.size(), stream);
    auto in     = raft::make_const_mdspan(data.view());
    auto by_row = raft::make_device_vector<OutT, int>(handle, rows);
    auto by_col = raft::make_device_vector<OutT, int>(handle, cols);
    auto rows_h = [&] { return to_host(by_row.data_handle(), (size_t)rows, stream); };
    auto cols_h = [&] { return to_host(by_col.data_handle(), (size_t)cols, stream); };

    norm<L1Norm, raft::Apply::ALONG_ROWS>(handle, in, by_row.view());
    CHECK(all_close(rows_h(), host_reduce(data_h, rows, cols, true, true, 0, nullptr, ab, add, idf), tol));
    norm<L2Norm, raft::Apply::ALONG_ROWS>(handle, in, by_row.view());
    CHECK(all_close(rows_h(), host_reduce(data_h, rows, cols, true, true, 0, nullptr, sq, add, idf), tol));
    norm<L2Norm, raft::Apply::ALONG_ROWS>(handle, in, by_row.view(), raft::sqrt_op());
    CHECK(all_close(rows_h(), host_reduce(data_h, rows, cols, true, true, 0, nullptr, sq, add, sqr), tol));
    norm<LinfNorm, raft::Apply::ALONG_ROWS>(handle, in, by_row.view());
    CHECK(all_close(rows_h(), host_reduce(data_h, rows, cols, true, true, 0, nullptr, ab, mx, idf), tol));
    norm<L1Norm, raft::Apply::ALONG_COLUMNS>(handle, in, by_col.view());
    CHECK(all_close(cols_h(), host_reduce(data_h, rows, cols, true, false, 0, nullptr, ab, add, idf), tol));
    norm<L2Norm, raft::Apply::ALONG_COLUMNS>(handle, in, by_col.view(), raft::sqrt_op());
    CHECK(all_close(cols_h(), host_reduce(data_h, rows, cols, true, false, 0, nullptr, sq, add, sqr), tol));
    norm<LinfNorm, raft::Apply::ALONG_COLUMNS>(handle, in, by_col.view());
    CHECK(all_close(cols_h(), host_reduce(data_h, rows, cols, true, false, 0, nullptr, ab, mx, idf), tol));
    // pointer forms
    rowNorm<L2Norm, true>(by_row.data_handle(), data.data_handle(), cols, rows, stream,
                          raft::sqrt_op());
    CHECK(all_close(rows_h(), host_reduce(data_h, rows, cols, true, true, 0, nullptr, sq, add, sqr), tol));
    colNorm<L1Norm, true>(by_col.data_handle(), data.data_handle(), cols, rows, stream);
    CHECK(all_close(cols_h(), host_reduce(data_h, rows, cols, true, false, 0, nullptr, ab, add, idf), tol));
  }
}

// ---------------------------------------------------------------------------
// cpp/tests/stats/mean.cu, stddev.cu, sum.cu
// ---------------------------------------------------------------------------
template <typename T>
void mean_stddev(double tol)
{
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  for (int rm = 0; rm < 2; ++rm)
    for (auto [rows, cols] : std::vector<std::pair<int, int>>{{1024, 32}, {1024, 64}, {1024, 128},
                                                              {1024, 256}, {100000, 2}, {31, 1},
                                                              {1, 257}}) {
      auto data_h = normal<T>((size_t)rows * cols, 1.0, 2.0, 1234);
      auto data_d = raft::make_device_vector<T, int>(handle, rows * cols);
      raft::update_device(data_d.data_handle(), data_h.data(), data_h.size(), stream);
      auto mu  = raft::make_device_vector<T, int>(handle, cols);
      auto sd  = raft::make_device_vector<T, int>(handle, cols);
      auto var = raft::make_device_vector<T, int>(handle, cols);
      auto sm  = raft::make_device_vector<T, int>(handle, cols);
      auto mu_c = raft::make_device_vector_view<const T, int>(mu.data_handle(), cols);
      std::vector<double> want_mu(cols, 0.0), want_sum(cols, 0.0);
      for (int j = 0; j < cols; ++j) {
        double s = 0;
        for (int i = 0; i < rows; ++i)
          s += (double)data_h[at(rm, rows, cols, i, j)];
        want_sum[j] = s;
        want_mu[j]  = s / rows;
      }
      for (int sample = 0; sample < 2; ++sample) {
        if (sample && rows == 1) continue;
        if (rm) {
          auto v = raft::make_device_matrix_view<const T, int, raft::row_major>(
            data_d.data_handle(), rows, cols);
          raft::stats::mean(handle, v, mu.view());
          raft::stats::stddev(handle, v, mu_c, sd.view(), (bool)sample);
          raft::stats::vars(handle, v, mu_c, var.view(), (bool)sample);
          raft::stats::sum(handle, v, sm.view());
        } else {
          auto v = raft::make_device_matrix_view<const T, int, raft::col_major>(
            data_d.data_handle(), rows, cols);
          raft::stats::mean(handle, v, mu.view());
          raft::stats::stddev(handle, v, mu_c, sd.view(), (bool)sample);
          raft::stats::vars(handle, v, mu_c, var.view(), (bool)sample);
          raft::stats::sum(handle, v, sm.view());
        }
        auto mu_h = to_host(mu.data_handle(), (size_t)cols, stream);
        CHECK(all_close(mu_h, want_mu, tol));
        CHECK(all_close(to_host(sm.data_handle(), (size_t)cols, stream), want_sum, tol));
        std::vector<double> want_sd(cols), want_var(cols);
        for (int j = 0; j < cols; ++j) {
          double ss = 0;
          for (int i = 0; i < rows; ++i) {
            const double x = (double)data_h[at(rm, rows, cols, i, j)];
            ss += x * x;
          }
          const double r  = 1.0 / (sample ? rows - 1 : rows);
          const double rmn = sample ? r * rows : 1.0;
          want_var[j]     = std::fabs(ss * r - (double)mu_h[j] * (double)mu_h[j] * rmn);
          want_sd[j]      = std::sqrt(want_var[j]);
        }
        // E[x^2] - mu^2 cancels: the reference checks stddev to 1e-1 of the generator's
        // sigma (cpp/tests/stats/stddev.cu:120-182); here against the same formula in fp64
        const double tol_sd = std::is_same_v<T, float> ? 2e-3 : 1e-7;
        auto sd_h  = to_host(sd.data_handle(), (size_t)cols, stream);
        auto var_h = to_host(var.data_handle(), (size_t)cols, stream);
        CHECK(all_close(sd_h, want_sd, tol_sd));
        CHECK(all_close(var_h, want_var, tol_sd));
        // cpp/tests/stats/stddev.cu:198-202: sqrt(vars) == stddev
        bool same = true;
        for (int j = 0; j < cols; ++j)
          same &= std::fabs(std::sqrt((double)var_h[j]) - (double)sd_h[j]) <= 1e-6 * (1 + sd_h[j]);
        CHECK(same);
      }
    }
}

// ---------------------------------------------------------------------------
// cpp/tests/stats/meanvar.cu:20-150: normal data, both layouts, sample and population
// variance, checked by the reference's statistical bounds (mean_tol, var_tol with
// N_SIGMAS = 6) and against a two-pass fp64 evaluation
// ---------------------------------------------------------------------------
template <typename T>
void meanvar_cases(double tol)
{
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  struct Case { double mean, stddev; int rows, cols; bool sample, row_major; };
  std::vector<Case> cases;
  for (bool rm : {false, true})
    for (int cols : {32, 64, 128, 256, 257}) {
      cases.push_back({1.0, 2.0, 1024, cols, true, rm});
      cases.push_back({-1.0, 2.0, 1024, cols, false, rm});
    }
  cases.push_back({-1.0, 2.0, 700, 13, false, true});
  cases.push_back({10.0, 2.0, 50000, 811, false, true});
  cases.push_back({3.0, 1.0, 1, 9, true, true});
  for (const auto& c : cases) {
    const size_t n = (size_t)c.rows * c.cols;
    auto data_h    = normal<T>(n, c.mean, c.stddev, 1234);
    auto data_d    = raft::make_device_vector<T, int>(handle, (int)n);
    raft::update_device(data_d.data_handle(), data_h.data(), n, stream);
    auto mean = raft::make_device_vector<T, int>(handle, c.cols);
    auto var  = raft::make_device_vector<T, int>(handle, c.cols);
    if (c.row_major) {
      raft::stats::meanvar(handle,
                           raft::make_device_matrix_view<const T, int, raft::row_major>(
                             data_d.data_handle(), c.rows, c.cols),
                           mean.view(), var.view(), c.sample);
    } else {
      raft::stats::meanvar(handle,
                           raft::make_device_matrix_view<const T, int, raft::col_major>(
                             data_d.data_handle(), c.rows, c.cols),
                           mean.view(), var.view(), c.sample);
    }
    auto mean_h = to_host(mean.data_handle(), (size_t)c.cols, stream);
    auto var_h  = to_host(var.data_handle(), (size_t)c.cols, stream);
    std::vector<double> want_m(c.cols), want_v(c.cols);
    for (int j = 0; j < c.cols; ++j) {
      double s = 0;
      for (int i = 0; i < c.rows; ++i)
        s += (double)data_h[at(c.row_major, c.rows, c.cols, i, j)];
      const double m = s / c.rows;
      double ss      = 0;
      for (int i = 0; i < c.rows; ++i) {
        const double d = (double)data_h[at(c.row_major, c.rows, c.cols, i, j)] - m;
        ss += d * d;
      }
      want_m[j] = m;
      want_v[j] = ss / std::max(1, c.sample ? c.rows - 1 : c.rows);
    }
    CHECK(all_close(mean_h, want_m, tol));
    CHECK(all_close(var_h, want_v, tol));
    if (c.rows > 1) {
      const double mean_tol = 6.0 * c.stddev / std::sqrt((double)c.rows);
      const double var_tol =
        6.0 * c.stddev * c.stddev * std::sqrt(2.0 / std::max(1, c.rows - 1));
      bool ok = true;
      for (int j = 0; j < c.cols; ++j) {
        ok &= std::fabs((double)mean_h[j] - c.mean) <= mean_tol;
        ok &= std::fabs((double)var_h[j] - c.stddev * c.stddev) <= var_tol;
      }
      CHECK(ok);
    }
    // the pointer form gives the same results
    auto mean2 = raft::make_device_vector<T, int>(handle, c.cols);
    auto var2  = raft::make_device_vector<T, int>(handle, c.cols);
    raft::stats::meanvar(mean2.data_handle(), var2.data_handle(), data_d.data_handle(), c.cols,
                         c.rows, c.sample, c.row_major, stream);
    CHECK(to_host(mean2.data_handle(), (size_t)c.cols, stream) == mean_h);
    CHECK(to_host(var2.data_handle(), (size_t)c.cols, stream) == var_h);
  }
  // size mismatch between data and var is rejected (stats/meanvar.cuh:84)
  auto data = raft::make_device_matrix<T, int, raft::row_major>(handle, 4, 5);
  auto m5   = raft::make_device_vector<T, int>(handle, 5);
  auto v4   = raft::make_device_vector<T, int>(handle, 4);
  bool threw = false;
  try {
    raft::stats::meanvar(handle,
                         raft::make_device_matrix_view<const T, int, raft::row_major>(
                           data.data_handle(), 4, 5),
                         m5.view(), v4.view(), false);
  } catch (const raft::logic_error&) {
    threw = true;
  }
  CHECK(threw);
}

// cpp/tests/stats/cov.cu:37-105: the mean through stats::mean, cov through the mdspan form (the
// grid, rows cut to keep the host reference short, plus a width that is no multiple of four), the
// 3 x 2 column-major known answer through the pointer form, the centred data left behind, and
// the refusal of stable == false.
template <typename T>
void cov_cases(double tol)
{
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  struct Case { double mean, var; int rows, cols; bool sample, row_major; };
  std::vector<Case> cases;
  for (bool rm : {false, true})
    for (int cols : {32, 64, 128, 256, 70})
      for (bool sample : {true, false})
        cases.push_back({sample ? 1.0 : -1.0, 2.0, 4096, cols, sample, rm});
  for (const auto& c : cases) {
    const size_t n = (size_t)c.rows * c.cols;
    auto data_h    = normal<T>(n, c.mean, c.var, 1234);
    auto data_d    = raft::make_device_vector<T, int>(handle, (int)n);
    raft::update_device(data_d.data_handle(), data_h.data(), n, stream);
    auto mu   = raft::make_device_vector<T, int>(handle, c.cols);
    auto cv   = raft::make_device_vector<T, int>(handle, c.cols * c.cols);
    if (c.row_major) {
      using layout = raft::row_major;
      raft::stats::mean<true>(mu.data_handle(), data_d.data_handle(), c.cols, c.rows, stream);
      raft::stats::cov(handle,
                       raft::make_device_matrix_view<T, std::uint32_t, layout>(data_d.data_handle(), c.rows, c.cols),
                       raft::make_device_vector_view<const T, std::uint32_t>(mu.data_handle(), c.cols),
                       raft::make_device_matrix_view<T, std::uint32_t, layout>(cv.data_handle(), c.cols, c.cols),
                       c.sample, true);
    } else {
      using layout = raft::col_major;
      raft::stats::mean<false>(mu.data_handle(), data_d.data_handle(), c.cols, c.rows, stream);
      raft::stats::cov(handle,
                       raft::make_device_matrix_view<T, std::uint32_t, layout>(data_d.data_handle(), c.rows, c.cols),
                       raft::make_device_vector_view<const T, std::uint32_t>(mu.data_handle(), c.cols),
                       raft::make_device_matrix_view<T, std::uint32_t, layout>(cv.data_handle(), c.cols, c.cols),
                       c.sample, true);
    }
    auto mu_h  = to_host(mu.data_handle(), (size_t)c.cols, stream);
    auto cv_h  = to_host(cv.data_handle(), (size_t)c.cols * c.cols, stream);
    auto cen_h = to_host(data_d.data_handle(), n, stream);
    // host reference: centre in T around the device's mean, contract in double
    std::vector<T> cen(n);
    for (int i = 0; i < c.rows; ++i)
      for (int j = 0; j < c.cols; ++j) {
        const size_t k = at(c.row_major, c.rows, c.cols, i, j);
        cen[k]         = (T)(data_h[k] - mu_h[j]);
      }
    CHECK(cen_h == cen);  // "this will get mean-centered at the end!"
    const double alpha = (double)(T(1) / (c.sample ? T(c.rows - 1) : T(c.rows)));
    bool ok = true, diag_ok = true;
    std::vector<double> dg(c.cols);
    for (int a = 0; a < c.cols; ++a) {
      double s = 0;
      for (int i = 0; i < c.rows; ++i) {
        const double v = (double)cen[at(c.row_major, c.rows, c.cols, i, a)];
        s += v * v;
      }
      dg[a] = s * alpha;
    }
    for (int a = 0; a < c.cols; ++a)
      for (int b = a; b < c.cols; ++b) {
        double s = 0;
        for (int i = 0; i < c.rows; ++i)
          s += (double)cen[at(c.row_major, c.rows, c.cols, i, a)] *
               (double)cen[at(c.row_major, c.rows, c.cols, i, b)];
        const double want = s * alpha;
        const double lim  = tol * std::sqrt(dg[a] * dg[b]);
        ok &= std::fabs((double)cv_h[(size_t)a * c.cols + b] - want) <= lim;
        ok &= cv_h[(size_t)a * c.cols + b] == cv_h[(size_t)b * c.cols + a];
      }
    CHECK(ok);
    // diagonalMatch(var * var, ..., CompareApprox(2 * 0.03)) with a sample of 4096 rows
    for (int a = 0; a < c.cols; ++a) {
      const double d = (double)cv_h[(size_t)a * c.cols + a], w = c.var * c.var;
      diag_ok &= std::fabs(d - w) / std::max(std::fabs(d), w) <= 0.12;
    }
    CHECK(diag_ok);
  }
  {
    T data_h[6]       = {1.0, 2.0, 5.0, 4.0, 2.0, 1.0};
    T cov_cm_ref_h[4] = {4.3333, -2.8333, -2.8333, 2.333};
    auto data_cm = raft::make_device_vector<T, int>(handle, 6);
    auto mean_cm = raft::make_device_vector<T, int>(handle, 2);
    auto cov_cm  = raft::make_device_vector<T, int>(handle, 4);
    raft::update_device(data_cm.data_handle(), data_h, 6, stream);
    raft::stats::mean<false>(mean_cm.data_handle(), data_cm.data_handle(), 2, 3, stream);
    raft::stats::cov<false>(handle, cov_cm.data_handle(), data_cm.data_handle(),
                            mean_cm.data_handle(), 2, 3, true, true, stream);
    auto got = to_host(cov_cm.data_handle(), 4, stream);
    bool ok  = true;
    for (int i = 0; i < 4; ++i) {
      const double a = (double)got[i], b = (double)cov_cm_ref_h[i];
      ok &= std::fabs(a - b) / std::max(std::fabs(a), std::fabs(b)) <= 0.06;
    }
    CHECK(ok);
    bool threw = false;
    try {
      raft::stats::cov<false>(handle, cov_cm.data_handle(), data_cm.data_handle(),
                              mean_cm.data_handle(), 2, 3, true, false, stream);
    } catch (const raft::exception&) {
      threw = true;
    }
    CHECK(threw);
    // size mismatch between data and covar (stats/cov.cuh:88-89)
    threw = false;
    try {
      raft::stats::cov(handle,
                       raft::make_device_matrix_view<T, int, raft::row_major>(data_cm.data_handle(), 3, 2),
                       raft::make_device_vector_view<const T, int>(mean_cm.data_handle(), 2),
                       raft::make_device_matrix_view<T, int, raft::row_major>(cov_cm.data_handle(), 2, 1),
                       true, true);
    } catch (const raft::logic_error&) {
      threw = true;
    }
    CHECK(threw);
  }
}

// cpp/tests/stats/mean.cu:177-185: int8 -> half
void mean_int8_to_half()
{
  raft::resources handle;
  auto stream    = raft::resource::get_cuda_stream(handle);
  const int rows = 1024, cols = 64;
  std::mt19937 g(1234);
  std::uniform_int_distribution<int> d(-20, 30);
  std::vector<std::int8_t> data_h((size_t)rows * cols);
  for (auto& x : data_h)
    x = (std::int8_t)d(g);
  auto data = raft::make_device_matrix<std::int8_t, int, raft::row_major>(handle, rows, cols);
  auto mu   = raft::make_device_vector<__half, int>(handle, cols);
  raft::update_device(data.data_handle(), data_h.data(), data_h.size(), stream);
  raft::stats::mean(handle, raft::make_const_mdspan(data.view()), mu.view());
  auto mu_h = to_host(mu.data_handle(), (size_t)cols, stream);
  bool ok   = true;
  for (int j = 0; j < cols; ++j) {
    double s = 0;
    for (int i = 0; i < rows; ++i)
      s += data_h[(size_t)i * cols + j];
    ok &= std::fabs((double)__half2float(mu_h[j]) - s / rows) <= 0.02 + 2e-3 * std::fabs(s / rows);
  }
  CHECK(ok);
}

// cpp/tests/stats/sum.cu:50-98,139-140
template <typename T>
void sum_accuracy(T value, double large, double tol)
{
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  for (int rm = 0; rm < 2; ++rm)
    for (auto [rows, cols] : std::vector<std::pair<int, int>>{{4, 5}, {1024, 32}, {1024, 256},
                                                              {17, 5}, {7, 23}, {3, 97}, {1, 30}}) {
      for (int compensate = 0; compensate < 2; ++compensate) {
        const int len = rows * cols;
        std::vector<T> data_h(len);
        for (int i = 0; i < len; i++) {
          data_h[i]     = T(double(value));
          const int row = rm ? i / cols : i % rows;
          if (compensate && row % 3 == 2) {
            data_h[i]                      = T(double(value) * large);
            data_h[rm ? (i - cols) : (i - 1)]     = T(-1 * double(value) * large);
            data_h[rm ? (i - 2 * cols) : (i - 2)] = T(3.0 * double(value));
          }
        }
        auto data_d = raft::make_device_vector<T, int>(handle, len);
        auto out    = raft::make_device_vector<T, int>(handle, cols);
        raft::update_device(data_d.data_handle(), data_h.data(), (size_t)len, stream);
        if (rm) {
          raft::stats::sum(handle,
                           raft::make_device_matrix_view<const T, int, raft::row_major>(
                             data_d.data_handle(), rows, cols),
                           out.view());
        } else {
          raft::stats::sum(handle,
                           raft::make_device_matrix_view<const T, int, raft::col_major>(
                             data_d.data_handle(), rows, cols),
                           out.view());
        }
        std::vector<double> want(cols, double(rows) * double(value));
        CHECK(all_close(to_host(out.data_handle(), (size_t)cols, stream), want, tol));
      }
    }
}

// cpp/tests/matrix/argmax.cu:71-75, argmin.cu:71-75
template <typename T>
void arg_fixtures()
{
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  std::vector<T> h{T(0.1), T(0.2), T(0.3), T(0.4), T(0.4), T(0.3),
                   T(0.2), T(0.1), T(0.2), T(0.3), T(0.5), T(0.0)};
  auto in  = raft::make_device_matrix<T, std::uint32_t, raft::row_major>(handle, 3, 4);
  auto out = raft::make_device_vector<int, std::uint32_t>(handle, 3);
  raft::update_device(in.data_handle(), h.data(), h.size(), stream);
  auto in_c = raft::make_device_matrix_view<const T, std::uint32_t, raft::row_major>(
    in.data_handle(), 3, 4);
  raft::matrix::argmax(handle, in_c, out.view());
  CHECK((to_host(out.data_handle(), 3, stream) == std::vector<int>{3, 0, 2}));
  raft::matrix::argmin(handle, in_c, out.view());
  CHECK((to_host(out.data_handle(), 3, stream) == std::vector<int>{0, 3, 3}));
  auto out64 = raft::make_device_vector<std::int64_t, std::uint32_t>(handle, 3);
  raft::matrix::argmax(handle, in_c, out64.view());
  CHECK((to_host(out64.data_handle(), 3, stream) == std::vector<std::int64_t>{3, 0, 2}));
}

// cpp/tests/linalg/map_then_reduce.cu:101-169
void map_reduce_cases()
{
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  {
    const int len = 1 << 20;
    auto h        = uniform<float>(len, -1.0, 1.0, 1234);
    auto in       = raft::make_device_vector<float, int>(handle, len);
    auto out      = raft::make_device_scalar<float>(handle);
    raft::update_device(in.data_handle(), h.data(), h.size(), stream);
    raft::linalg::mapThenSumReduce(out.data_handle(), (size_t)len, raft::identity_op(), stream,
                                   in.data_handle());
    double want = 0;
    for (float x : h)
      want += x;
    CHECK(std::fabs((double)to_host(out.data_handle(), 1, stream)[0] - want) <= 1e-3);
    raft::linalg::mapThenSumReduce(out.data_handle(), (size_t)len, raft::sq_op(), stream,
                                   in.data_handle());
    want = 0;
    for (float x : h)
      want += (double)x * x;
    CHECK(std::fabs((double)to_host(out.data_handle(), 1, stream)[0] - want) <= 1e-3 * want);
  }
  {
    const int len = 1237;
    auto h        = uniform<float>(len, 2.0, 3.0, 1234);
    h[42]         = 1.0f;
    h[337]        = 5.0f;
    auto in       = raft::make_device_vector<float, int>(handle, len);
    auto out      = raft::make_device_scalar<float>(handle);
    raft::update_device(in.data_handle(), h.data(), h.size(), stream);
    auto in_c = raft::make_device_vector_view<const float, int>(in.data_handle(), len);
    raft::linalg::map_reduce(handle, in_c, out.view(), std::numeric_limits<float>::max(),
                             raft::identity_op(), raft::min_op());
    CHECK(to_host(out.data_handle(), 1, stream)[0] == 1.0f);
    raft::linalg::map_reduce(handle, in_c, out.view(), std::numeric_limits<float>::lowest(),
                             raft::identity_op(), raft::max_op());
    CHECK(to_host(out.data_handle(), 1, stream)[0] == 5.0f);
  }
}

// a second handle on a stream of its own, reused across many calls that need the
// handle-owned workspace (split rows, column partials)
void handle_workspace_reuse()
{
  hipStream_t s;
  RAFT_HIP_TRY(hipStreamCreate(&s));
  {
    raft::device_resources handle(s);
    const int rows = 4, cols = 1 << 20;
    auto h    = uniform<float>((size_t)rows * cols, -1.0, 1.0, 99);
    auto data = raft::make_device_matrix<float, int, raft::row_major>(handle, rows, cols);
    auto out  = raft::make_device_vector<float, int>(handle, rows);
    raft::update_device(data.data_handle(), h.data(), h.size(), s);
    auto add = [](double a, double b) { return a + b; };
    auto idm = [](double x, int) { return x; };
    auto idf = [](double x) { return x; };
    auto want = host_reduce(h, rows, cols, true, true, 0.0, nullptr, idm, add, idf);
    for (int rep = 0; rep < 5; ++rep) {
      raft::linalg::reduce<raft::Apply::ALONG_ROWS>(handle, raft::make_const_mdspan(data.view()),
                                                    out.view(), 0.0f);
      CHECK(all_close(to_host(out.data_handle(), (size_t)rows, s), want, 1e-5));
    }
  }
  RAFT_HIP_TRY(hipStreamDestroy(s));
}

// Handles are copyable (the reference passes raft::resources by value in places) and copies
// share the workspace; a copy on another stream must not overwrite partials that work queued
// on the first stream still reads: results of interleaved calls on two streams stay right.
void handle_copies_and_stream_changes()
{
  hipStream_t s1, s2;
  RAFT_HIP_TRY(hipStreamCreate(&s1));
  RAFT_HIP_TRY(hipStreamCreate(&s2));
  {
    raft::resources a(s1);
    raft::resources b = a;  // shares a's workspace
    b.set_stream(s2);
    const int rows = 4, cols = 1 << 20;
    auto h1 = uniform<float>((size_t)rows * cols, -1.0, 1.0, 5);
    auto h2 = uniform<float>((size_t)rows * cols, -1.0, 1.0, 6);
    auto d1 = raft::make_device_matrix<float, int, raft::row_major>(a, rows, cols);
    auto d2 = raft::make_device_matrix<float, int, raft::row_major>(b, rows, cols);
    auto o1 = raft::make_device_vector<float, int>(a, rows);
    auto o2 = raft::make_device_vector<float, int>(b, rows);
    raft::update_device(d1.data_handle(), h1.data(), h1.size(), s1);
    raft::update_device(d2.data_handle(), h2.data(), h2.size(), s2);
    auto add = [](double x, double y) { return x + y; };
    auto idm = [](double x, int) { return x; };
    auto idf = [](double x) { return x; };
    auto w1  = host_reduce(h1, rows, cols, true, true, 0.0, nullptr, idm, add, idf);
    auto w2  = host_reduce(h2, rows, cols, true, true, 0.0, nullptr, idm, add, idf);
    for (int rep = 0; rep < 4; ++rep) {
      raft::linalg::reduce<raft::Apply::ALONG_ROWS>(a, raft::make_const_mdspan(d1.view()), o1.view(), 0.0f);
      raft::linalg::reduce<raft::Apply::ALONG_ROWS>(b, raft::make_const_mdspan(d2.view()), o2.view(), 0.0f);
    }
    CHECK(all_close(to_host(o1.data_handle(), (size_t)rows, s1), w1, 1e-5));
    CHECK(all_close(to_host(o2.data_handle(), (size_t)rows, s2), w2, 1e-5));
    auto by_value = [](raft::resources r, hipStream_t want) { return r.get_stream() == want; };
    CHECK(by_value(a, s1) && by_value(b, s2));
  }
  RAFT_HIP_TRY(hipStreamDestroy(s1));
  RAFT_HIP_TRY(hipStreamDestroy(s2));
}

// After a warm-up call a handle neither allocates nor makes the host wait: the column mean and
// stddev (two-pass column plan), a split-row reduction (ticket counters in the handle's
// workspace) and meanvar are recorded through one handle into a HIP graph; the graph is
// replayed over new contents of the same buffers, with eager work in between, and every replay
// is held to the host reference.
void handle_calls_under_graph_capture()
{
  hipStream_t s;
  RAFT_HIP_TRY(hipStreamCreate(&s));
  {
    raft::resources handle(s);
    const int rows = 20000, cols = 64;        // column plans
    const int lrows = 4, lcols = 1 << 20;      // rows split over several workgroups
    auto data  = raft::make_device_matrix<float, int, raft::row_major>(handle, rows, cols);
    auto mu    = raft::make_device_vector<float, int>(handle, cols);
    auto sd    = raft::make_device_vector<float, int>(handle, cols);
    auto mv_m  = raft::make_device_vector<float, int>(handle, cols);
    auto mv_v  = raft::make_device_vector<float, int>(handle, cols);
    auto ldata = raft::make_device_matrix<float, int, raft::row_major>(handle, lrows, lcols);
    auto lout  = raft::make_device_vector<float, int>(handle, lrows);
    auto run   = [&] {
      auto dv = raft::make_const_mdspan(data.view());
      raft::stats::mean(handle, dv, mu.view());
      raft::stats::stddev(handle, dv, raft::make_const_mdspan(mu.view()), sd.view(), true);
      raft::stats::meanvar(handle, dv, mv_m.view(), mv_v.view(), true);
      raft::linalg::reduce<raft::Apply::ALONG_ROWS>(handle, raft::make_const_mdspan(ldata.view()),
                                                    lout.view(), 0.0f);
    };
    auto fill = [&](unsigned long long seed, std::vector<float>& h, std::vector<float>& lh) {
      h  = normal<float>((size_t)rows * cols, 3.0, 2.0, seed);
      lh = uniform<float>((size_t)lrows * lcols, -1.0, 1.0, seed + 1);
      raft::update_device(data.data_handle(), h.data(), h.size(), s);
      raft::update_device(ldata.data_handle(), lh.data(), lh.size(), s);
      RAFT_HIP_TRY(hipStreamSynchronize(s));
    };
    auto check = [&](const std::vector<float>& h, const std::vector<float>& lh) {
      auto add = [](double a, double b) { return a + b; };
      auto idm = [](double x, int) { return x; };
      auto idf = [](double x) { return x; };
      std::vector<double> wm(cols), ws(cols), wv(cols);
      for (int j = 0; j < cols; ++j) {
        double a = 0, q = 0;
        for (int i = 0; i < rows; ++i)
          a += h[(size_t)i * cols + j];
        a /= rows;
        for (int i = 0; i < rows; ++i) {
          const double d = h[(size_t)i * cols + j] - a;
          q += d * d;
        }
        wm[j] = a, wv[j] = q / (rows - 1), ws[j] = std::sqrt(wv[j]);
      }
      CHECK(all_close(to_host(mu.data_handle(), (size_t)cols, s), wm, 1e-5));
      CHECK(all_close(to_host(sd.data_handle(), (size_t)cols, s), ws, 1e-4));
      CHECK(all_close(to_host(mv_m.data_handle(), (size_t)cols, s), wm, 1e-5));
      CHECK(all_close(to_host(mv_v.data_handle(), (size_t)cols, s), wv, 1e-5));
      CHECK(all_close(to_host(lout.data_handle(), (size_t)lrows, s),
                      host_reduce(lh, lrows, lcols, true, true, 0.0, nullptr, idm, add, idf), 1e-5));
    };
    std::vector<float> h, lh;
    fill(1, h, lh);
    run();  // warm-up: the workspace reaches its size, the ticket words are cleared
    check(h, lh);

    // the recorded calls must find the workspace as the warm-up left it: same buffer, no growth
    void* const ws_before = handle.workspace(1);
    size_t free_before = 0, free_after = 0, total = 0;
    RAFT_HIP_TRY(hipMemGetInfo(&free_before, &total));
    hipGraph_t graph;
    hipGraphExec_t exec;
    RAFT_HIP_TRY(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal));
    run();
    RAFT_HIP_TRY(hipStreamEndCapture(s, &graph));
    RAFT_HIP_TRY(hipMemGetInfo(&free_after, &total));
    CHECK(handle.workspace(1) == ws_before);
    CHECK(free_after == free_before);  // nothing was allocated while recording
    RAFT_HIP_TRY(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
    for (unsigned long long rep = 0; rep < 3; ++rep) {
      fill(100 + 7 * rep, h, lh);
      RAFT_HIP_TRY(hipGraphLaunch(exec, s));
      check(h, lh);
      run();  // eager work between the replays, through the same workspace
      check(h, lh);
    }
    RAFT_HIP_TRY(hipGraphExecDestroy(exec));
    RAFT_HIP_TRY(hipGraphDestroy(graph));
  }
  RAFT_HIP_TRY(hipStreamDestroy(s));
}

// A change of the handle's stream costs no host wait: with several milliseconds of reductions
// queued on the first stream, the first call on the second returns at once, and its
// result is right although both calls share the workspace.
void handle_stream_change_does_not_block()
{
  hipStream_t s1, s2;
  RAFT_HIP_TRY(hipStreamCreate(&s1));
  RAFT_HIP_TRY(hipStreamCreate(&s2));
  {
    raft::resources handle(s1);
    const int rows = 4, cols = 16 << 20;  // 256 MB, rows split over workgroups
    auto big  = raft::make_device_matrix<float, int, raft::row_major>(handle, rows, cols);
    auto bout = raft::make_device_vector<float, int>(handle, rows);
    auto h    = uniform<float>((size_t)rows * (1 << 20), -1.0, 1.0, 21);
    auto small = raft::make_device_matrix<float, int, raft::row_major>(handle, rows, 1 << 20);
    auto sout  = raft::make_device_vector<float, int>(handle, rows);
    RAFT_HIP_TRY(hipMemsetAsync(big.data_handle(), 0, sizeof(float) * (size_t)rows * cols, s1));
    raft::update_device(small.data_handle(), h.data(), h.size(), s1);
    auto call_big = [&] {
      raft::linalg::reduce<raft::Apply::ALONG_ROWS>(handle, raft::make_const_mdspan(big.view()),
                                                    bout.view(), 0.0f);
    };
    call_big();  // warm-up
    RAFT_HIP_TRY(hipDeviceSynchronize());
    auto now = [] { return std::chrono::steady_clock::now(); };
    const auto t0 = now();
    for (int i = 0; i < 200; ++i)
      call_big();  // 200 x 256 MB: about 8 ms of device work on s1
    const auto t1 = now();
    raft::resource::set_cuda_stream(handle, s2);
    raft::linalg::reduce<raft::Apply::ALONG_ROWS>(handle, raft::make_const_mdspan(small.view()),
                                                  sout.view(), 0.0f);
    const auto t2 = now();
    const bool s1_busy = hipStreamQuery(s1) == hipErrorNotReady;
    RAFT_HIP_TRY(hipStreamSynchronize(s1));
    const auto t3 = now();
    const double enqueue_ms = std::chrono::duration<double, std::milli>(t1 - t0).count();
    const double switch_ms  = std::chrono::duration<double, std::milli>(t2 - t1).count();
    const double drain_ms   = std::chrono::duration<double, std::milli>(t3 - t2).count();
    std::printf("  200 calls enqueued in %.2f ms, call after the stream change %.3f ms, "
                "first stream drained %.2f ms later\n", enqueue_ms, switch_ms, drain_ms);
    CHECK(s1_busy);            // the first stream still had work when the second call returned
    CHECK(switch_ms < 1.0);    // ... so the call did not wait for it on the host
    auto add = [](double a, double b) { return a + b; };
    auto idm = [](double x, int) { return x; };
    auto idf = [](double x) { return x; };
    CHECK(all_close(to_host(sout.data_handle(), (size_t)rows, s2),
                    host_reduce(h, rows, 1 << 20, true, true, 0.0, nullptr, idm, add, idf), 1e-5));
    CHECK(all_close(to_host(bout.data_handle(), (size_t)rows, s1),
                    std::vector<double>(rows, 0.0), 1e-6));
  }
  RAFT_HIP_TRY(hipStreamDestroy(s1));
  RAFT_HIP_TRY(hipStreamDestroy(s2));
}

// cpp/tests/linalg/normalize.cu:40-135: row_normalize against rowNorm followed by a
// per-row division, rows {11,101,12345} x cols {2,3,7,12,33,125,254} x {L1,L2,Linf}
template <typename T, typename Idx>
void row_normalize_cases(double tol)
{
  using namespace raft::linalg;
  raft::resources handle;
  auto stream = raft::resource::get_cuda_stream(handle);
  for (int rows : {11, 101, 12345})
    for (int cols : {2, 3, 7, 12, 33, 125, 254}) {
      auto h   = uniform<T>((size_t)rows * cols, -10.0, 10.0, 1234);
      auto in  = raft::make_device_matrix<T, Idx, raft::row_major>(handle, (Idx)rows, (Idx)cols);
      auto out = raft::make_device_matrix<T, Idx, raft::row_major>(handle, (Idx)rows, (Idx)cols);
      raft::update_device(in.data_handle(), h.data(), h.size(), stream);
      auto in_v = raft::make_device_matrix_view<const T, Idx, raft::row_major>(in.data_handle(),
                                                                               (Idx)rows, (Idx)cols);
      for (int nt = 0; nt < 3; ++nt) {
        if (nt == 0) row_normalize<L1Norm>(handle, in_v, out.view());
        if (nt == 1) row_normalize<L2Norm>(handle, in_v, out.view());
        if (nt == 2) row_normalize<LinfNorm>(handle, in_v, out.view());
        auto got = to_host(out.data_handle(), h.size(), stream);
        std::vector<double> want(h.size());
        for (int i = 0; i < rows; ++i) {
          double n = 0;
          for (int j = 0; j < cols; ++j) {
            const double x = (double)h[(size_t)i * cols + j];
            n = nt == 0 ? n + std::fabs(x) : nt == 1 ? n + x * x : std::max(n, std::fabs(x));
          }
          if (nt == 1) n = std::sqrt(n);
          for (int j = 0; j < cols; ++j)
            want[(size_t)i * cols + j] = (double)h[(size_t)i * cols + j] / n;
        }
        CHECK(all_close(got, want, tol));
      }
    }
}

}  // namespace

TEST_CASE(RowNormalizeFI32) { row_normalize_cases<float, int>(1e-5); }
TEST_CASE(RowNormalizeDI32) { row_normalize_cases<double, int>(1e-8); }
TEST_CASE(RowNormalizeFU32) { row_normalize_cases<float, std::uint32_t>(1e-5); }
TEST_CASE(ReduceSimpleF) { simple_max<float>(); }
TEST_CASE(ReduceSimpleD) { simple_max<double>(); }
TEST_CASE(ReduceTestFFI32) { reduce_full<float, float, int>(2e-6, {11, 1234}, {7, 33, 128, 500}); }
TEST_CASE(ReduceTestFFU32) { reduce_full<float, float, std::uint32_t>(2e-6, {11, 1234}, {7, 33, 128, 500}); }
TEST_CASE(ReduceTestFFI64) { reduce_full<float, float, std::int64_t>(2e-6, {11, 1234}, {7, 33, 128, 500}); }
TEST_CASE(ReduceTestFFU64) { reduce_full<float, float, std::uint64_t>(2e-6, {11, 1234}, {7, 33, 128, 500}); }
TEST_CASE(ReduceTestDDI32) { reduce_full<double, double, int>(1e-9, {11, 1234}, {7, 33, 128, 500}); }
TEST_CASE(ReduceTestFDI32) { reduce_full<float, double, int>(1e-9, {11, 1234}, {7, 33, 128, 500}); }
TEST_CASE(ReduceTestFFThick) { reduce_full<float, float, int>(1e-4, {3, 9}, {17771, 33333, 100000}); }
TEST_CASE(ReduceTestKVPIF) { reduce_kvp<float>(); }
TEST_CASE(ReduceTestKVPID) { reduce_kvp<double>(); }
TEST_CASE(CoalescedStridedF) { coalesced_and_strided<float>(2e-6); }
TEST_CASE(CoalescedStridedD) { coalesced_and_strided<double>(1e-9); }
TEST_CASE(NormF) { norms<float, float>(1e-5); }
TEST_CASE(NormD) { norms<double, double>(1e-9); }
TEST_CASE(MeanStddevF) { mean_stddev<float>(1e-5); }
TEST_CASE(MeanStddevD) { mean_stddev<double>(1e-9); }
TEST_CASE(MeanVarF) { meanvar_cases<float>(1e-5); }
TEST_CASE(MeanVarD) { meanvar_cases<double>(1e-9); }
TEST_CASE(CovF) { cov_cases<float>(1e-5); }
TEST_CASE(CovD) { cov_cases<double>(1e-12); }
TEST_CASE(MeanInt8ToHalf) { mean_int8_to_half(); }
TEST_CASE(SumAccuracyF) { sum_accuracy<float>(0.0001f, 1e7, 0.001); }
TEST_CASE(SumAccuracyD) { sum_accuracy<double>(0.000001, 1e12, 0.0001); }
TEST_CASE(ArgFixturesF) { arg_fixtures<float>(); }
TEST_CASE(ArgFixturesD) { arg_fixtures<double>(); }
TEST_CASE(MapReduce) { map_reduce_cases(); }
TEST_CASE(HandleWorkspaceReuse) { handle_workspace_reuse(); }
TEST_CASE(HandleCopiesAndStreamChanges) { handle_copies_and_stream_changes(); }
TEST_CASE(HandleCallsUnderGraphCapture) { handle_calls_under_graph_capture(); }
TEST_CASE(HandleStreamChangeDoesNotBlock) { handle_stream_change_does_not_block(); }

int main()
{
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess || n == 0) {
    std::printf("no GPU visible\n");
    return 2;
  }
  return t::run_all();
}
