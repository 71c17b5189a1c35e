// Host-only tests of the C++ API layer (no GPU needed): the functor vocabulary,
// views, precondition errors and the plan selector.  Restates
// cpp/tests/core/operators_host.cpp of the reference for the functors on the path.
#include <raft/core/device_mdspan.hpp>
#include <raft/core/operators.hpp>
#include <raft/linalg/norm.cuh>
#include <raft/linalg/reduce.cuh>
#include <raft/matrix/argmax.cuh>
#include <raft/stats/mean.cuh>
#include <raft/stats/stddev.cuh>
#include <raft/stats/sum.cuh>
#include <raft/util/itertools.hpp>

#include "check.hpp"

using kvp = raft::KeyValuePair<int, float>;

// cpp/tests/core/operators_host.cpp:134-172
TEST_CASE(arg_ops_truth_table)
{
  kvp a(0, 1.2f), b(0, 3.4f), c(1, 1.2f);
  raft::argmin_op mn;
  CHECK(mn(a, b) == a);
  CHECK(mn(b, a) == a);
  CHECK(mn(a, c) == a);
  CHECK(mn(c, a) == a);
  CHECK(mn(b, c) == c);
  CHECK(mn(c, b) == c);
  raft::argmax_op mx;
  CHECK(mx(a, b) == b);
  CHECK(mx(b, a) == b);
  CHECK(mx(a, c) == a);
  CHECK(mx(c, a) == a);
  CHECK(mx(b, c) == b);
  CHECK(mx(c, b) == b);
}

// cpp/tests/core/operators_host.cpp: the remaining functors used on the path
TEST_CASE(functor_values)
{
  CHECK(raft::identity_op{}(12.34f) == 12.34f);
  CHECK(raft::identity_op{}(12.34f, 0, 80, 6) == 12.34f);
  CHECK(raft::cast_op<int>{}(12.34f) == 12);
  CHECK(raft::key_op{}(kvp(12, 3.4f)) == 12);
  CHECK(raft::value_op{}(kvp(12, 3.4f)) == 3.4f);
  CHECK(std::abs(raft::sqrt_op{}(12.34f) - std::sqrt(12.34f)) < 1e-6f);
  CHECK(raft::nz_op{}(0.0f) == 0.0f && raft::nz_op{}(12.34f) == 1.0f);
  CHECK(raft::abs_op{}(-12.34f) == 12.34f && raft::abs_op{}(-7) == 7);
  CHECK(raft::sq_op{}(-3) == 9);
  CHECK(raft::add_op{}(12.0f, 13.0f) == 25.0f);
  CHECK(raft::mul_op{}(3, 4) == 12);
  CHECK(raft::min_op{}(3.0f, 5.0f) == 3.0f && raft::max_op{}(3.0f, 5.0f) == 5.0f);
  CHECK(raft::max_op{}(std::nanf(""), 5.0f) == 5.0f);  // NaN is ignored
  CHECK(raft::const_op<float>(12.34f)(13, 37.0f) == 12.34f);
  CHECK(raft::mul_const_op<float>(2.0f)(2.5f) == 5.0f);
  CHECK(raft::div_const_op<float>(2.0f)(5.0f) == 2.5f);
  CHECK(raft::add_const_op<int>(8)(-50) == -42);
  CHECK(raft::sqdiff_op{}(3.0f, 5.0f) == 4.0f);
  CHECK(raft::absdiff_op{}(3.0f, 5.0f) == 2.0f);
  auto comp = raft::compose_op(raft::sqrt_op(), raft::abs_op(), raft::cast_op<float>(),
                               raft::add_const_op<int>(8));
  CHECK(std::abs(comp(-50) - 6.480741f) < 1e-5f);
  raft::map_args_op<raft::add_op, raft::sqrt_op, raft::cast_op<float>> m;
  CHECK(std::abs(m(42.0f, 10) - 16.480741f) < 1e-5f);
  auto p = raft::value_to_kvp_op<int>{}(2.5f, 7);
  CHECK(p.key == 7 && p.value == 2.5f);
  static_assert(sizeof(raft::KeyValuePair<int, float>) == 8);
  static_assert(sizeof(raft::KeyValuePair<int, double>) == 16);
  static_assert(sizeof(raft::KeyValuePair<std::int64_t, float>) == 16);
}

TEST_CASE(views_and_layout_predicates)
{
  float* p = reinterpret_cast<float*>(0x1000);
  auto m   = raft::make_device_matrix_view<float, int>(p, 3, 4);
  CHECK(m.extent(0) == 3 && m.extent(1) == 4 && m.size() == 12u);
  CHECK(m.stride(0) == 4 && m.stride(1) == 1 && m.is_exhaustive());
  CHECK(raft::is_row_major(m) && !raft::is_col_major(m) && raft::is_row_or_column_major(m));
  auto c = raft::make_device_matrix_view<float, int, raft::col_major>(p, 3, 4);
  CHECK(c.stride(0) == 1 && c.stride(1) == 3 && raft::is_col_major(c));
  auto cm = raft::make_const_mdspan(m);
  static_assert(std::is_same_v<decltype(cm)::element_type, const float>);
  CHECK(cm.data_handle() == p);
  auto s = raft::make_device_strided_matrix_view<float, int, raft::row_major>(p, 3, 4, 6);
  CHECK(raft::is_row_major(s) && !s.is_exhaustive());
  auto s2 = raft::make_device_strided_matrix_view<float, int, raft::row_major>(p, 3, 4, 0);
  CHECK(s2.is_exhaustive());
  auto v = raft::make_device_vector_view<float, int>(p, 5);
  CHECK(v.size() == 5u && v.extent(0) == 5);
  auto sc = raft::make_device_scalar_view<float>(p);
  CHECK(sc.size() == 1u);
}

// RAFT_EXPECTS failures: linalg/reduce.cuh:157-168, stats/mean.cuh:93-95,
// stats/stddev.cuh:112-113, matrix/argmax.cuh:32-33 in the reference.  The checks run
// before anything touches the device, so the pointers are never dereferenced.
TEST_CASE(shape_errors_throw_logic_error)
{
  raft::resources h;
  float* p  = reinterpret_cast<float*>(0x1000);
  int* ip   = reinterpret_cast<int*>(0x2000);
  auto data = raft::make_device_matrix_view<const float, int>(p, 3, 4);
  auto out3 = raft::make_device_vector_view<float, int>(p, 3);
  auto out4 = raft::make_device_vector_view<float, int>(p, 4);
  CHECK_THROWS_AS(raft::linalg::reduce<raft::Apply::ALONG_ROWS>(h, data, out4, 0.0f),
                  raft::logic_error);
  CHECK_THROWS_AS(raft::linalg::reduce<raft::Apply::ALONG_COLUMNS>(h, data, out3, 0.0f),
                  raft::logic_error);
  auto strided = raft::make_device_strided_matrix_view<const float, int, raft::row_major>(p, 3, 4, 6);
  CHECK_THROWS_AS(raft::linalg::reduce<raft::Apply::ALONG_ROWS>(h, strided, out3, 0.0f),
                  raft::logic_error);
  CHECK_THROWS_AS((raft::linalg::norm<raft::linalg::L2Norm, raft::Apply::ALONG_ROWS>(
                    h, data, out4, raft::sqrt_op())),
                  raft::logic_error);
  CHECK_THROWS_AS(raft::stats::mean(h, data, out3), raft::logic_error);
  CHECK_THROWS_AS(raft::stats::sum(h, data, out3), raft::logic_error);
  auto mu3 = raft::make_device_vector_view<const float, int>(p, 3);
  auto mu4 = raft::make_device_vector_view<const float, int>(p, 4);
  CHECK_THROWS_AS(raft::stats::stddev(h, data, mu3, out3, false), raft::logic_error);
  CHECK_THROWS_AS(raft::stats::stddev(h, data, mu4, out3, false), raft::logic_error);
  CHECK_THROWS_AS(raft::stats::vars(h, data, mu3, out4, true), raft::logic_error);
  auto idx4 = raft::make_device_vector_view<int, int>(ip, 4);
  CHECK_THROWS_AS(raft::matrix::argmax(h, data, idx4), raft::logic_error);
  try {
    raft::linalg::reduce<raft::Apply::ALONG_ROWS>(h, data, out4, 0.0f);
  } catch (const raft::logic_error& e) {
    const std::string w = e.what();
    CHECK(w.rfind("RAFT failure at ", 0) == 0);
    CHECK(w.find("Output should be equal to number of rows in Input") != std::string::npos);
  }
}

TEST_CASE(plan_selector)
{
  auto plan = [](int in_dt, int out_dt, long rows, long cols, int apply = RMI_ALONG_ROWS,
                 int red = RMI_RED_ADD, int main = RMI_MAIN_IDENTITY) {
    rmi_reduce_desc d{};
    d.in_dtype = in_dt, d.out_dtype = out_dt, d.n_rows = rows, d.n_cols = cols;
    d.apply = apply, d.reduce_op = red, d.main_op = main;
    rmi_plan p{};
    CHECK(rmi_plan_query(&d, &p) == RMI_OK);
    return p;
  };
  auto p = plan(RMI_F32, RMI_F32, 1000000, 128);
  CHECK(p.kind == RMI_PLAN_ROW_WAVE && p.lanes_per_row == 8 && p.vec_bytes == 16);
  p = plan(RMI_I8, RMI_I64, 16777216, 8);
  CHECK(p.kind == RMI_PLAN_ROW_LANES);
  p = plan(RMI_I8, RMI_I64, 16777216, 4);
  CHECK(p.kind == RMI_PLAN_ROW_WAVE && p.lanes_per_row == 1);  // four rows per vector: through LDS, a thread per row
  p = plan(RMI_BF16, RMI_BF16, 16777216, 2);
  CHECK(p.kind == RMI_PLAN_ROW_LANES);  // outputs narrower than 32 bits are packed by a lane
  p = plan(RMI_I8, RMI_I64, 4096, 16384);
  CHECK(p.kind == RMI_PLAN_ROW_BLOCK && p.passes == 1);
  p = plan(RMI_BF16, RMI_F32, 8, 4194304);
  CHECK(p.kind == RMI_PLAN_ROW_SPLIT && p.passes == 2 && p.workspace_bytes > RMI_WORKSPACE_TICKET_BYTES);
  p = plan(RMI_F32, RMI_F32, 10000000, 64, RMI_ALONG_COLUMNS);
  CHECK(p.kind == RMI_PLAN_COL_TILE && p.n_outputs == 64 && p.reduce_len == 10000000);
  p = plan(RMI_F32, RMI_KVP_I32_F32, 65536, 32000, RMI_ALONG_ROWS, RMI_RED_ARGMAX, RMI_MAIN_KVP);
  CHECK(p.kind == RMI_PLAN_ROW_BLOCK && p.block_threads == 256 && p.passes == 1);
  p = plan(RMI_F32, RMI_F32, 100, 7);
  CHECK(p.vec_bytes == 16);  // 28-byte rows: one 16-byte lane load and three tail elements
  p = plan(RMI_F32, RMI_F32, 100, 3);
  CHECK(p.vec_bytes == 16 && p.lanes_per_row == 1);  // 12-byte rows go through LDS as whole vectors
  p = plan(RMI_F32, RMI_F32, 5, 0);
  CHECK(p.kind == RMI_PLAN_EMPTY);
  rmi_reduce_desc bad{};
  bad.in_dtype = 99;
  rmi_plan q{};
  CHECK(rmi_plan_query(&bad, &q) == RMI_ERR_BAD_ENUM);
  bad          = rmi_reduce_desc{};
  bad.in_dtype = RMI_F32, bad.out_dtype = RMI_I32;
  CHECK(rmi_plan_query(&bad, &q) == RMI_ERR_UNSUPPORTED);
  bad.out_dtype = RMI_F32, bad.n_rows = -1;
  CHECK(rmi_plan_query(&bad, &q) == RMI_ERR_BAD_SHAPE);
  CHECK(rmi_plan_query(nullptr, &q) == RMI_ERR_NULL);
  CHECK(std::string(rmi_status_string(RMI_ERR_WORKSPACE)).size() > 0);
  CHECK(rmi_abi_version() == RMI_ABI_VERSION);
}

TEST_CASE(itertools_product)
{
  struct P {
    int a;
    float b;
    bool c;
  };
  auto v = raft::util::itertools::product<P>({1, 2}, {0.5f}, {true, false});
  CHECK(v.size() == 4u);
  CHECK(v[0].a == 1 && v[0].c == true && v[1].c == false && v[3].a == 2);
}

int main() { return t::run_all(); }
