// Benchmarks of the reduction primitives over the shape grids of the reference's own
// benchmark programs, timed the way its fixture times them: before every timed call a
// scratch buffer is overwritten to evict the caches, then one call is bracketed by two
// events on the stream (cpp/bench/prims/common/benchmark.hpp:59-158).  Grids:
//   reduce            cpp/bench/prims/linalg/reduce.cu:44-55
//   rowNorm           cpp/bench/prims/linalg/norm.cu:57-69
//   rowNormalize      cpp/bench/prims/linalg/normalize.cu:57-69
//   map_then_reduce   cpp/bench/prims/linalg/map_then_reduce.cu:41-56
//   Argmin            cpp/bench/prims/matrix/argmin.cu:55-60
// One line per case: name, shape, mean time per call, algorithmic GB/s.
//
// copy_roof (no counterpart in the reference) measures what this GPU sustains when a kernel
// writes as many bytes as it reads: a plain streaming copy swept over loads in flight per
// lane, workgroups per CU (one-shot grid or persistent), and non-temporal loads / stores, at
// 134 MB + 134 MB and 512 MB + 512 MB, over rotating buffers.  It is the roof that the
// shapes with 1:1 traffic (row_normalize, row sums of 8-byte rows into int64) are held to.
// read_roof is the same for kernels that only read (16-byte loads XORed into a register), at the
// input sizes of the benchmark shapes from 10 MiB to 2.4 GiB.  call_path times back-to-back calls of
// the smallest benchmark shape from a native loop (C ABI, header API, HIP graph replay).
//
// usage: prims_bench [--filter substring] [--min-iters N] [--max-bytes B] [--no-flush]
#include <raft/core/device_mdarray.hpp>
#include <raft/core/device_mdspan.hpp>
#include <raft/core/resources.hpp>
#include <raft/linalg/map_then_reduce.cuh>
#include <raft/linalg/matrix_vector_op.cuh>
#include <raft/linalg/norm.cuh>
#include <raft/linalg/normalize.cuh>
#include <raft/linalg/reduce.cuh>
#include <raft/matrix/argmin.cuh>
#include <raft/util/cudart_utils.hpp>

#include <rmi_reduce.h>

#include <algorithm>
#include <chrono>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

namespace {

// uniform values in [lo, hi) from a counter hash: cheap, reproducible, no state
template <typename T>
__global__ void fill_uniform(T* p, size_t n, double lo, double hi, unsigned long long seed)
{
  size_t i            = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    unsigned long long z = (i + seed) * 0x9E3779B97F4A7C15ull;
    z ^= z >> 30;
    z *= 0xBF58476D1CE4E5B9ull;
    z ^= z >> 27;
    z *= 0x94D049BB133111EBull;
    z ^= z >> 31;
    const double u = (double)(z >> 11) * (1.0 / 9007199254740992.0);
    p[i]           = (T)(lo + (hi - lo) * u);
  }
}

__global__ void fill_words(unsigned* p, size_t n, unsigned v)
{
  size_t i            = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride)
    p[i] = v;
}

struct Options {
  std::string filter;
  int min_iters    = 10;
  size_t max_bytes = (size_t)96 << 30;
  bool flush       = true;
};

template <typename T>
struct Identity {  // the reference benchmark's own functor: takes the header-template path
  __host__ __device__ T operator()(T a) const { return a; }
};

class Harness {
 public:
  explicit Harness(const Options& o) : opt_(o)
  {
    stream_ = raft::resource::get_cuda_stream(handle_);
    // three times the last-level cache, as the reference flushes three times its L2; the
    // 256 MB memory-side cache of this GPU is the level that matters here
    int l2 = 0;
    RAFT_HIP_TRY(hipDeviceGetAttribute(&l2, hipDeviceAttributeL2CacheSize, 0));
    flush_bytes_ = 3 * std::max<size_t>((size_t)l2, (size_t)256 << 20);
    RAFT_HIP_TRY(hipMalloc(&flush_buf_, flush_bytes_));
    RAFT_HIP_TRY(hipEventCreate(&e0_));
    RAFT_HIP_TRY(hipEventCreate(&e1_));
  }
  ~Harness()
  {
    (void)hipFree(flush_buf_);
    (void)hipEventDestroy(e0_);
    (void)hipEventDestroy(e1_);
  }
  raft::resources& handle() { return handle_; }
  hipStream_t stream() const { return stream_; }
  bool wanted(const std::string& name) const
  {
    return opt_.filter.empty() || name.find(opt_.filter) != std::string::npos;
  }
  bool fits(size_t bytes) const { return bytes <= opt_.max_bytes; }

  template <typename F>
  void run(const std::string& name, const std::string& shape, size_t alg_bytes, F&& call)
  {
    call();  // warm-up: code objects, workspace
    RAFT_HIP_TRY(hipStreamSynchronize(stream_));
    double total_ms = 0.0;
    int iters       = 0;
    // at least min_iters calls and 20 ms of kernel time, at most 200 calls
    while (iters < opt_.min_iters || (total_ms < 20.0 && iters < 200)) {
      if (opt_.flush)
        fill_words<<<2048, 256, 0, stream_>>>(static_cast<unsigned*>(flush_buf_),
                                              flush_bytes_ / 4, (unsigned)iters);
      RAFT_HIP_TRY(hipEventRecord(e0_, stream_));
      call();
      RAFT_HIP_TRY(hipEventRecord(e1_, stream_));
      RAFT_HIP_TRY(hipEventSynchronize(e1_));
      float ms = 0.f;
      RAFT_HIP_TRY(hipEventElapsedTime(&ms, e0_, e1_));
      total_ms += ms;
      ++iters;
    }
    const double us = total_ms * 1e3 / iters;
    std::printf("%-34s %-22s %10.2f us %9.1f GB/s  iters=%d\n", name.c_str(), shape.c_str(), us,
                (double)alg_bytes / (us * 1e-6) / 1e9, iters);
    std::fflush(stdout);
  }

 private:
  Options opt_;
  raft::resources handle_;
  hipStream_t stream_ = nullptr;
  void* flush_buf_    = nullptr;
  size_t flush_bytes_ = 0;
  hipEvent_t e0_{}, e1_{};
};

template <typename T>
struct DeviceBuf {
  T* p     = nullptr;
  size_t n = 0;
  explicit DeviceBuf(size_t count) : n(count) { RAFT_HIP_TRY(hipMalloc(&p, std::max<size_t>(n, 1) * sizeof(T))); }
  ~DeviceBuf() { (void)hipFree(p); }
  DeviceBuf(const DeviceBuf&)            = delete;
  DeviceBuf& operator=(const DeviceBuf&) = delete;
  void uniform(double lo, double hi, hipStream_t s)
  {
    if (n) fill_uniform<<<4096, 256, 0, s>>>(p, n, lo, hi, 1234ull);
  }
};

template <typename T>
const char* tname()
{
  return sizeof(T) == 4 ? "float" : "double";
}

std::string shape2(long long r, long long c) { return std::to_string(r) + "x" + std::to_string(c); }

template <typename T>
void bench_reduce(Harness& h)
{
  const std::vector<std::pair<int, int>> sizes{{8 * 1024, 1024},  {1024, 8 * 1024},
                                               {8 * 1024, 8 * 1024}, {32 * 1024, 1024},
                                               {1024, 32 * 1024},  {32 * 1024, 32 * 1024}};
  for (bool along_rows : {false, true})
    for (auto size : sizes) {
      const int rows = size.first, cols = size.second;
      const std::string name =
        std::string("reduce<") + tname<T>() + ">/" + (along_rows ? "along_rows" : "along_cols");
      const size_t n = (size_t)rows * cols;
      if (!h.wanted(name) || !h.fits(n * sizeof(T))) continue;
      DeviceBuf<T> in(n), out((size_t)std::max(rows, cols));
      in.uniform(-1.0, 1.0, h.stream());
      h.run(name, shape2(rows, cols), n * sizeof(T), [&] {
        if (along_rows)
          raft::linalg::reduce<true, true>(out.p, in.p, cols, rows, T(0), h.stream());
        else
          raft::linalg::reduce<true, false>(out.p, in.p, cols, rows, T(0), h.stream());
      });
    }
}

template <typename T, typename IdxT>
void bench_row_norm(Harness& h)
{
  const std::string name = std::string("rowNorm<") + tname<T>() + "," +
                           (sizeof(IdxT) == 4 ? "int" : "int64_t") + ">";
  if (!h.wanted(name)) return;
  for (IdxT rows : {10, 100, 1000, 10000, 100000})
    for (IdxT cols : {16, 32, 64, 128, 256, 512, 1024}) {
      const size_t n = (size_t)rows * cols;
      DeviceBuf<T> in(n), dots((size_t)rows);
      in.uniform(-10.0, 10.0, h.stream());
      h.run(name, shape2(rows, cols), n * sizeof(T), [&] {
        auto iv = raft::make_device_matrix_view<const T, IdxT, raft::row_major>(in.p, rows, cols);
        auto ov = raft::make_device_vector_view<T, IdxT>(dots.p, rows);
        raft::linalg::norm<raft::linalg::L2Norm, raft::Apply::ALONG_ROWS>(h.handle(), iv, ov,
                                                                          raft::sqrt_op());
      });
    }
}

template <typename T, typename IdxT>
void bench_row_normalize(Harness& h)
{
  const std::string name = std::string("rowNormalize<") + tname<T>() + "," +
                           (sizeof(IdxT) == 4 ? "int" : "int64_t") + ">";
  if (!h.wanted(name)) return;
  for (IdxT rows : {10, 100, 1000, 10000, 100000})
    for (IdxT cols : {8, 16, 32, 64, 128, 256, 512, 1024, 2048, 4096, 8192, 16384}) {
      const size_t n = (size_t)rows * cols;
      DeviceBuf<T> in(n), out(n);
      in.uniform(-10.0, 10.0, h.stream());
      h.run(name, shape2(rows, cols), 2 * n * sizeof(T), [&] {
        auto iv = raft::make_device_matrix_view<const T, IdxT, raft::row_major>(in.p, rows, cols);
        auto ov = raft::make_device_matrix_view<T, IdxT, raft::row_major>(out.p, rows, cols);
        raft::linalg::row_normalize<raft::linalg::L2Norm>(h.handle(), iv, ov);
      });
    }
}

template <typename T>
void bench_map_then_reduce(Harness& h)
{
  const std::vector<int> lens{1024 * 1024,     32 * 1024 * 1024,     1024 * 1024 * 1024,
                              1024 * 1024 + 2, 32 * 1024 * 1024 + 2, 1024 * 1024 * 1024 + 2,
                              1024 * 1024 + 1, 32 * 1024 * 1024 + 1, 1024 * 1024 * 1024 + 1};
  for (int len : lens) {
    const size_t n = (size_t)len;
    if (!h.fits(n * sizeof(T))) continue;
    const std::string user = std::string("map_then_reduce<") + tname<T>() + ">/user_functor";
    const std::string lib  = std::string("map_then_reduce<") + tname<T>() + ">/identity_op";
    if (!h.wanted(user) && !h.wanted(lib)) continue;
    DeviceBuf<T> in(n), out(1);
    in.uniform(-1.0, 1.0, h.stream());
    if (h.wanted(user))
      h.run(user, std::to_string(len), n * sizeof(T), [&] {
        raft::linalg::mapThenSumReduce(out.p, len, Identity<T>(), h.stream(), in.p);
      });
    if (h.wanted(lib))
      h.run(lib, std::to_string(len), n * sizeof(T), [&] {
        raft::linalg::mapThenSumReduce(out.p, len, raft::identity_op(), h.stream(), in.p);
      });
  }
}

template <typename T>
void bench_argmin(Harness& h)
{
  const std::string name = std::string("Argmin<") + tname<T>() + ",uint32_t,int64_t>";
  if (!h.wanted(name)) return;
  for (std::int64_t rows : {1000, 10000, 100000, 1000000, 10000000})
    for (std::int64_t cols : {64, 128, 256, 512, 1024}) {
      const size_t n = (size_t)rows * cols;
      if (!h.fits(n * sizeof(T))) continue;
      DeviceBuf<T> matrix(n);
      DeviceBuf<std::uint32_t> indices((size_t)rows);
      matrix.uniform(-1.0, 1.0, h.stream());
      h.run(name, shape2(rows, cols), n * sizeof(T), [&] {
        auto mv =
          raft::make_device_matrix_view<const T, std::int64_t, raft::row_major>(matrix.p, rows, cols);
        auto iv = raft::make_device_vector_view<std::uint32_t, std::int64_t>(indices.p, rows);
        raft::matrix::argmin(h.handle(), mv, iv);
      });
    }
}

// bench/prims/linalg/matrix_vector_op.cu:136-176: round dimensions in both layouts and
// broadcast directions, then odd widths with input / output pointers one element off
struct Add1Vec {
  template <typename T>
  __host__ __device__ T operator()(T a, T b) const { return a + b; }
};
struct Add2Vec {
  template <typename T>
  __host__ __device__ T operator()(T a, T b, T c) const { return a + b + c; }
};

template <typename T, bool TWO>
void bench_mat_vec_op(Harness& h)
{
  const std::string name = std::string("matrixVectorOp<") + tname<T>() + (TWO ? ",2 vectors>" : ",1 vector>");
  if (!h.wanted(name)) return;
  struct Case { long long rows, cols; bool row_major, along_rows; int in_off, out_off; };
  std::vector<Case> cases;
  for (bool rm : {true, false})
    for (bool ar : {true, false})
      for (long long rows : {1000LL, 100000LL, 1000000LL})
        for (long long cols : {8LL, 64LL, 256LL, 1024LL})
          cases.push_back({rows, cols, rm, ar, 0, 0});
  for (bool rm : {true, false})
    for (bool ar : {true, false})
      for (auto rc : std::vector<std::pair<long long, long long>>{{44739207, 7}, {44739207, 15}, {44739207, 16},
                                                                  {44739207, 17}, {2611236, 256}, {2611236, 257},
                                                                  {2611236, 263}})
        for (int io : {0, 1})
          for (int oo : {0, 1})
            cases.push_back({rc.first, rc.second, rm, ar, io, oo});
  for (const auto& c : cases) {
    const size_t n = (size_t)c.rows * c.cols;
    if (!h.fits(2 * n * sizeof(T))) continue;
    DeviceBuf<T> in(n + 1), out(n + 1), v1((size_t)(c.along_rows ? c.cols : c.rows)),
      v2((size_t)(c.along_rows ? c.cols : c.rows));
    in.uniform(-1.0, 1.0, h.stream());
    v1.uniform(-1.0, 1.0, h.stream());
    v2.uniform(-1.0, 1.0, h.stream());
    const std::string shape = shape2(c.rows, c.cols) + (c.row_major ? " rm" : " cm") + (c.along_rows ? " ar" : " ac") +
                              " +" + std::to_string(c.in_off) + "+" + std::to_string(c.out_off);
    h.run(name, shape, 2 * n * sizeof(T), [&] {
      T* o       = out.p + c.out_off;
      const T* i = in.p + c.in_off;
      const long long D = c.cols, N = c.rows;
      auto go = [&](auto rm, auto ar) {
        if constexpr (TWO)
          raft::linalg::matrixVectorOp<decltype(rm)::value, decltype(ar)::value>(o, i, v1.p, v2.p, D, N, Add2Vec{}, h.stream());
        else
          raft::linalg::matrixVectorOp<decltype(rm)::value, decltype(ar)::value>(o, i, v1.p, D, N, Add1Vec{}, h.stream());
      };
      if (c.row_major && c.along_rows) go(std::true_type{}, std::true_type{});
      else if (c.row_major) go(std::true_type{}, std::false_type{});
      else if (c.along_rows) go(std::false_type{}, std::true_type{});
      else go(std::false_type{}, std::false_type{});
    });
  }
}

// ---- copy roof ------------------------------------------------------------------------
typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));

template <int U, bool NT_LD, bool NT_ST, bool PERSIST>
__global__ __launch_bounds__(256) void stream_copy(const u32x4_t* __restrict__ in,
                                                   u32x4_t* __restrict__ out, size_t nvec)
{
  // nvec is a multiple of 256 * U: no tails, the copy's own best case
  const size_t step = (size_t)gridDim.x * 256 * U;
  for (size_t base = (size_t)blockIdx.x * 256 * U; base < nvec; base += step) {
    u32x4_t x[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const u32x4_t* p = in + base + (size_t)u * 256 + threadIdx.x;
      x[u]             = NT_LD ? __builtin_nontemporal_load(p) : *p;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      u32x4_t* q = out + base + (size_t)u * 256 + threadIdx.x;
      if (NT_ST)
        __builtin_nontemporal_store(x[u], q);
      else
        *q = x[u];
    }
    if (!PERSIST) break;
  }
}

template <int U, bool NT_LD, bool NT_ST>
void copy_roof_case(hipStream_t s, int n_cu, size_t bytes, std::vector<void*>& src,
                    std::vector<void*>& dst, hipEvent_t e0, hipEvent_t e1, double& best,
                    std::string& best_name)
{
  const size_t nvec = bytes / 16;
  for (int per_cu : {0, 2, 4, 8, 16}) {  // 0: one workgroup per 256 * U vectors
    const size_t grid = per_cu == 0 ? nvec / (256 * U) : (size_t)n_cu * per_cu;
    auto launch = [&](int i) {
      const u32x4_t* a = static_cast<const u32x4_t*>(src[i % src.size()]);
      u32x4_t* b       = static_cast<u32x4_t*>(dst[i % dst.size()]);
      if (per_cu == 0)
        stream_copy<U, NT_LD, NT_ST, false><<<dim3((unsigned)grid), 256, 0, s>>>(a, b, nvec);
      else
        stream_copy<U, NT_LD, NT_ST, true><<<dim3((unsigned)grid), 256, 0, s>>>(a, b, nvec);
    };
    const int reps = 40;
    for (int i = 0; i < 5; ++i)
      launch(i);
    RAFT_HIP_TRY(hipEventRecord(e0, s));
    for (int i = 0; i < reps; ++i)
      launch(i);
    RAFT_HIP_TRY(hipEventRecord(e1, s));
    RAFT_HIP_TRY(hipEventSynchronize(e1));
    float ms = 0.f;
    RAFT_HIP_TRY(hipEventElapsedTime(&ms, e0, e1));
    const double us   = ms * 1e3 / reps;
    const double gbps = 2.0 * bytes / (us * 1e-6) / 1e9;
    char name[160];
    std::snprintf(name, sizeof name, "loads=%d nt_load=%d nt_store=%d %s", U, (int)NT_LD, (int)NT_ST,
                  per_cu == 0 ? "one-shot" : (std::to_string(per_cu) + " wg/cu").c_str());
    std::printf("%-34s %-22s %10.2f us %9.1f GB/s  %s\n", "copy_roof",
                (std::to_string(bytes >> 20) + "MiB+" + std::to_string(bytes >> 20) + "MiB").c_str(), us,
                gbps, name);
    if (gbps > best) best = gbps, best_name = name;
  }
}

void bench_copy_roof(Harness& h)
{
  if (!h.wanted("copy_roof")) return;
  int n_cu = 256;
  RAFT_HIP_TRY(hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, 0));
  hipEvent_t e0, e1;
  RAFT_HIP_TRY(hipEventCreate(&e0));
  RAFT_HIP_TRY(hipEventCreate(&e1));
  for (size_t bytes : {(size_t)128 << 20, (size_t)512 << 20}) {
    // enough source / destination pairs that a buffer is long out of the 256 MB memory-side
    // cache when its turn comes again
    const int nbuf = bytes >= ((size_t)512 << 20) ? 3 : 6;
    std::vector<void*> src(nbuf), dst(nbuf);
    for (int i = 0; i < nbuf; ++i) {
      RAFT_HIP_TRY(hipMalloc(&src[i], bytes));
      RAFT_HIP_TRY(hipMalloc(&dst[i], bytes));
      fill_words<<<2048, 256, 0, h.stream()>>>(static_cast<unsigned*>(src[i]), bytes / 4, 17u + i);
    }
    RAFT_HIP_TRY(hipStreamSynchronize(h.stream()));
    double best = 0.0;
    std::string best_name;
#define RAFT_COPY_ROOF(U)                                                                         \
  copy_roof_case<U, false, false>(h.stream(), n_cu, bytes, src, dst, e0, e1, best, best_name);    \
  copy_roof_case<U, true, false>(h.stream(), n_cu, bytes, src, dst, e0, e1, best, best_name);     \
  copy_roof_case<U, false, true>(h.stream(), n_cu, bytes, src, dst, e0, e1, best, best_name);     \
  copy_roof_case<U, true, true>(h.stream(), n_cu, bytes, src, dst, e0, e1, best, best_name)
    RAFT_COPY_ROOF(1);
    RAFT_COPY_ROOF(2);
    RAFT_COPY_ROOF(4);
    RAFT_COPY_ROOF(8);
#undef RAFT_COPY_ROOF
    std::printf("%-34s %-22s best %9.1f GB/s  %s\n", "copy_roof/best",
                (std::to_string(bytes >> 20) + "MiB+" + std::to_string(bytes >> 20) + "MiB").c_str(), best,
                best_name.c_str());
    // correctness of the last copy, so the sweep cannot time a kernel that moved nothing
    std::vector<unsigned> a(1024), b(1024);
    RAFT_HIP_TRY(hipMemcpy(a.data(), static_cast<char*>(src[0]) + bytes - 4096, 4096, hipMemcpyDeviceToHost));
    RAFT_HIP_TRY(hipMemcpy(b.data(), static_cast<char*>(dst[0]) + bytes - 4096, 4096, hipMemcpyDeviceToHost));
    if (a != b) std::printf("copy_roof: COPY MISMATCH\n");
    for (int i = 0; i < nbuf; ++i) {
      (void)hipFree(src[i]);
      (void)hipFree(dst[i]);
    }
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
}

// ---- roof of 16-byte accesses off a 16-byte boundary -------------------------------------
// Rows whose byte length is no multiple of 16 (33 bf16, 129 floats, 70 int8) put every lane's
// 16-byte load and store at an address that is only element-aligned.  The same streaming copy
// and read as above, with both pointers moved 2, 4 or 8 bytes off a 16-byte boundary, is the
// ceiling for such shapes: what the memory pipeline sustains when no access is aligned.
typedef u32x4_t u32x4_any_t __attribute__((aligned(1)));

template <bool NT>
__global__ __launch_bounds__(256) void offset_copy(const char* __restrict__ in, char* __restrict__ out)
{
  const size_t i       = ((size_t)blockIdx.x * 256 + threadIdx.x) * 16;
  const u32x4_any_t* p = reinterpret_cast<const u32x4_any_t*>(in + i);
  u32x4_any_t* q       = reinterpret_cast<u32x4_any_t*>(out + i);
  if (NT)
    __builtin_nontemporal_store(__builtin_nontemporal_load(p), q);
  else
    *q = *p;
}

template <bool NT>
__global__ __launch_bounds__(256) void offset_read(const char* __restrict__ in, unsigned* __restrict__ out)
{
  u32x4_t acc = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const size_t i       = (((size_t)blockIdx.x * 4 + u) * 256 + threadIdx.x) * 16;
    const u32x4_any_t* p = reinterpret_cast<const u32x4_any_t*>(in + i);
    acc ^= NT ? __builtin_nontemporal_load(p) : *p;
  }
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u) out[blockIdx.x & 1023] = acc[0];
}

void bench_offset_roof(Harness& h)
{
  if (!h.wanted("offset_roof")) return;
  hipEvent_t e0, e1;
  RAFT_HIP_TRY(hipEventCreate(&e0));
  RAFT_HIP_TRY(hipEventCreate(&e1));
  const size_t bytes = (size_t)256 << 20;
  const int nbuf     = 4;
  std::vector<char*> src(nbuf), dst(nbuf);
  for (int i = 0; i < nbuf; ++i) {
    RAFT_HIP_TRY(hipMalloc(&src[i], bytes + 256));
    RAFT_HIP_TRY(hipMalloc(&dst[i], bytes + 256));
    fill_words<<<2048, 256, 0, h.stream()>>>(reinterpret_cast<unsigned*>(src[i]), (bytes + 256) / 4, 5u + i);
  }
  unsigned* sink = nullptr;
  RAFT_HIP_TRY(hipMalloc(&sink, 4096));
  RAFT_HIP_TRY(hipStreamSynchronize(h.stream()));
  const unsigned copy_grid = (unsigned)(bytes / 16 / 256);
  const unsigned read_grid = copy_grid / 4;
  for (int off : {0, 2, 4, 8}) {
    for (int nt = 0; nt < 2; ++nt) {
      for (int what = 0; what < 2; ++what) {  // 0: copy, 1: read
        auto launch = [&](int i) {
          const char* a = src[i % nbuf] + off;
          char* b       = dst[i % nbuf] + off;
          if (what == 0 && nt) offset_copy<true><<<copy_grid, 256, 0, h.stream()>>>(a, b);
          if (what == 0 && !nt) offset_copy<false><<<copy_grid, 256, 0, h.stream()>>>(a, b);
          if (what == 1 && nt) offset_read<true><<<read_grid, 256, 0, h.stream()>>>(a, sink);
          if (what == 1 && !nt) offset_read<false><<<read_grid, 256, 0, h.stream()>>>(a, sink);
        };
        const int reps = 40;
        for (int i = 0; i < 5; ++i)
          launch(i);
        RAFT_HIP_TRY(hipEventRecord(e0, h.stream()));
        for (int i = 0; i < reps; ++i)
          launch(i);
        RAFT_HIP_TRY(hipEventRecord(e1, h.stream()));
        RAFT_HIP_TRY(hipEventSynchronize(e1));
        float ms = 0.f;
        RAFT_HIP_TRY(hipEventElapsedTime(&ms, e0, e1));
        const double us   = ms * 1e3 / reps;
        const double gbps = (what == 0 ? 2.0 : 1.0) * bytes / (us * 1e-6) / 1e9;
        char name[96];
        std::snprintf(name, sizeof name, "%s +%d bytes non-temporal=%d", what == 0 ? "copy" : "read", off, nt);
        std::printf("%-34s %-22s %10.2f us %9.1f GB/s  %4.1f %% of 8 TB/s  %s\n", "offset_roof",
                    what == 0 ? "256MiB+256MiB" : "256MiB", us, gbps, gbps / 80.0, name);
      }
    }
  }
  for (int i = 0; i < nbuf; ++i) {
    (void)hipFree(src[i]);
    (void)hipFree(dst[i]);
  }
  (void)hipFree(sink);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
}

// ---- read roof ------------------------------------------------------------------------
// What the GPU sustains when a kernel only reads: every lane XORs its 16-byte loads into a
// register and one word per workgroup is written at the end (so that nothing can be dropped).
template <int U, bool NT_LD, bool PERSIST>
__global__ __launch_bounds__(256) void stream_read(const u32x4_t* __restrict__ in,
                                                   unsigned* __restrict__ out, size_t nvec)
{
  __shared__ unsigned sm[4];
  u32x4_t acc       = {0u, 0u, 0u, 0u};
  const size_t step = (size_t)gridDim.x * 256 * U;
  for (size_t base = (size_t)blockIdx.x * 256 * U; base < nvec; base += step) {
    u32x4_t x[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const u32x4_t* p = in + base + (size_t)u * 256 + threadIdx.x;
      x[u]             = NT_LD ? __builtin_nontemporal_load(p) : *p;
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
      acc ^= x[u];
    if (!PERSIST) break;
  }
  unsigned w = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
  for (int m = 32; m >= 1; m >>= 1)
    w ^= (unsigned)__shfl_xor((int)w, m, 64);
  if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = w;
  __syncthreads();
  if (threadIdx.x == 0) out[blockIdx.x] = sm[0] ^ sm[1] ^ sm[2] ^ sm[3];
}

template <int U, bool NT_LD>
void read_roof_case(hipStream_t s, int n_cu, size_t bytes, std::vector<void*>& src, unsigned* out,
                    hipEvent_t e0, hipEvent_t e1, double& best, std::string& best_name)
{
  const size_t nvec = bytes / 16;
  for (int per_cu : {0, 2, 4, 8, 16}) {  // 0: one workgroup per 256 * U vectors
    const size_t grid = per_cu == 0 ? nvec / (256 * U) : (size_t)n_cu * per_cu;
    auto launch = [&](int i) {
      const u32x4_t* a = static_cast<const u32x4_t*>(src[i % src.size()]);
      if (per_cu == 0)
        stream_read<U, NT_LD, false><<<dim3((unsigned)grid), 256, 0, s>>>(a, out, nvec);
      else
        stream_read<U, NT_LD, true><<<dim3((unsigned)grid), 256, 0, s>>>(a, out, nvec);
    };
    const int reps = 40;
    for (int i = 0; i < 5; ++i)
      launch(i);
    RAFT_HIP_TRY(hipEventRecord(e0, s));
    for (int i = 0; i < reps; ++i)
      launch(i);
    RAFT_HIP_TRY(hipEventRecord(e1, s));
    RAFT_HIP_TRY(hipEventSynchronize(e1));
    float ms = 0.f;
    RAFT_HIP_TRY(hipEventElapsedTime(&ms, e0, e1));
    const double us   = ms * 1e3 / reps;
    const double gbps = (double)bytes / (us * 1e-6) / 1e9;
    char name[160];
    std::snprintf(name, sizeof name, "loads=%d nt_load=%d %s", U, (int)NT_LD,
                  per_cu == 0 ? "one-shot" : (std::to_string(per_cu) + " wg/cu").c_str());
    std::printf("%-34s %-22s %10.2f us %9.1f GB/s  %s\n", "read_roof",
                (std::to_string(bytes >> 20) + "MiB").c_str(), us, gbps, name);
    if (gbps > best) best = gbps, best_name = name;
  }
}

// Sizes: those of the benchmark shapes (10, 32, 64, 128, 512 and 2440 MiB); the buffers rotate over
// at least 512 MiB so that none is read from the memory-side cache.
void bench_read_roof(Harness& h)
{
  if (!h.wanted("read_roof")) return;
  int n_cu = 256;
  RAFT_HIP_TRY(hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, 0));
  hipEvent_t e0, e1;
  RAFT_HIP_TRY(hipEventCreate(&e0));
  RAFT_HIP_TRY(hipEventCreate(&e1));
  unsigned* out = nullptr;
  RAFT_HIP_TRY(hipMalloc(&out, ((size_t)2560 << 20) / (16 * 256) * sizeof(unsigned)));
  for (size_t mib : {(size_t)10, (size_t)32, (size_t)64, (size_t)128, (size_t)512, (size_t)2440}) {
    const size_t bytes = mib << 20;
    int nbuf           = (int)((((size_t)640 << 20) + bytes - 1) / bytes);
    if (nbuf < 2) nbuf = 2;
    if (nbuf > 64) nbuf = 64;
    std::vector<void*> src(nbuf);
    for (int i = 0; i < nbuf; ++i) {
      RAFT_HIP_TRY(hipMalloc(&src[i], bytes));
      fill_words<<<2048, 256, 0, h.stream()>>>(static_cast<unsigned*>(src[i]), bytes / 4, 29u + i);
    }
    RAFT_HIP_TRY(hipStreamSynchronize(h.stream()));
    double best = 0.0;
    std::string best_name;
#define RAFT_READ_ROOF(U)                                                              \
  read_roof_case<U, false>(h.stream(), n_cu, bytes, src, out, e0, e1, best, best_name); \
  read_roof_case<U, true>(h.stream(), n_cu, bytes, src, out, e0, e1, best, best_name)
    RAFT_READ_ROOF(1);
    RAFT_READ_ROOF(2);
    RAFT_READ_ROOF(4);
    RAFT_READ_ROOF(8);
#undef RAFT_READ_ROOF
    std::printf("%-34s %-22s best %9.1f GB/s  %s\n", "read_roof/best",
                (std::to_string(bytes >> 20) + "MiB").c_str(), best, best_name.c_str());
    for (int i = 0; i < nbuf; ++i)
      (void)hipFree(src[i]);
  }
  (void)hipFree(out);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
}

// ---- call path ------------------------------------------------------------------------
// Back-to-back calls of the smallest benchmark shape (row sums of 10000 x 256 floats, 10 MB:
// 1.3 us at 8 TB/s) over 64 rotating inputs, issued from C++ so that the caller's own cost per
// call is that of a native loop: through the C ABI, through the header API, and as the replay of
// one HIP graph holding the same launches.  Prints the time per call by events and the host's
// time to issue a call.
void bench_call_path(Harness& h)
{
  if (!h.wanted("call_path")) return;
  const int rows = 10000, cols = 256, nbuf = 64, reps = 2048;
  std::vector<DeviceBuf<float>*> in;
  for (int i = 0; i < nbuf; ++i) {
    in.push_back(new DeviceBuf<float>((size_t)rows * cols));
    in.back()->uniform(-1.0, 1.0, h.stream());
  }
  DeviceBuf<float> out((size_t)rows);
  hipStream_t s = h.stream();
  hipEvent_t e0, e1;
  RAFT_HIP_TRY(hipEventCreate(&e0));
  RAFT_HIP_TRY(hipEventCreate(&e1));
  rmi_reduce_desc d{};
  d.in_dtype = RMI_F32, d.out_dtype = RMI_F32, d.layout = RMI_ROW_MAJOR, d.apply = RMI_ALONG_ROWS;
  d.n_rows = rows, d.n_cols = cols;
  d.main_op = RMI_MAIN_IDENTITY, d.reduce_op = RMI_RED_ADD, d.final_op = RMI_FIN_IDENTITY;
  auto via_abi = [&](int i) {
    if (rmi_reduce(&d, in[i % nbuf]->p, out.p, nullptr, 0, s) != RMI_OK) std::abort();
  };
  auto via_header = [&](int i) {
    raft::linalg::reduce<true, true>(out.p, (const float*)in[i % nbuf]->p, cols, rows, 0.0f, s);
  };
  auto timed = [&](const char* what, auto&& call) {
    for (int i = 0; i < 64; ++i)
      call(i);
    RAFT_HIP_TRY(hipStreamSynchronize(s));
    const auto t0 = std::chrono::steady_clock::now();
    RAFT_HIP_TRY(hipEventRecord(e0, s));
    for (int i = 0; i < reps; ++i)
      call(i);
    RAFT_HIP_TRY(hipEventRecord(e1, s));
    const auto t1 = std::chrono::steady_clock::now();
    RAFT_HIP_TRY(hipEventSynchronize(e1));
    float ms = 0.f;
    RAFT_HIP_TRY(hipEventElapsedTime(&ms, e0, e1));
    const double us = ms * 1e3 / reps;
    std::printf("%-34s %-22s %10.2f us %9.1f GB/s  host issues a call in %.2f us\n",
                (std::string("call_path/") + what).c_str(), shape2(rows, cols).c_str(), us,
                (double)rows * (cols + 1) * 4 / (us * 1e-6) / 1e9,
                std::chrono::duration<double, std::micro>(t1 - t0).count() / reps);
  };
  timed("c_abi", via_abi);
  timed("header", via_header);
  // the same launches as one graph: 256 calls captured, replayed reps / 256 times
  hipGraph_t graph;
  hipGraphExec_t exec;
  RAFT_HIP_TRY(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal));
  for (int i = 0; i < 256; ++i)
    via_abi(i);
  RAFT_HIP_TRY(hipStreamEndCapture(s, &graph));
  RAFT_HIP_TRY(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
  RAFT_HIP_TRY(hipGraphLaunch(exec, s));
  RAFT_HIP_TRY(hipStreamSynchronize(s));
  RAFT_HIP_TRY(hipEventRecord(e0, s));
  for (int i = 0; i < reps / 256; ++i)
    RAFT_HIP_TRY(hipGraphLaunch(exec, s));
  RAFT_HIP_TRY(hipEventRecord(e1, s));
  RAFT_HIP_TRY(hipEventSynchronize(e1));
  float ms = 0.f;
  RAFT_HIP_TRY(hipEventElapsedTime(&ms, e0, e1));
  std::printf("%-34s %-22s %10.2f us %9.1f GB/s\n", "call_path/hip_graph",
              shape2(rows, cols).c_str(), ms * 1e3 / reps,
              (double)rows * (cols + 1) * 4 / (ms * 1e-3 / reps) / 1e9);
  RAFT_HIP_TRY(hipGraphExecDestroy(exec));
  RAFT_HIP_TRY(hipGraphDestroy(graph));
  for (auto* b : in)
    delete b;
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
}

}  // namespace

int main(int argc, char** argv)
{
  Options opt;
  for (int i = 1; i < argc; ++i) {
    if (!std::strcmp(argv[i], "--filter") && i + 1 < argc) opt.filter = argv[++i];
    else if (!std::strcmp(argv[i], "--min-iters") && i + 1 < argc) opt.min_iters = std::atoi(argv[++i]);
    else if (!std::strcmp(argv[i], "--max-bytes") && i + 1 < argc) opt.max_bytes = std::strtoull(argv[++i], nullptr, 10);
    else if (!std::strcmp(argv[i], "--no-flush")) opt.flush = false;
    else {
      std::fprintf(stderr, "usage: %s [--filter s] [--min-iters n] [--max-bytes b] [--no-flush]\n", argv[0]);
      return 2;
    }
  }
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess || n == 0) {
    std::fprintf(stderr, "no GPU visible\n");
    return 2;
  }
  Harness h(opt);
  bench_reduce<float>(h);
  bench_reduce<double>(h);
  bench_row_norm<float, int>(h);
  bench_row_norm<double, int>(h);
  bench_row_norm<float, std::int64_t>(h);
  bench_row_norm<double, std::int64_t>(h);
  bench_row_normalize<float, int>(h);
  bench_row_normalize<double, int>(h);
  bench_row_normalize<float, std::int64_t>(h);
  bench_row_normalize<double, std::int64_t>(h);
  bench_map_then_reduce<float>(h);
  bench_map_then_reduce<double>(h);
  bench_argmin<float>(h);
  bench_argmin<double>(h);
  bench_mat_vec_op<float, false>(h);
  bench_mat_vec_op<float, true>(h);
  bench_mat_vec_op<double, false>(h);
  bench_mat_vec_op<double, true>(h);
  bench_copy_roof(h);
  bench_read_roof(h);
  bench_offset_roof(h);
  bench_call_path(h);
  return 0;
}
