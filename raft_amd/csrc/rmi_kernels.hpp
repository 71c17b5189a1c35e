// The gfx950 reduction kernels, templated on an accumulator policy
// (rmi_device.hpp).  VEC16 = true: a row is read as 16-byte vectors
// (global_load_dwordx4 per lane, at any byte alignment); a row length that is not
// a multiple of the vector width ends with one more vector that overlaps the
// previous one and counts only its new elements.  false: one element per
// lane-load, used for rows shorter than 16 bytes.
//
//   row_lanes_kernel  K whole rows inside one 16-byte vector: no cross-lane step
//   row_short_kernel  one vector per lane, G lanes per row (a power of two up to 8,
//                     or the row's own lane-load count up to 32), 4 row-tiles in
//                     flight per wave
//   row_wave_kernel   G<=64 lanes of one wave per row, at most 4 loads per lane
//   row_dense_kernel  whole adjacent rows per workgroup, one lane-load per load slot, rows
//                     combined through LDS (rows whose lane-loads fill no power of two)
//   row_block_kernel  teams of 64..1024 threads per row chunk, B chunks per row;
//                     B == 1 writes outputs, B > 1 writes partials
//   col_kernel        reduction along the strided dimension
//   col_wide_kernel   ... of rows of more than 128 lane-loads: whole rows per workgroup step
//   fold_kernel       second pass: partials[n_out][B] -> outputs
//   fold_rows_kernel  second pass of col_wide_kernel: partials[B][n_out] -> outputs
#pragma once

#include "rmi_device.hpp"

namespace rmi {

constexpr int kBlock      = 256;  // threads per workgroup (the team kernel may use up to 1024)
constexpr int kUnroll     = 4;    // independent 16-byte loads in flight per lane
constexpr int kColUnroll  = 4;    // rows per lane and tile in the column kernel
constexpr int kStageBytes  = 4096 + 128 + 16;  // LDS staging area of one wave (row_wave_kernel)
constexpr int kStageLoads  = 5;  // lane-loads that cover 4096 + 112 bytes
constexpr int kTeamUnroll = 4;    // lane-loads per batch in the team-per-row kernel
constexpr int kFan        = 16;   // split rows: workgroups per first-level ticket counter
constexpr int kLineWords  = 32;   // a ticket counter has a 128-byte line to itself

struct RowArgs {
  const void* in;
  void* partial;   // [n_out][B] accumulators, ROW_SPLIT only
  i64 n_out;       // rows
  i64 len;         // elements per row
  i64 row_bytes;   // len * sizeof(element)
  i64 nvec;        // whole lane-loads per row: len / VEC (VEC16) or len (element-wise)
  i64 chunk;       // lane-loads per team chunk (row_block_kernel)
  int tail;        // VEC16: elements after the last whole vector (len % VEC)
  int G;           // lanes per row (row_short / row_wave); row_dense_kernel: lane-loads of a row
  int logG;
  int B;           // chunks per row (row_block_kernel)
  int logT;        // row_block_kernel: a team is 64 << logT threads
  int R;           // row_short_kernel, any G: 64 / G rows per wave step;
                   // row_dense_kernel: rows of a bundle, 256 * kDenseSlots / G
  u32 invG;        // row_short_kernel, any G: 65536 / G + 1, so that (x * invG) >> 16 == x / G
  u32 invR;        // likewise for R                              for every x < 64
  u32* ticket;     // row_block_kernel, B > 1: zeroed ticket counters, each alone on a 128-byte
                   // line; the workgroup that takes a row's last ticket folds its partials
                   // (nullptr: a second launch does)
  int LB;          // ... with LB lanes (a power of two <= 64), as fold_kernel would
  int head_skip;   // row_block_kernel, 1- and 2-byte elements: rows are read from their
                   // first whole 32-bit word on, the elements before it by the first thread
  int chunk_rows;  // row_flat_kernel: whole rows of a workgroup's chunk; logG: log2 of the lanes
  float inv_row_bytes;  // ... that fold one row, and 1 / row_bytes
  Epilogue epi;
};

struct ColArgs {
  const void* in;
  void* partial;   // [n_out][B] accumulators when B > 1
  i64 n_out;       // D: length of the contiguous dimension
  i64 len;         // N: number of strided rows folded
  i64 row_bytes;   // D * sizeof(element)
  i64 nvec;        // whole lane-loads per row: D / VEC (VEC16) or D (element-wise)
  int tail;        // VEC16: columns after the last whole vector (D % VEC)
  int TX;          // lanes along the contiguous dimension (<= 128); col_wide_kernel: lane-loads
                   // of a workgroup's piece of a row
  int TY;          // rows per step: kBlock / TX, rounded down; col_wide_kernel: rows of a bundle
  int logTX;       // log2(TX) when TX is a power of two
  int dense;       // TX is not a power of two or exceeds a wave: thread t is lane t % TX of
                   // row t / TX, the last kBlock - TX * TY threads idle, and the rows of a
                   // step are combined through LDS instead of lane exchanges
  int treeTY;      // dense: TY rounded up to a power of two
  int B;           // gridDim.y
  // Rows read in groups (group > 0): `in` is taken as a [len][group * cols] matrix of whole
  // 16-byte vectors, column c of which is real column c % cols; the `rem` elements after
  // the last whole group are added one by one, and every real column gets group * B
  // partials, ordered [cols][group][B].
  int group;
  i64 cols;
  i64 rem;
  Epilogue epi;
};

struct FoldArgs {
  const void* partial;  // [n_out][B]
  i64 n_out;
  int B;
  int LB;  // lanes per output (power of two <= 64)
  int logLB;
  Epilogue epi;
};

// A lane-load held in registers between issue and use.  `row` points at the first
// byte of a row, `v` counts lane-loads from there.
template <class P, bool VEC16>
struct Held {
  using in_t                = typename P::in_t;
  using type                = std::conditional_t<VEC16, u32x4, typename In<in_t>::nat>;
  static constexpr int STEP = VEC16 ? P::VEC : 1;  // elements per lane-load
  static __device__ __forceinline__ type load(const char* row, i64 v)
  {
    if constexpr (VEC16) {
      return load16(row + v * 16);
    } else {
      return In<in_t>::ld(reinterpret_cast<const in_t*>(row) + v);
    }
  }
  static __device__ __forceinline__ void push(typename P::acc_t& a, const type& x, i64 idx0)
  {
    if constexpr (VEC16) {
      P::push_vec(a, x, idx0);
    } else {
      P::push(a, x, idx0);
    }
  }
  // Lane-load `v` of a row of `nvec` whole vectors and `tail` further elements:
  // v < nvec is whole vector v; v == nvec is the overlapping last vector that ends
  // at the row's end (VEC16 rows hold at least one whole vector).
  static __device__ __forceinline__ type load_any(const char* row, i64 v, i64 nvec, i64 len)
  {
    if constexpr (VEC16) {
      return load16(v < nvec ? row + v * 16 : row + (len - P::VEC) * (i64)sizeof(in_t));
    } else {
      return In<in_t>::ld(reinterpret_cast<const in_t*>(row) + v);
    }
  }
  static __device__ __forceinline__ void push_any(typename P::acc_t& a,
                                                  const type& x,
                                                  i64 v,
                                                  i64 nvec,
                                                  i64 len,
                                                  int tail)
  {
    if constexpr (VEC16 && P::kTail == kTailDup) {
      P::push_vec(a, x, v < nvec ? v * P::VEC : len - P::VEC);
    } else if constexpr (VEC16 && P::kTail == kTailZero) {
      // bytes [0, skip) of the overlapping vector are cleared; the masks are wave-uniform
      const int skip = (P::VEC - tail) * (int)sizeof(in_t);
      u32x4 y;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const int s = skip - 4 * w;
        const u32 m = s >= 4 ? 0u : s <= 0 ? ~0u : ~0u << (8 * s);
        y[w]        = v < nvec ? x[w] : x[w] & m;
      }
      P::push_vec(a, y, v * P::VEC);
    } else if constexpr (VEC16) {
      if (v < nvec) {
        P::push_vec(a, x, v * P::VEC);
      } else {
        push_vec_from<P>(a, x, len - P::VEC, P::VEC - tail);
      }
    } else {
      P::push(a, x, v);
    }
  }
};

// Policies that scan a batch of vectors downwards (P::scan_t, see PolKvp).
template <class P, class = void>
struct scans_batches : std::false_type {};
template <class P>
struct scans_batches<P, std::void_t<typename P::scan_t>> : std::true_type {};

// The vectors x[u] with live(u) of one lane's batch into the accumulator; base(u) is the index
// of the first element of x[u] along the row, and rises with u.
template <class P, bool FRESH, int N, class Live, class Base>
__device__ __forceinline__ void scan_batch(typename P::acc_t& acc, const u32x4 (&x)[N], Live live, Base base)
{
  typename P::scan_t s = P::scan_begin();
  static_for<N>([&](auto uu) {
    constexpr int u = N - 1 - decltype(uu)::value;
    if (live(u)) P::template scan_vec<u * P::VEC>(s, x[u]);
  });
  static_assert((P::VEC & (P::VEC - 1)) == 0, "slots split into vector and element by shifts");
  constexpr int kLogVec = P::VEC == 1 ? 0 : P::VEC == 2 ? 1 : P::VEC == 4 ? 2 : P::VEC == 8 ? 3 : 4;
  static_assert((1 << kLogVec) == P::VEC, "vectors of 1 to 16 elements");
  const int u = s.slot < 0 ? 0 : s.slot >> kLogVec;
  P::template scan_end<FRESH>(acc, s, (decltype(acc.key))(base(u) + (s.slot & (P::VEC - 1))));
}

// Accumulator held by lane `src` of the wave (ds_bpermute, word by word).
template <class P>
__device__ __forceinline__ typename P::acc_t shfl_acc(const typename P::acc_t& a, int src)
{
  using acc_t = typename P::acc_t;
  static_assert(sizeof(acc_t) % 4 == 0, "accumulators are moved word by word");
  constexpr int NW = sizeof(acc_t) / 4;
  u32 w[NW];
  __builtin_memcpy(w, &a, sizeof(acc_t));
#pragma unroll
  for (int i = 0; i < NW; ++i)
    w[i] = (u32)__shfl((int)w[i], src, kWave);
  acc_t r;
  __builtin_memcpy(&r, w, sizeof(acc_t));
  return r;
}

// Accumulator of lane (lane ^ mask).
template <class P>
__device__ __forceinline__ typename P::acc_t bperm_acc(const typename P::acc_t& a, int mask)
{
  using acc_t = typename P::acc_t;
  static_assert(sizeof(acc_t) % 4 == 0, "accumulators are moved word by word");
  constexpr int NW = sizeof(acc_t) / 4;
  u32 w[NW];
  __builtin_memcpy(w, &a, sizeof(acc_t));
#pragma unroll
  for (int i = 0; i < NW; ++i)
    w[i] = (u32)__shfl_xor((int)w[i], mask, kWave);
  acc_t r;
  __builtin_memcpy(&r, w, sizeof(acc_t));
  return r;
}

// policies that fold the four 8-bit elements of a word with one instruction (P::kNarrow)
template <class P, class = void>
struct lanes_by_words : std::false_type {};
template <class P>
struct lanes_by_words<P, std::void_t<decltype(P::kNarrow)>> : std::bool_constant<P::kNarrow> {};

// ---------------------------------------------------------------------------
// K rows per 16-byte vector (row length VEC/K elements).  Lane-local; U lane-loads per lane.
// ---------------------------------------------------------------------------
template <class P, int K, int U = kUnroll>
__global__ __launch_bounds__(kBlock) void row_lanes_kernel(RowArgs a)
{
  using in_t      = typename P::in_t;
  using acc_t     = typename P::acc_t;
  constexpr int D = P::VEC / K;  // elements per row
  const i64 nfull = a.n_out / K; // vectors made only of whole, in-range rows
  const char* inb = static_cast<const char*>(a.in);

  u32x4 x[U];
  if (nfull > 0) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      // consecutive lanes take consecutive vectors within each unroll slot; the loads are
      // unconditional (a vector past the end re-reads the last one): loads under a lane
      // mask make the compiler wait for each of them in turn
      const i64 v = ((i64)blockIdx.x * U + u) * kBlock + threadIdx.x;
      x[u]        = load16(inb + (v < nfull ? v : nfull - 1) * 16);
    }
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const i64 v = ((i64)blockIdx.x * U + u) * kBlock + threadIdx.x;
    if (v < nfull) {
      acc_t acc[K];
      if constexpr (lanes_by_words<P>::value && D % 4 == 0) {
        // rows of whole words of 8-bit elements: a dot-product instruction per word
        static_for<K>([&](auto r) {
          int32_t t = P::word_i32(x[u][r * (D / 4)]);
          static_for<D / 4 - 1>([&](auto w) {
            t = P::template red<int32_t>(t, P::word_i32(x[u][r * (D / 4) + w + 1]));
          });
          acc[r] = (acc_t)t;
        });
      } else {
        static_for<K>([&](auto r) {
          acc[r] = P::neutral();
          static_for<D>([&](auto j) {
            P::push(acc[r], In<in_t>::template get<r * D + j>(x[u]), (i64)j);
          });
        });
      }
      finish_run<P, K>(a.epi, v * K, acc);
    }
  }
  // Rows past the last whole vector (fewer than K of them): one lane each.
  if (blockIdx.x == 0 && threadIdx.x < (unsigned)(a.n_out - nfull * K)) {
    const i64 row = nfull * K + threadIdx.x;
    acc_t acc     = P::neutral();
    for (int j = 0; j < D; ++j)
      P::push(acc, In<in_t>::ld(static_cast<const in_t*>(a.in) + row * D + j), (i64)j);
    finish<P>(a.epi, row, acc);
  }
}

// ---------------------------------------------------------------------------
// The last batch of a row (or chunk): N lane-loads per lane at v, v + stride, ...,
// of which those below `end` exist.  N is the same for the whole wave (the caller
// derives it from wave-uniform values and dispatches on it), so no load instruction
// is spent on positions no lane has; within the batch loads are unconditional (a
// position past `end` re-reads the last one) and only the accumulation is masked.
// Loads under a lane mask are conditional definitions, after which the compiler
// copies registers and waits for every load in turn.
// ---------------------------------------------------------------------------
template <class P, bool VEC16, int N, class IdxT>
__device__ __forceinline__ void last_batch(typename P::acc_t& acc, const char* rp, IdxT v,
                                           IdxT stride, IdxT end, i64 nvec, i64 len, int tail)
{
  using H = Held<P, VEC16>;
  typename H::type x[N];
#pragma unroll
  for (int u = 0; u < N; ++u) {
    const IdxT vl = v + u * stride < end ? v + u * stride : end - 1;
    x[u]          = H::load_any(rp, vl, nvec, len);
  }
  if constexpr (VEC16 && scans_batches<P>::value) {
    scan_batch<P, false>(
      acc, x, [&](int u) { return v + u * stride < end; },
      [&](int u) { return v + u * stride < (IdxT)nvec ? (i64)(v + u * stride) * P::VEC : len - P::VEC; });
  } else {
#pragma unroll
    for (int u = 0; u < N; ++u)
      if (v + u * stride < end) H::push_any(acc, x[u], v + u * stride, nvec, len, tail);
  }
}

// n = 1 .. 4 lane-loads per lane, wave-uniform
template <class P, bool VEC16, class IdxT>
__device__ __forceinline__ void last_batch_n(int n, typename P::acc_t& acc, const char* rp,
                                             IdxT v, IdxT stride, IdxT end, i64 nvec, i64 len,
                                             int tail)
{
  switch (n) {
    case 1: last_batch<P, VEC16, 1, IdxT>(acc, rp, v, stride, end, nvec, len, tail); break;
    case 2: last_batch<P, VEC16, 2, IdxT>(acc, rp, v, stride, end, nvec, len, tail); break;
    case 3: last_batch<P, VEC16, 3, IdxT>(acc, rp, v, stride, end, nvec, len, tail); break;
    default: last_batch<P, VEC16, 4, IdxT>(acc, rp, v, stride, end, nvec, len, tail); break;
  }
}

// n = 1 .. 9 lane-loads per lane, wave-uniform (the team kernel's rows of one trip)
template <class P, bool VEC16, class IdxT>
__device__ __forceinline__ void last_batch_n9(int n, typename P::acc_t& acc, const char* rp,
                                              IdxT v, IdxT stride, IdxT end, i64 nvec, i64 len,
                                              int tail)
{
  switch (n) {
    case 5: last_batch<P, VEC16, 5, IdxT>(acc, rp, v, stride, end, nvec, len, tail); break;
    case 6: last_batch<P, VEC16, 6, IdxT>(acc, rp, v, stride, end, nvec, len, tail); break;
    case 7: last_batch<P, VEC16, 7, IdxT>(acc, rp, v, stride, end, nvec, len, tail); break;
    case 8: last_batch<P, VEC16, 8, IdxT>(acc, rp, v, stride, end, nvec, len, tail); break;
    case 9: last_batch<P, VEC16, 9, IdxT>(acc, rp, v, stride, end, nvec, len, tail); break;
    default: last_batch_n<P, VEC16, IdxT>(n, acc, rp, v, stride, end, nvec, len, tail); break;
  }
}

// ---------------------------------------------------------------------------
// Short rows: nvec <= G, one lane-load per lane per row, kUnroll tiles of
// 64/G rows in flight per wave.  ANYG = false: G is a power of two.  true: G is
// the row's lane-load count itself (4..32), 64 / G whole rows share the wave and
// its last 64 % G lanes idle; 9 lane-loads then keep 63 lanes busy where 16
// lanes per row would idle 7 of every 16.
// ---------------------------------------------------------------------------
template <class P, bool VEC16, bool ANYG = false>
__global__ __launch_bounds__(kBlock) void row_short_kernel(RowArgs a)
{
  using acc_t     = typename P::acc_t;
  using H         = Held<P, VEC16>;
  const char* inb = static_cast<const char*>(a.in);
  const int lane  = threadIdx.x & (kWave - 1);
  const i64 wid   = (i64)blockIdx.x * (kBlock / kWave) + (threadIdx.x >> 6);
  const int G     = a.G;
  const int R     = ANYG ? a.R : kWave >> a.logG;
  const int g     = ANYG ? (int)(((u32)lane * a.invG) >> 16) : lane >> a.logG;
  const int c     = ANYG ? lane - g * G : lane & (G - 1);
  const i64 nload  = a.nvec + (a.tail > 0 ? 1 : 0);  // the tail is one more lane-load
  const bool incol = ANYG ? g < R : c < nload;

  // Loads are unconditional: a lane without work (past the row's last lane-load, or a
  // row past the matrix) re-reads the nearest vector that has some.  Loads under a lane
  // mask are conditional definitions, after which the compiler copies registers and
  // waits for every load in turn.
  typename H::type x[kUnroll];
  i64 row[kUnroll];
  const i64 cl = incol ? (i64)c : nload - 1;
#pragma unroll
  for (int t = 0; t < kUnroll; ++t) {
    row[t]       = (wid * kUnroll + t) * R + g;
    const i64 rl = row[t] < a.n_out ? row[t] : a.n_out - 1;
    x[t]         = H::load_any(inb + rl * a.row_bytes, cl, a.nvec, a.len);
  }
  acc_t acc[kUnroll];
#pragma unroll
  for (int t = 0; t < kUnroll; ++t) {
    acc[t] = P::neutral();
    if constexpr (VEC16 && scans_batches<P>::value) {
      const u32x4 one[1] = {x[t]};
      const bool live    = incol && row[t] < a.n_out;
      scan_batch<P, true>(
        acc[t], one, [&](int) { return live; },
        [&](int) { return c < a.nvec ? (i64)c * P::VEC : a.len - P::VEC; });
    } else {
      if (incol && row[t] < a.n_out) H::push_any(acc[t], x[t], c, a.nvec, a.len, a.tail);
    }
  }
  const i64 wave_row0 = wid * kUnroll * R;
  if constexpr (ANYG) {
    // fold each row's lanes into its first one: lane c takes lane c + s for s = 1, 2, 4 ...
    for (int s = 1; s < G; s <<= 1) {
#pragma unroll
      for (int t = 0; t < kUnroll; ++t) {
        const acc_t v = shfl_acc<P>(acc[t], lane + s);
        if (c + s < G) P::merge(acc[t], v);
      }
    }
    // lane q takes the wave's q-th output (tile q / R, row q % R of it): one contiguous
    // run of kUnroll * R <= 64 outputs per wave
    const int tq  = (int)(((u32)lane * a.invR) >> 16);
    const int src = (lane - tq * R) * G;
    acc_t mine    = acc[0];
#pragma unroll
    for (int t = 0; t < kUnroll; ++t) {
      const acc_t v = shfl_acc<P>(acc[t], src);
      if (tq == t) mine = v;
    }
    if (lane < kUnroll * R && wave_row0 + lane < a.n_out) finish<P>(a.epi, wave_row0 + lane, mine);
    return;
  }
#pragma unroll
  for (int t = 0; t < kUnroll; ++t)
    group_allreduce<P>(acc[t], G);

  // Every lane of a group now holds its row's result.  Hand the results to lanes
  // so that consecutive lanes own consecutive rows: the wave's kUnroll*R outputs
  // then leave as one contiguous run per store instead of R-element pieces.
  if (G == 1) {
#pragma unroll
    for (int t = 0; t < kUnroll; ++t)
      if (row[t] < a.n_out) finish<P>(a.epi, row[t], acc[t]);
    return;
  }
  const int logR   = 6 - a.logG;
  const int src    = (lane & (R - 1)) << a.logG;  // first lane of group (lane % R)
  const int my_sub = lane >> logR;                // which R-run of a 64-row span this lane serves
  acc_t mine[kUnroll];
#pragma unroll
  for (int t = 0; t < kUnroll; ++t) {
    const acc_t v = shfl_acc<P>(acc[t], src);
    const int s   = (t << logR) >> 6;                   // 64-row span that tile t falls in
    const int sub = t - ((s << 6) >> logR);             // position of tile t inside that span
#pragma unroll
    for (int sc = 0; sc < kUnroll; ++sc)
      if (s == sc && my_sub == sub) mine[sc] = v;
  }
  const int spans = (kUnroll * R + kWave - 1) >> 6;
#pragma unroll
  for (int sc = 0; sc < kUnroll; ++sc) {
    const int q = lane + (sc << 6);
    if (sc < spans && q < kUnroll * R && wave_row0 + q < a.n_out)
      finish<P>(a.epi, wave_row0 + q, mine[sc]);
  }
}

// ---------------------------------------------------------------------------
// G lanes of one wave per row, kUnroll loads in flight per lane.  The plan
// gives every lane at most kUnroll lane-loads per row (nvec <= kUnroll*G); the
// loop is there for forced plans.
// ---------------------------------------------------------------------------
template <class P, bool VEC16, bool STAGED = false>
__global__ __launch_bounds__(kBlock) void row_wave_kernel(RowArgs a)
{
  using acc_t     = typename P::acc_t;
  using H         = Held<P, VEC16>;
  constexpr int S = H::STEP;
  const int lane  = threadIdx.x & (kWave - 1);
  const i64 wid   = (i64)blockIdx.x * (kBlock / kWave) + (threadIdx.x >> 6);
  const int G     = a.G;
  const int R     = kWave >> a.logG;
  const int c     = lane & (G - 1);
  const i64 row   = wid * R + (lane >> a.logG);
  const i64 nvec  = a.nvec;

  acc_t acc = P::neutral();
  if constexpr (STAGED) {
    // Rows are whole 16-byte vectors (tail == 0) at 16-byte aligned addresses, but their
    // lane-group pieces would straddle 128-byte lines.  The wave reads its R rows as one
    // contiguous span that starts on a line, lane after lane, into its LDS area (every
    // line is requested once), and the lane groups then take their vectors from LDS.
    static_assert(VEC16, "staging moves 16-byte vectors");
    extern __shared__ __attribute__((aligned(16))) char stage_lds[];
    char* lw        = stage_lds + (threadIdx.x >> 6) * kStageBytes;
    const char* inb = static_cast<const char*>(a.in);
    const i64 row0  = wid * R;
    const i64 rows_here = a.n_out - row0 < R ? a.n_out - row0 : R;
    if (rows_here > 0) {
      const i64 s0   = row0 * a.row_bytes;            // the span, in bytes from a.in
      const i64 s1   = s0 + rows_here * a.row_bytes;
      const int lead = (int)((reinterpret_cast<uintptr_t>(inb) + (uintptr_t)s0) & 127);  // multiple of 16
      const i64 w0   = s0 - lead;                     // line-aligned start (may precede a.in)
      // Every lane loads and stores unconditionally: a position outside the span is
      // clamped to the span's first or last vector, which some lane moves anyway (the
      // same line, the same LDS bytes, the same data).  Loads under a lane mask would be
      // conditional definitions, after which the compiler copies registers and waits for
      // each load in turn.
      u32x4 x[kStageLoads];
      i64 off[kStageLoads];
#pragma unroll
      for (int u = 0; u < kStageLoads; ++u) {
        off[u] = w0 + ((i64)u * kWave + lane) * 16;
        off[u] = off[u] < s0 ? s0 : (off[u] > s1 - 16 ? s1 - 16 : off[u]);
        x[u]   = load16(inb + off[u]);
      }
#pragma unroll
      for (int u = 0; u < kStageLoads; ++u)
        *reinterpret_cast<u32x4*>(lw + (off[u] - w0)) = x[u];
    }
    // LDS operations of one wave complete in order; keep the compiler from moving the
    // reads of other lanes' data above the writes
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (row < a.n_out) {
      const int lead = (int)((reinterpret_cast<uintptr_t>(inb) + (uintptr_t)(row0 * a.row_bytes)) & 127);
      const char* rp = lw + lead + (row - row0) * a.row_bytes;
      u32x4 x[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const i64 v = c + u * G < nvec ? c + u * G : nvec - 1;  // clamped, not masked: see above
        x[u]        = *reinterpret_cast<const u32x4*>(rp + v * 16);
      }
      if constexpr (scans_batches<P>::value) {
        scan_batch<P, true>(
          acc, x, [&](int u) { return c + u * G < nvec; }, [&](int u) { return (i64)(c + u * G) * S; });
      } else {
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
          if (c + u * G < nvec) P::push_vec(acc, x[u], (i64)(c + u * G) * S);
      }
    }
  } else if (row < a.n_out) {
    const char* rp = static_cast<const char*>(a.in) + row * a.row_bytes;
    i64 v          = c;
    // Whole batches that every lane of the group takes part in (forced plans only: the
    // automatic plan leaves at most kUnroll lane-loads per lane).  The condition is the
    // same for all lanes of a group: were it per lane, the lanes with one more whole
    // vector would run this loop and the others the masked batch below, one after the
    // other, and the row would take two trips to memory.
    for (; (v - c) + (i64)kUnroll * G <= nvec; v += kUnroll * G) {
      typename H::type x[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u)
        x[u] = H::load(rp, v + u * G);
      if constexpr (VEC16 && scans_batches<P>::value) {
        scan_batch<P, false>(
          acc, x, [](int) { return true; }, [&](int u) { return (v + u * G) * S; });
      } else {
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
          H::push(acc, x[u], (v + u * G) * S);
      }
    }
    const i64 nload = nvec + (a.tail > 0 ? 1 : 0);  // the tail is one more lane-load
    // the last batch: what is left of the row, up to kUnroll lane-loads per lane; the
    // count is the same for every lane of the wave
    const i64 left = nload - (v - c);
    if (left > 0)  // G is a power of two: no 64-bit division on the device
      last_batch_n<P, VEC16, i64>((int)((left + G - 1) >> a.logG), acc, rp, v, (i64)G, nload, nvec,
                                  a.len, a.tail);
  }
  group_allreduce<P>(acc, G);
  if (c == 0 && row < a.n_out) finish<P>(a.epi, row, acc);
}

// The hand-off between workgroups of one launch below is written for the cache hierarchy and
// the s_waitcnt encoding of gfx942 / gfx950 and is outside the HIP memory model; refuse to
// build it for anything else.
#if defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx950__) && !defined(__gfx942__)
#error "the single-launch hand-off between workgroups is written for gfx942 / gfx950"
#endif
// s_waitcnt immediate, gfx9 encoding: vmcnt = 0 (bits 3:0 and 15:14), expcnt (6:4) and
// lgkmcnt (11:8) left at their maxima, i.e. "wait until every vector memory operation of
// this wave has completed or been acknowledged".
constexpr int kWaitVmcnt0 = 0x0F70;

// Partials that another workgroup of the SAME launch reads (single-launch split rows) are
// written and read past the caches, word by word as device-scope relaxed atomics
// (global_store / global_load with sc1): the eight L2 caches of the chip are not coherent
// with each other inside a launch, and making them so with device-scope fences costs a
// write-back and an invalidation of a whole L2 per workgroup (2048 workgroups: 100 us).
template <class T>
__device__ __forceinline__ void store_coherent(T* p, const T& v)
{
  static_assert(sizeof(T) % 8 == 0, "accumulators are moved in 8-byte words");
  constexpr int NW = sizeof(T) / 8;
  u64 w[NW];
  __builtin_memcpy(w, &v, sizeof(T));
#pragma unroll
  for (int i = 0; i < NW; ++i)
    __hip_atomic_store(reinterpret_cast<u64*>(p) + i, w[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <class T>
__device__ __forceinline__ T load_coherent(const T* p)
{
  static_assert(sizeof(T) % 8 == 0, "accumulators are moved in 8-byte words");
  constexpr int NW = sizeof(T) / 8;
  u64 w[NW];
#pragma unroll
  for (int i = 0; i < NW; ++i)
    w[i] = __hip_atomic_load(reinterpret_cast<const u64*>(p) + i, __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
  T v;
  __builtin_memcpy(&v, w, sizeof(T));
  return v;
}

template <class P, bool COHERENT = false>
__device__ __forceinline__ typename P::acc_t fold_lane(const typename P::acc_t* p, int B, int LB,
                                                       int lb);

#ifndef RMI_HEAD_SKIP
#define RMI_HEAD_SKIP 1
#endif
// A stored element as the type the policies accumulate.
template <class T>
__device__ __forceinline__ typename In<T>::nat stored_to_nat(const T& v)
{
  if constexpr (std::is_same_v<T, bf16_t>) {
    return as_f32((u32)v.bits << 16);
  } else {
    return (typename In<T>::nat)v;
  }
}

// ---------------------------------------------------------------------------
// Teams of T = 64 << logT threads (1..16 waves); each team sweeps one chunk of
// one row in batches of kTeamUnroll loads per lane.  A workgroup holds
// blockDim.x / T teams.  B chunks per row: B == 1 writes outputs, B > 1 writes
// partials.  Those are folded by a second launch, or, when the caller brought zeroed
// ticket words (one per row), by the workgroup that finishes a row last: it learns that
// from the ticket it takes, reads the B partials in index order like the second launch
// would, and its ticket wraps the word back to zero.  The order of the fold does not
// depend on which workgroup does it, so results are bitwise repeatable.
// ---------------------------------------------------------------------------
template <class P, bool VEC16>
__global__ __launch_bounds__(1024) void row_block_kernel(RowArgs a)
{
  using acc_t     = typename P::acc_t;
  using H         = Held<P, VEC16>;
  constexpr int S = H::STEP;
  constexpr int U = kTeamUnroll;
  __shared__ acc_t sm[16];

  const int T     = kWave << a.logT;
  const int team  = threadIdx.x >> (6 + a.logT);
  const int t     = threadIdx.x & (T - 1);
  const int teams = blockDim.x >> (6 + a.logT);
  const i64 unit  = (i64)blockIdx.x * teams + team;  // (row, chunk) index
  const bool live = unit < a.n_out * a.B;
  i64 row         = unit;
  int b           = 0;
  if (a.B > 1) {
    row = unit / a.B;
    b   = (int)(unit - row * a.B);
  }

  acc_t acc = P::neutral();
  if (live) {
    const char* rp = static_cast<const char*>(a.in) + row * a.row_bytes;
    i64 nvec = a.nvec, len = a.len;
    int tail = a.tail;
    // Rows that start off a 32-bit word are read from their next whole word on; the one to
    // three elements before it go to the first thread of the row's first chunk, which loads
    // them here, ahead of its vectors, and accumulates them after those (used first, they
    // would add a trip to memory to every row).
    constexpr bool kHead = RMI_HEAD_SKIP != 0 && VEC16 && sizeof(typename P::in_t) < 4 && P::CLS != kClsKvp;
    constexpr int kHeadMax = kHead ? 4 / (int)sizeof(typename P::in_t) - 1 : 1;
    [[maybe_unused]] typename P::in_t hv[kHeadMax];
    [[maybe_unused]] int he = 0;
    if constexpr (kHead) {
      using in_t       = typename P::in_t;
      constexpr int es = (int)sizeof(in_t);
      const int skip = a.head_skip != 0 ? (int)((4 - (reinterpret_cast<uintptr_t>(rp) & 3)) & 3) / es : 0;
      he             = (t == 0 && b == 0) ? skip : 0;
#pragma unroll
      for (int j = 0; j < kHeadMax; ++j)
        if (j < he) hv[j] = reinterpret_cast<const in_t*>(rp)[j];
      rp += skip * es;
      len -= skip;
      nvec = len / P::VEC;
      tail = (int)(len - nvec * P::VEC);
    }
    const i64 v0   = (i64)b * a.chunk;
    const i64 v1   = (v0 + a.chunk < nvec) ? (v0 + a.chunk) : nvec;
    // `vb` is the first lane-load of the team's next batch: every loop condition below
    // is the same for all lanes of the team, so a wave follows one path (a per-lane
    // condition would send the lanes with one more whole batch through a loop and the
    // others through the last batch, one after the other).
    i64 vb = v0;
    // the chunk's lane-loads, the row's tail elements counting as one more for the last chunk
    const i64 vend = v1 + ((tail > 0 && b == a.B - 1) ? 1 : 0);
    // A chunk of at most 2 * U + 1 lane-loads per thread makes ONE trip to memory, whatever its
    // length: every load is issued before the first is used, positions past the chunk re-read
    // its last vector.  (Whole batches first and the rest behind them made two or three
    // dependent trips of rows just beyond a whole batch: fp32 D = 1025 ... 1100 ran at 45-50 %,
    // D = 2049 at 67 %.  The ninth load takes the one vector more of rows like D = 4097.)
    const bool one_trip = vend - v0 <= (i64)(2 * U + 1) * T;
    // A chunk of fewer than three batches per thread is read 2 * U lane-loads at a
    // time: all of it is in flight at once and the accumulate step starts as the first
    // vectors arrive.
    if (!one_trip && a.chunk < (i64)3 * U * T) {
      constexpr int W = 2 * U;
      for (; vb + (i64)W * T <= v1; vb += (i64)W * T) {
        typename H::type x[W];
#pragma unroll
        for (int u = 0; u < W; ++u)
          x[u] = H::load(rp, vb + t + (i64)u * T);
        if constexpr (VEC16 && scans_batches<P>::value) {
          scan_batch<P, false>(
            acc, x, [](int) { return true; }, [&](int u) { return (vb + t + (i64)u * T) * S; });
        } else {
#pragma unroll
          for (int u = 0; u < W; ++u)
            H::push(acc, x[u], (vb + t + (i64)u * T) * S);
        }
      }
    }
    // Whole batches of U lane-loads; the next batch is issued before the current one is
    // accumulated, so its latency overlaps the arithmetic (the loop holds no stores:
    // gfx9 counts loads and stores in one in-order counter).
    if (!one_trip && vb + (i64)U * T <= v1) {
      typename H::type x[U];
#pragma unroll
      for (int u = 0; u < U; ++u)
        x[u] = H::load(rp, vb + t + (i64)u * T);
      for (;;) {
        const i64 vn    = vb + (i64)U * T;
        const bool more = vn + (i64)U * T <= v1;
        typename H::type y[U];
        if (more) {
#pragma unroll
          for (int u = 0; u < U; ++u)
            y[u] = H::load(rp, vn + t + (i64)u * T);
        }
        if constexpr (VEC16 && scans_batches<P>::value) {
          scan_batch<P, false>(
            acc, x, [](int) { return true; }, [&](int u) { return (vb + t + (i64)u * T) * S; });
        } else {
#pragma unroll
          for (int u = 0; u < U; ++u)
            H::push(acc, x[u], (vb + t + (i64)u * T) * S);
        }
        vb = vn;
        if (!more) break;
#pragma unroll
        for (int u = 0; u < U; ++u)
          x[u] = y[u];
      }
    }
    // what is left (or the whole chunk in one trip): at most 2 * U + 1 lane-loads per lane, the
    // overlapping last vector of the row among them
    if (vb < vend)
      last_batch_n9<P, VEC16, i64>((int)((vend - vb + T - 1) >> (6 + a.logT)), acc, rp, vb + t, (i64)T,
                                   vend, nvec, len, tail);
    if constexpr (kHead) {
#pragma unroll
      for (int j = 0; j < kHeadMax; ++j)
        if (j < he) P::push(acc, stored_to_nat<typename P::in_t>(hv[j]), (i64)j);
    }
  }

  wave_allreduce<P>(acc);
  if (a.logT > 0) {  // combine the team's waves through LDS
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & (kWave - 1)) == 0) sm[wave] = acc;
    __syncthreads();
    if (t == 0) {
      const int w0 = team << a.logT;
      for (int w = 1; w < (1 << a.logT); ++w)
        P::merge(acc, sm[w0 + w]);
    }
  }
  if (t == 0 && live) {
    if (a.B == 1) {
      finish<P>(a.epi, row, acc);
    } else if (a.ticket != nullptr) {
      store_coherent(static_cast<acc_t*>(a.partial) + row * a.B + b, acc);
    } else {
      static_cast<acc_t*>(a.partial)[row * a.B + b] = acc;
    }
  }
  if (a.B > 1 && a.ticket != nullptr) {  // one team per workgroup here (T == blockDim.x)
    // Only the first wave goes on: it holds the thread that stored the partial, and its
    // lanes learn from that thread whether they fold (a value read from its first lane,
    // no barrier and no trip through LDS).
    if (threadIdx.x >= kWave) return;
    int last = 0;
    if (threadIdx.x == 0 && live) {
      // Counters wrap to zero with their last ticket (atomicInc), so the area is clean for
      // the next call.  Up to kFan chunks: one counter per row.  More: chunks count in
      // groups of kFan, the last of a group counts for the row.  Line 0 of a row's lines
      // is the row's counter, lines 1.. its groups'.
      constexpr int kLine = kLineWords;
      // The partial's stores (past the caches, same thread) must have completed before the
      // ticket is taken.  A device-scope release would do that and write a whole L2 back
      // besides; a workgroup-scope one orders the compiler but emits no wait (the waves of
      // a workgroup share their CU's cache).  So: wait for this wave's outstanding memory
      // operations, after which a write-through store has been acknowledged by the memory
      // side.
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      __builtin_amdgcn_s_waitcnt(kWaitVmcnt0);
      if (a.B <= kFan) {
        last = atomicInc(a.ticket + row * kLine, (u32)a.B - 1) == (u32)a.B - 1;
      } else {
        const int groups = (a.B + kFan - 1) / kFan;
        const int g      = b / kFan;
        const int gsize  = g == groups - 1 ? a.B - g * kFan : kFan;
        u32* lines       = a.ticket + row * (groups + 1) * kLine;
        if (atomicInc(lines + (1 + g) * kLine, (u32)gsize - 1) == (u32)gsize - 1)
          last = atomicInc(lines, (u32)groups - 1) == (u32)groups - 1;
      }
    }
    last = __builtin_amdgcn_readfirstlane(last);
    if (last) {
      // every other workgroup's ticket, and with it its partial, is at the memory side by now
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
      const int lane = threadIdx.x;
      acc_t total    = P::neutral();
      if (lane < a.LB)
        total = fold_lane<P, true>(static_cast<const acc_t*>(a.partial) + row * a.B, a.B, a.LB, lane);
      group_allreduce<P>(total, a.LB);
      if (lane == 0) finish<P>(a.epi, row, total);
    }
  }
}

// ---------------------------------------------------------------------------
// Reduction along the strided dimension of a [len][n_out] row-major array.
// Thread (tx, ty): tx owns one lane-load wide group of adjacent columns for
// the whole kernel, ty strides over the rows of the tiles dealt to this block.
// TX is the row's lane-load count itself when that is at most 128 (TY whole rows
// per step, one contiguous span), else an equal cut of it.
// Persistent: kColBlocksPerCu workgroups per CU; row tiles of TY*kColUnroll rows
// are dealt round-robin over blockIdx.y, so at any moment the grid reads one
// compact, advancing window of the matrix, and a workgroup's next tile is in
// flight while it accumulates the current one.  (The loop holds no stores, which
// is what lets loads stay in flight across iterations: gfx9 counts loads and
// stores in one in-order counter.)
// ---------------------------------------------------------------------------
// policies that gather column terms in 32-bit accumulators first (P::kColNarrow)
template <class P, class = void>
struct col_narrow : std::false_type {};
template <class P>
struct col_narrow<P, std::void_t<decltype(P::kColNarrow)>> : std::bool_constant<P::kColNarrow> {};

template <class P, bool VEC16>
__global__ __launch_bounds__(kBlock) void col_kernel(ColArgs a)
{
  using acc_t     = typename P::acc_t;
  using in_t      = typename P::in_t;
  constexpr int S = VEC16 ? P::VEC : 1;
  constexpr bool NARROW = VEC16 && col_narrow<P>::value;
  // mean-and-variance accumulators: shift set once, count added once (see PolMeanVar)
  constexpr bool SHIFTED = VEC16 && P::CLS == kClsMeanVar;
  // arg-reductions walk the rows downwards, where their rule takes three instructions, not seven
  constexpr bool DOWN = VEC16 && scans_batches<P>::value;
  constexpr int W = kBlock / kWave;
  __shared__ acc_t sm[W * kWave * S];

  const int t      = threadIdx.x;
  const int TX     = a.TX;
  const int TY     = a.TY;
  const int ty     = a.dense ? (int)((unsigned)t / (unsigned)TX) : t >> a.logTX;
  const int tx     = t - ty * TX;
  const bool live  = ty < TY;
  const i64 cv     = (i64)blockIdx.x * TX + tx;
  const bool whole = live && cv < a.nvec;                          // a full lane-load of columns
  const bool part  = live && VEC16 && cv == a.nvec && a.tail > 0;  // the last, partial group
  const i64 RT     = (i64)TY * kColUnroll;
  const i64 n_full = a.len / RT;
  const char* inb  = static_cast<const char*>(a.in);

  acc_t acc[S];
#pragma unroll
  for (int j = 0; j < S; ++j)
    acc[j] = P::neutral();

  if constexpr (VEC16) {
    // The row length need not be a multiple of the vector width: the last, partial
    // group of columns reads the vector that ends at the row's end.  Its first
    // S - tail columns belong to the group before it; they are accumulated here a
    // second time and dropped at the end, which is cheaper than masking every step.
    if (whole || part) {
      const char* p = whole ? inb + cv * 16 : inb + (a.n_out - S) * (i64)sizeof(in_t);
      i64 tile      = blockIdx.y;
      u32x4 x[kColUnroll];
      int32_t narrow[NARROW ? S : 1] = {};
      int gathered                   = 0;  // lane-loads in `narrow`
      auto flush = [&]() {
        if constexpr (NARROW) {
#pragma unroll
          for (int j = 0; j < S; ++j) {
            acc[j] += narrow[j];
            narrow[j] = 0;
          }
          gathered = 0;
        }
      };
      i64 steps = 0;  // SHIFTED: vectors folded by the loop
      // DOWN: the workgroup's tiles are dealt from the matrix's last whole tile backwards and a
      // tile's rows are folded last to first, so a thread meets falling row indices throughout
      auto tile_at = [&](i64 tl) { return DOWN ? n_full - 1 - tl : tl; };
      auto load_tile = [&](u32x4 (&v)[kColUnroll], i64 tl) {
#pragma unroll
        for (int u = 0; u < kColUnroll; ++u)
          v[u] = load16(p + (tl * RT + ty + (i64)u * TY) * a.row_bytes);
      };
      auto fold_tile = [&](const u32x4 (&v)[kColUnroll], i64 tl) {
        if constexpr (NARROW) {
#pragma unroll
          for (int u = 0; u < kColUnroll; ++u)
            P::push_cols_narrow(narrow, v[u]);
          gathered += kColUnroll;
          if (gathered >= P::kColFlush) flush();
        } else if constexpr (SHIFTED) {
#pragma unroll
          for (int u = 0; u < kColUnroll; ++u)
            P::cols_steps(acc, v[u]);
          steps += kColUnroll;
        } else if constexpr (DOWN) {
#pragma unroll
          for (int u = kColUnroll - 1; u >= 0; --u)
            P::push_cols_down(acc, v[u], tl * RT + ty + (i64)u * TY);
        } else {
#pragma unroll
          for (int u = 0; u < kColUnroll; ++u)
            P::push_cols(acc, v[u], tl * RT + ty + (i64)u * TY);
        }
      };
      if (tile < n_full) {
        load_tile(x, tile_at(tile));
        if constexpr (SHIFTED) P::cols_set_shift(acc, x[0]);
      }
      // The next tile's loads are issued before the current tile is folded.  (Two register
      // sets taking turns with unconditional loads, so that the fold waits for its own
      // tile's loads only, measured 1-5 % slower on every shape: sums 355.7 -> 361.8 us on
      // 10M x 64 floats, arg-max 382 -> 401 us, 4M x 129 311 -> 329 us.)
      while (tile < n_full) {
        const i64 next = tile + a.B;
        u32x4 y[kColUnroll];
        if (next < n_full) load_tile(y, tile_at(next));
        fold_tile(x, tile_at(tile));
#pragma unroll
        for (int u = 0; u < kColUnroll; ++u)
          x[u] = y[u];
        tile = next;
      }
      flush();
      if constexpr (SHIFTED) P::cols_count(acc, (double)steps);
      if ((i64)blockIdx.y == n_full % a.B) {  // the rows past the last whole tile
        for (i64 r = n_full * RT + ty; r < a.len; r += TY)
          P::push_cols(acc, load16(p + r * a.row_bytes), r);
        if (a.group > 0 && ty == 0) {  // the real rows past the last whole group
          const in_t* e = reinterpret_cast<const in_t*>(inb + a.len * a.row_bytes) + cv * S;
#pragma unroll
          for (int j = 0; j < S; ++j)
            if (cv * S + j < a.rem) P::push(acc[j], In<in_t>::ld(e + j), 0);
        }
      }
    }
  } else if (whole) {
    const in_t* p = reinterpret_cast<const in_t*>(inb) + cv;
    for (i64 tile = blockIdx.y; tile < n_full; tile += a.B) {
      const i64 r = tile * RT + ty;
      typename In<in_t>::nat x[kColUnroll];
#pragma unroll
      for (int u = 0; u < kColUnroll; ++u)
        x[u] = In<in_t>::ld(p + (r + (i64)u * TY) * a.n_out);
#pragma unroll
      for (int u = 0; u < kColUnroll; ++u)
        P::push(acc[0], x[u], r + (i64)u * TY);
    }
    if ((i64)blockIdx.y == n_full % a.B) {
      for (i64 r = n_full * RT + ty; r < a.len; r += TY)
        P::push(acc[0], In<in_t>::ld(p + r * a.n_out), r);
    }
  }

  if (a.dense) {
    // rows of the step sit TX threads apart: a tree over them in LDS, rows 0..TY-1 of
    // every lane into row 0 (idle threads hold the neutral element)
#pragma unroll
    for (int j = 0; j < S; ++j)
      sm[t * S + j] = acc[j];
    __syncthreads();
    for (int s = a.treeTY >> 1; s >= 1; s >>= 1) {
      if (ty < s && ty + s < TY) {
#pragma unroll
        for (int j = 0; j < S; ++j)
          P::merge(sm[t * S + j], sm[(t + s * TX) * S + j]);
      }
      __syncthreads();
    }
  } else {
    // lanes of one wave that share tx sit TX, 2*TX, ... apart
    for (int m = TX; m < kWave; m <<= 1) {
#pragma unroll
      for (int j = 0; j < S; ++j)
        P::merge(acc[j], bperm_acc<P>(acc[j], m));
    }
    // one value per (wave, tx, j) through LDS, folded by the block's first TX threads
    const int lane = t & (kWave - 1);
    const int wave = t >> 6;
    if (lane < TX) {
#pragma unroll
      for (int j = 0; j < S; ++j)
        sm[(wave * kWave + lane) * S + j] = acc[j];
    }
    __syncthreads();
  }
  if (t < TX && (whole || part)) {
    // the partial group holds the row's last S columns; its first S - tail are
    // already covered by the group before it
    const int first = whole ? 0 : S - a.tail;
    const i64 col0  = whole ? cv * S : a.n_out - S;
#pragma unroll
    for (int j = 0; j < S; ++j) {
      if (j >= first) {
        acc_t r = sm[t * S + j];
        if (!a.dense) {
          for (int w = 1; w < W; ++w)
            P::merge(r, sm[(w * kWave + t) * S + j]);
        }
        const i64 col = col0 + j;
        if (a.group > 0) {
          const unsigned rg = (unsigned)col / (unsigned)a.cols;
          const unsigned c  = (unsigned)col - rg * (unsigned)a.cols;
          static_cast<acc_t*>(a.partial)[((i64)c * a.group + rg) * a.B + blockIdx.y] = r;
        } else if (a.B == 1) {
          finish<P>(a.epi, col, r);
        } else {
          static_cast<acc_t*>(a.partial)[col * a.B + blockIdx.y] = r;
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Rows whose lane-load count fits neither a power-of-two lane group nor whole rows per
// wave (17 lane-loads: 17 of 32 lanes, or 51 of 64).  The 256 * K load slots of a workgroup
// are dealt densely over the lane-loads of a.R adjacent rows (a bundle): slot k of thread t
// is lane-load (k * 256 + t) % G of row (k * 256 + t) / G, so the workgroup reads one
// contiguous span and at most G - 1 slots idle.  Every slot reduces its own vector, the
// values meet in LDS, and one thread per row folds the row's G values in lane order and
// writes the output.  kDenseBundles bundles are in flight (8 loads per thread, all issued
// before the first use); four workgroups per CU take turns between their LDS phases.
// Loads of rows past the matrix are clamped to its last vector and their values dropped.
// ---------------------------------------------------------------------------
constexpr int kDenseSlots   = 2;
constexpr int kDenseBundles = 4;

template <class P>
__global__ __launch_bounds__(kBlock) void row_dense_kernel(RowArgs a)
{
  using acc_t     = typename P::acc_t;
  using in_t      = typename P::in_t;
  using H         = Held<P, true>;
  constexpr int K = kDenseSlots, R = kDenseBundles;
  extern __shared__ __align__(16) unsigned char row_dense_lds[];
  acc_t* sm       = reinterpret_cast<acc_t*>(row_dense_lds);  // [R][rows of a bundle * G]
  const int t     = threadIdx.x;
  const int G     = a.G;  // lane-loads of a row
  const int rb    = a.R;  // rows of a bundle: 256 * K / G
  const int width = rb * G;
  i64 off[K];
  int lane[K];
  bool live[K];
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const unsigned f = (unsigned)(k * kBlock + t);
    const unsigned q = f / (unsigned)G;
    lane[k]          = (int)(f - q * (unsigned)G);
    live[k]          = (int)q < rb;
    off[k] = !live[k] ? 0
                      : (i64)q * a.row_bytes +
                          (lane[k] < a.nvec ? (i64)lane[k] * 16 : (a.len - P::VEC) * (i64)sizeof(in_t));
  }
  const char* inb = static_cast<const char*>(a.in);
  const i64 last  = a.n_out * a.row_bytes - 16;  // the matrix's last whole vector
  const i64 step  = (i64)R * rb;
  for (i64 r = (i64)blockIdx.x * step; r < a.n_out; r += (i64)gridDim.x * step) {
    u32x4 x[R][K];
#pragma unroll
    for (int q = 0; q < R; ++q)
#pragma unroll
      for (int k = 0; k < K; ++k) {
        const i64 o = (r + (i64)q * rb) * a.row_bytes + off[k];
        x[q][k]     = load16(inb + (o < last ? o : last));
      }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int q = 0; q < R; ++q)
#pragma unroll
      for (int k = 0; k < K; ++k) {
        acc_t v = P::neutral();
        if constexpr (scans_batches<P>::value) {
          const u32x4 one[1] = {x[q][k]};
          scan_batch<P, true>(
            v, one, [](int) { return true; },
            [&](int) { return lane[k] < a.nvec ? (i64)lane[k] * P::VEC : a.len - P::VEC; });
        } else {
          H::push_any(v, x[q][k], lane[k], a.nvec, a.len, a.tail);
        }
        if (live[k]) sm[q * width + k * kBlock + t] = v;
      }
    __syncthreads();
    for (int i = t; i < R * rb; i += kBlock) {
      const int q   = i / rb;
      const int rr  = i - q * rb;
      const i64 row = r + (i64)q * rb + rr;
      if (row < a.n_out) {
        const acc_t* p = sm + q * width + rr * G;
        acc_t acc      = p[0];
        for (int l = 1; l < G; ++l)
          P::merge(acc, p[l]);
        finish<P>(a.epi, row, acc);
      }
    }
    __syncthreads();
  }
}

// ---------------------------------------------------------------------------
// Rows shorter than a 16-byte vector that do not divide one (3 floats, 5 bytes ...).  Read
// element by element, a lane per element, such rows ran at 17-35 % of the memory rate.  Here a
// workgroup takes a.chunk_rows whole rows (a multiple of 16 rows, so the chunk starts on a
// 16-byte boundary when the input does; 16 KB at most), reads them as aligned 16-byte vectors
// into LDS, all
// loads in flight at once, and every thread then reduces whole rows out of LDS element by
// element: any reduction, consecutive threads write consecutive outputs.
// ---------------------------------------------------------------------------
constexpr int kSmallVecs  = 4;                    // vectors per thread
constexpr int kSmallBytes = kBlock * kSmallVecs * 16;  // bytes of a workgroup's chunk at most
template <class P>
__global__ __launch_bounds__(kBlock) void row_small_kernel(RowArgs a)
{
  using in_t  = typename P::in_t;
  using acc_t = typename P::acc_t;
  constexpr int ES = (int)sizeof(in_t);
  __shared__ __align__(16) unsigned char sm[kSmallBytes];
  const int t     = threadIdx.x;
  const int rb    = (int)a.row_bytes;
  const i64 row0  = (i64)blockIdx.x * a.chunk_rows;
  const i64 left  = a.n_out - row0;
  const int rows  = left < a.chunk_rows ? (int)left : a.chunk_rows;
  const int bytes = rows * rb;   // kSmallBytes at most
  const int nfull = bytes >> 4;  // whole vectors of the chunk
  const char* base = static_cast<const char*>(a.in) + row0 * rb;
  if (nfull > 0) {
    u32x4 x[kSmallVecs];
#pragma unroll
    for (int k = 0; k < kSmallVecs; ++k) {  // unconditional, clamped
      const int v = t + k * kBlock;
      x[k]        = load16(base + 16 * (v < nfull ? v : nfull - 1));
    }
#pragma unroll
    for (int k = 0; k < kSmallVecs; ++k) {
      const int v = t + k * kBlock;
      if (v < nfull) *reinterpret_cast<u32x4*>(sm + 16 * v) = x[k];
    }
  }
  // what follows the last whole vector (the matrix's last chunk only), element by element
  for (int i = (nfull << 4) / ES + t; i < bytes / ES; i += kBlock)
    reinterpret_cast<in_t*>(sm)[i] = reinterpret_cast<const in_t*>(base)[i];
  __syncthreads();
  const in_t* e = reinterpret_cast<const in_t*>(sm);
  const int D   = (int)a.len;
  for (int r = t; r < rows; r += kBlock) {
    acc_t acc = P::neutral();
    for (int j = 0; j < D; ++j)
      P::push(acc, stored_to_nat<in_t>(e[r * D + j]), (i64)j);
    finish<P>(a.epi, row0 + r, acc);
  }
}

constexpr int kFlatVecs     = 4;                   // vectors per thread
constexpr int kFlatChunkVec = kBlock * kFlatVecs;  // 1024 vector slots, 16 KB
// Thread t takes the vectors t + 256 k - s of its chunk, s = the chunk's offset into its
// 128-byte line in vectors (taken from the output address): every wave-wide load and store
// instruction then covers eight whole lines, not seven and two halves that another
// instruction completes.  The first s slots of a workgroup fall before its chunk and idle, so a
// chunk holds up to kFlatChunkVec - 7 vectors.
constexpr int kFlatMaxVec = kFlatChunkVec - 7;


// ---------------------------------------------------------------------------
// Flat row reduction, for rows whose length is no multiple of a 128-byte line when the
// input starts on a 16-byte boundary.  The matrix is read as a flat run of ALIGNED 16-byte
// vectors, whatever the row length: a workgroup takes a chunk of whole rows that starts on
// a 16-byte boundary (a multiple of 16 / gcd(16, row bytes) rows, at most 16 KB), each
// thread kFlatVecs vectors of it, all loaded before anything else happens.  A vector holds
// elements of at most two rows (rows are 16 bytes or longer): every thread reduces the two
// parts of each of its vectors and leaves them in LDS, and 2^logG lanes per row then fold the
// row's parts in vector order (a fixed order: repeatable bits) and run the epilogue.  The
// matrix's last vector may be a partial one: it is read as the 16 bytes that END at the
// matrix's end and shifted down, so nothing is read past the input.
// ---------------------------------------------------------------------------
// mask of the bytes below s of a 32-bit word (s may be negative or beyond 4)
__device__ __forceinline__ u32 low_bytes_mask(int s)
{
  return s >= 4 ? ~0u : (s <= 0 ? 0u : ((1u << (8 * s)) - 1u));
}
// the vector moved down by k bytes (k in 1..15), zeros moving in at the top
__device__ __forceinline__ u32x4 shift_down_bytes(const u32x4& x, int k)
{
  const int wq = k >> 2, bq = k & 3;
  u32 e[8];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    e[i] = x[i], e[i + 4] = 0u;
  u32x4 y;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    u32 lo = 0u, hi = 0u;
#pragma unroll
    for (int i = 0; i < 4; ++i) {  // a select chain: wq is a run-time value
      if (wq == i) lo = e[w + i], hi = e[w + i + 1];
    }
    y[w] = bq == 0 ? lo : ((lo >> (8 * bq)) | (hi << (32 - 8 * bq)));
  }
  return y;
}

template <class P>
__global__ __launch_bounds__(kBlock) void row_flat_kernel(RowArgs a)
{
  using in_t  = typename P::in_t;
  using acc_t = typename P::acc_t;
  constexpr int VEC = P::VEC;
  constexpr int ES  = (int)sizeof(in_t);
  static_assert(sizeof(acc_t) <= 16, "two accumulators per vector slot are kept in LDS");
  __shared__ acc_t part0[kFlatChunkVec];  // a vector's elements of the row it starts in
  __shared__ acc_t part1[kFlatChunkVec];  // ... and of the next row

  const int t      = threadIdx.x;
  const int rb     = (int)a.row_bytes;
  const i64 row0   = (i64)blockIdx.x * a.chunk_rows;
  const i64 left   = a.n_out - row0;
  const int rows   = left < a.chunk_rows ? (int)left : a.chunk_rows;
  const int bytes  = rows * rb;
  const int rem    = bytes & 15;              // only the matrix's last chunk can end off a boundary
  const int nvec   = (bytes + 15) >> 4;       // vectors of the chunk, the partial one included
  const char* base = static_cast<const char*>(a.in) + row0 * rb;
  const int shift  = (int)((reinterpret_cast<uintptr_t>(base) >> 4) & 7);  // see kFlatMaxVec

  u32x4 x[kFlatVecs];
#pragma unroll
  for (int k = 0; k < kFlatVecs; ++k) {  // unconditional, clamped
    const int v  = t + k * kBlock - shift;
    const int vc = v < 0 ? 0 : (v < nvec ? v : nvec - 1);
    // the partial last vector: the 16 bytes that end at the chunk's end
    x[k] = load16((rem != 0 && vc == nvec - 1) ? base + bytes - 16 : base + 16 * (i64)vc);
  }
#pragma unroll
  for (int k = 0; k < kFlatVecs; ++k) {
    const int v = t + k * kBlock - shift;
    const int b = 16 * (v < 0 ? 0 : v);
    u32x4 xv    = x[k];
    int valid   = 16;  // bytes of the vector that belong to the matrix
    if (rem != 0 && v == nvec - 1) {
      xv    = shift_down_bytes(xv, 16 - rem);
      valid = rem;
    }
    // row that byte b belongs to: b < 16384, so the float quotient is off by one at most
    int r0 = (int)((float)b * a.inv_row_bytes);
    if ((r0 + 1) * rb <= b) ++r0;
    if (r0 * rb > b) --r0;
    const int own  = (r0 + 1) * rb - b;           // bytes from b on that belong to row r0
    const int sb   = own < valid ? own : valid;   // bytes of part 0
    const i64 idx0 = (b - r0 * rb) / ES;          // position in row r0 of the vector's first element
    acc_t s0 = P::neutral(), s1 = P::neutral();
    if constexpr (P::kTail == kTailZero) {
      // sums: cleared elements count for nothing, each part is pushed as a whole vector
      u32x4 lowv, highv;  // bytes [0, sb) and [sb, valid) of the vector
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const u32 m0 = low_bytes_mask(sb - 4 * w);
        lowv[w]      = xv[w] & m0;
        highv[w]     = xv[w] & low_bytes_mask(valid - 4 * w) & ~m0;
      }
      P::push_vec(s0, lowv, idx0);
      P::push_vec(s1, highv, 0);
    } else {
      static_for<VEC>([&](auto j) {
        constexpr int J = decltype(j)::value;
        const auto e    = In<in_t>::template get<J>(xv);
        if (J * ES < sb) P::push(s0, e, idx0 + J);
        else if (J * ES < valid) P::push(s1, e, (i64)J - sb / ES);
      });
    }
    if (v >= 0 && v < nvec) part0[v] = s0, part1[v] = s1;
  }
  __syncthreads();
  const int L     = 1 << a.logG;
  const int c     = t & (L - 1);
  const int step  = kBlock >> a.logG;
  const int npass = (rows + step - 1) / step;  // uniform: every lane of a group takes part in its exchanges
  for (int pass = 0; pass < npass; ++pass) {
    const int r  = pass * step + (t >> a.logG);
    const int rr = r < rows ? r : rows - 1;
    const int bs = rr * rb;
    const int vf = bs >> 4, vl = (bs + rb - 1) >> 4;
    acc_t acc    = P::neutral();
    for (int v = vf + c; v <= vl; v += L)
      P::merge(acc, (v == vf && (bs & 15)) ? part1[v] : part0[v]);
    group_allreduce<P>(acc, L);
    if (c == 0 && r < rows) finish<P>(a.epi, row0 + r, acc);
  }
}

// ---------------------------------------------------------------------------
// Column reduction of wide rows (more than 128 lane-loads).  The workgroup streams whole
// adjacent rows, i.e. one contiguous span of the matrix, where col_kernel reads pieces of at
// most 2 KB at the row's stride (32768 x 4097 floats: 96 us there, 81 us this way; x 2049:
// 99 / 80 us); rows too long for its load slots are cut into gridDim.x equal pieces of a.TX
// lane-loads, up to 20 KB each, and blockIdx.x names the piece.
// A thread has K load slots with a set of accumulators each, as many as 256 bytes of
// accumulators allow.  The 256 * K slots of the workgroup are dealt to the lane-loads of
// a.TY adjacent rows (a bundle) in order: slot k of thread t is lane-load (k * 256 + t) %
// TX of row (k * 256 + t) / TX of the bundle, so a slot always meets the same columns
// and at most TX - 1 slots idle.  R bundles are in flight, and bundles are dealt
// round-robin to the B workgroups.  Every load of a step is issued before the first is
// used, none under a condition (a load behind a branch makes the compiler wait for all
// earlier ones): idle slots load the row's first vector and their accumulators are dropped.
// At the end the bundle's rows are combined through LDS in row order, and the partials are
// stored [B][n_out], whole lines per workgroup; the epilogue is left to the second pass.
// ---------------------------------------------------------------------------
// (byte sums gather in 32-bit accumulators, see PolI::kColNarrow: four slots instead of two;
// the launch keeps the terms per slot below 2^17, so that nothing overflows)
template <class P>
constexpr int col_wide_sets()
{
  constexpr int acc = col_narrow<P>::value ? 4 : (int)sizeof(typename P::acc_t);
  constexpr int k   = 256 / (P::VEC * acc);
  return k < 1 ? 1 : (k > 5 ? 5 : k);
}
constexpr int col_wide_bundles(int K) { return (10 + K - 1) / K; }

template <class P>
__global__ __launch_bounds__(kBlock) void col_wide_kernel(ColArgs a)
{
  using acc_t     = typename P::acc_t;
  using in_t      = typename P::in_t;
  constexpr int S = P::VEC;
  constexpr int K = col_wide_sets<P>();
  constexpr int R = col_wide_bundles(K);
  constexpr bool NARROW = col_narrow<P>::value;
  using slot_t          = std::conditional_t<NARROW, int32_t, acc_t>;  // what a slot accumulates in
  extern __shared__ __align__(16) unsigned char col_wide_lds[];
  slot_t* sm      = reinterpret_cast<slot_t*>(col_wide_lds);  // [rows of a bundle][nload * S]
  const int t     = threadIdx.x;
  const int piece = a.TX;  // lane-loads of this workgroup's piece of a row (the whole row
                           // when it fits the slots), the last piece may hold fewer
  const int rb    = a.TY;  // rows of a bundle: 256 * K / piece
  const i64 total = a.nvec + (a.tail > 0 ? 1 : 0);
  const i64 l0    = (i64)blockIdx.x * piece;
  const int nload = (int)(total - l0 < piece ? total - l0 : piece);
  // byte offset of lane-load l within a row: whole vector l, or the vector that ends at the
  // row's end (its first S - tail columns belong to the lane-load before it)
  auto offset_of = [&](i64 l) { return l < a.nvec ? l * 16 : (a.n_out - S) * (i64)sizeof(in_t); };
  i64 off[K];   // ... of slot k, counted from the bundle's first row
  int sub[K];   // row of the bundle that slot k reads
  int lane[K];  // its lane-load of that row
  bool live[K];
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const unsigned f = (unsigned)(k * kBlock + t);
    const unsigned q = f / (unsigned)piece;
    sub[k]           = (int)q;
    lane[k]          = (int)(f - q * (unsigned)piece);
    live[k]          = (int)q < rb && lane[k] < nload;
    off[k]           = live[k] ? (i64)q * a.row_bytes + offset_of(l0 + lane[k]) : offset_of(l0);
  }
  slot_t acc[K][S];
#pragma unroll
  for (int k = 0; k < K; ++k)
#pragma unroll
    for (int j = 0; j < S; ++j) {
      if constexpr (NARROW) acc[k][j] = 0;
      else acc[k][j] = P::neutral();
    }
  auto push = [&](slot_t (&s)[S], const u32x4& v, i64 row) __attribute__((always_inline)) {
    if constexpr (NARROW) P::push_cols_narrow(s, v);
    else P::push_cols(s, v, row);
  };
  // arg-reductions: the workgroup's whole steps are dealt from the matrix's last one backwards
  // and a step's bundles are folded last to first, so a slot meets falling row indices
  constexpr bool DOWN = !NARROW && scans_batches<P>::value;

  const char* inb   = static_cast<const char*>(a.in);
  const i64 step    = (i64)R * rb;  // rows per step
  const i64 stride  = (i64)a.B * step;
  const i64 n_steps = DOWN ? a.len / step : 0;
  i64 r             = (i64)blockIdx.y * step;
  for (; r + step <= a.len; r += stride) {
    const i64 r0 = DOWN ? (n_steps - 1) * step - r : r;  // the step's first row
    u32x4 x[R][K];
#pragma unroll
    for (int q = 0; q < R; ++q)
#pragma unroll
      for (int k = 0; k < K; ++k)
        x[q][k] = load16(inb + (r0 + (i64)q * rb) * a.row_bytes + off[k]);
    // all of the step's loads first: left to itself the scheduler trades loads in flight for
    // registers and issues four or five of the ten before the first use
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (DOWN) {
#pragma unroll
      for (int q = R - 1; q >= 0; --q)
#pragma unroll
        for (int k = 0; k < K; ++k)
          P::push_cols_down(acc[k], x[q][k], r0 + (i64)q * rb + sub[k]);
    } else {
#pragma unroll
      for (int q = 0; q < R; ++q)
#pragma unroll
        for (int k = 0; k < K; ++k)
          push(acc[k], x[q][k], r0 + (i64)q * rb + sub[k]);
    }
  }
  // the rows after the last whole step go to the workgroup whose turn it is, bundle by bundle
  for (; r < a.len; r += rb) {
#pragma unroll
    for (int k = 0; k < K; ++k)
      if (live[k] && r + sub[k] < a.len)
        push(acc[k], load16(inb + r * a.row_bytes + off[k]), r + sub[k]);
  }

  const int width = nload * S;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    if (live[k]) {
#pragma unroll
      for (int j = 0; j < S; ++j)
        sm[sub[k] * width + lane[k] * S + j] = acc[k][j];
    }
  }
  __syncthreads();
  acc_t* out = static_cast<acc_t*>(a.partial) + (i64)blockIdx.y * a.n_out;
  for (int idx = t; idx < width; idx += kBlock) {
    const int ll = idx / S, j = idx - ll * S;
    const i64 l  = l0 + ll;
    // the last, partial lane-load holds the row's last S columns; its first S - tail are
    // already covered by the lane-load before it
    if (l == a.nvec && j < S - a.tail) continue;
    acc_t v = (acc_t)sm[idx];
    for (int q = 1; q < rb; ++q)
      P::merge(v, (acc_t)sm[q * width + idx]);
    out[l < a.nvec ? l * S + j : a.n_out - S + j] = v;
  }
}

// Second pass of col_wide_kernel over partials[B][n_out]: a workgroup folds 16 adjacent
// outputs (its loads cover whole lines of 8-byte accumulators); thread (c, s) folds partials
// s, s + 16, ... of output c in that order, then the 16 s are combined in a fixed tree.
template <class P>
__global__ __launch_bounds__(kBlock) void fold_rows_kernel(FoldArgs a)
{
  using acc_t = typename P::acc_t;
  __shared__ acc_t sm[kBlock];
  const int t = threadIdx.x;
  const int c = t & 15;
  const int s = t >> 4;
  const i64 o = (i64)blockIdx.x * 16 + c;
  acc_t acc   = P::neutral();
  if (o < a.n_out) {
    const acc_t* p = static_cast<const acc_t*>(a.partial) + o;
    int b          = s;
    constexpr int U = 8;  // 256 partials per output: two rounds of loads per thread
    for (; b + (U - 1) * 16 < a.B; b += U * 16) {
      acc_t x[U];
#pragma unroll
      for (int u = 0; u < U; ++u)
        x[u] = p[(i64)(b + u * 16) * a.n_out];
#pragma unroll
      for (int u = 0; u < U; ++u)
        P::merge(acc, x[u]);
    }
    for (; b < a.B; b += 16)
      P::merge(acc, p[(i64)b * a.n_out]);
  }
  sm[t] = acc;
  __syncthreads();
  for (int h = 8; h >= 1; h >>= 1) {
    if (s < h) P::merge(sm[t], sm[t + h * 16]);
    __syncthreads();
  }
  if (s == 0 && o < a.n_out) finish<P>(a.epi, o, sm[t]);
}

// ---------------------------------------------------------------------------
// Lane `lb` of the LB lanes that fold the B partials of one output: partials lb, lb + LB, ...
// in that order.  The caller combines the lanes with group_allreduce<P>(acc, LB).
// ---------------------------------------------------------------------------
template <class P, bool COHERENT>
__device__ __forceinline__ typename P::acc_t fold_lane(const typename P::acc_t* p, int B, int LB,
                                                       int lb)
{
  using acc_t = typename P::acc_t;
  auto get    = [&](int i) {
    if constexpr (COHERENT) {
      return load_coherent(p + i);
    } else {
      return p[i];
    }
  };
  acc_t acc = P::neutral();
  int b     = lb;
  for (; b + (kUnroll - 1) * LB < B; b += kUnroll * LB) {
    acc_t x[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
      x[u] = get(b + u * LB);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
      P::merge(acc, x[u]);
  }
  for (; b < B; b += LB)
    P::merge(acc, get(b));
  return acc;
}

// ---------------------------------------------------------------------------
// Second pass: LB lanes fold the B partials of one output in a fixed order,
// then the epilogue.  B == 0 writes final_op(init) (empty reductions).
// ---------------------------------------------------------------------------
template <class P>
__global__ __launch_bounds__(kBlock) void fold_kernel(FoldArgs a)
{
  using acc_t    = typename P::acc_t;
  const i64 gtid = (i64)blockIdx.x * kBlock + threadIdx.x;
  const i64 o    = gtid >> a.logLB;
  const int lb   = (int)(gtid & (a.LB - 1));
  acc_t acc      = P::neutral();
  if (o < a.n_out) acc = fold_lane<P>(static_cast<const acc_t*>(a.partial) + o * a.B, a.B, a.LB, lb);
  group_allreduce<P>(acc, a.LB);
  if (lb == 0 && o < a.n_out) finish<P>(a.epi, o, acc);
}

}  // namespace rmi
