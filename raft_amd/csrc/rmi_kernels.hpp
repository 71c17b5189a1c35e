// The gfx950 reduction kernels, templated on an accumulator policy
// (rmi_device.hpp).  VEC16 = true: rows are read as 16-byte vectors
// (global_load_dwordx4 per lane); false: one element per lane-load, used when
// a row's byte length or the base pointer is not a multiple of 16.
//
//   row_lanes_kernel  K whole rows inside one 16-byte vector: no cross-lane step
//   row_short_kernel  rows of at most G<=8 vectors: one vector per lane, G lanes
//                     per row, 4 row-tiles in flight per wave
//   row_wave_kernel   G<=64 lanes of one wave sweep a row, 4 loads in flight
//   row_block_kernel  teams of 64..1024 threads per row chunk, B chunks per row;
//                     B == 1 writes outputs, B > 1 writes partials
//   col_kernel        reduction along the strided dimension
//   fold_kernel       second pass: partials[n_out][B] -> outputs
#pragma once

#include "rmi_device.hpp"

namespace rmi {

constexpr int kBlock = 256;  // threads per workgroup of every first-pass kernel
constexpr int kUnroll = 4;   // independent 16-byte loads in flight per lane
constexpr int kColUnroll  = 4;  // rows per lane and tile in the column kernel
constexpr int kTeamUnroll = 8;  // loads in flight per lane in the team-per-row kernel

struct RowArgs {
  const void* in;
  void* partial;   // [n_out][B] accumulators, ROW_SPLIT only
  i64 n_out;       // rows
  i64 len;         // elements per row
  i64 nvec;        // lane-loads per row: len/VEC (VEC16) or len (scalar)
  i64 chunk;       // lane-loads per block chunk (row_block_kernel)
  int G;           // lanes per row (row_short / row_wave)
  int logG;
  int B;           // chunks per row (row_block_kernel)
  int logT;        // row_block_kernel: a team is 64 << logT threads
  Epilogue epi;
};

struct ColArgs {
  const void* in;
  void* partial;      // [n_out][B] accumulators when B > 1
  i64 n_out;          // D: length of the contiguous dimension
  i64 len;            // N: number of strided rows folded
  i64 nvec;           // lane-loads per row: D/VEC (VEC16) or D (scalar)
  int TX;             // lanes along the contiguous dimension (power of two <= 64)
  int logTX;
  int B;              // gridDim.y
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

template <class P, bool VEC16>
struct Loader {
  using in_t                = typename P::in_t;
  static constexpr int STEP = VEC16 ? P::VEC : 1;  // elements per lane-load
};

// A lane-load held in registers between issue and use.
template <class P, bool VEC16>
struct Held {
  using in_t = typename P::in_t;
  using type = std::conditional_t<VEC16, u32x4, typename In<in_t>::nat>;
  static __device__ __forceinline__ type load(const void* in, i64 at)
  {
    if constexpr (VEC16) {
      return load16(static_cast<const u32x4*>(in) + at);
    } else {
      return In<in_t>::ld(static_cast<const in_t*>(in) + at);
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
};

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

// ---------------------------------------------------------------------------
// K rows per 16-byte vector (row length VEC/K elements).  Lane-local.
// ---------------------------------------------------------------------------
template <class P, int K>
__global__ __launch_bounds__(kBlock) void row_lanes_kernel(RowArgs a)
{
  using in_t      = typename P::in_t;
  using acc_t     = typename P::acc_t;
  constexpr int D = P::VEC / K;  // elements per row
  const i64 nfull = a.n_out / K; // vectors made only of whole, in-range rows

  u32x4 x[kUnroll];
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    // consecutive lanes take consecutive vectors within each unroll slot
    const i64 v = ((i64)blockIdx.x * kUnroll + u) * kBlock + threadIdx.x;
    if (v < nfull) x[u] = load16(static_cast<const u32x4*>(a.in) + v);
  }
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    const i64 v = ((i64)blockIdx.x * kUnroll + u) * kBlock + threadIdx.x;
    if (v < nfull) {
      acc_t acc[K];
      static_for<K>([&](auto r) {
        acc[r] = P::neutral();
        static_for<D>([&](auto j) {
          P::push(acc[r], In<in_t>::template get<r * D + j>(x[u]), (i64)j);
        });
      });
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
// Short rows: nvec <= G, one lane-load per lane per row, kUnroll tiles of
// 64/G rows in flight per wave.
// ---------------------------------------------------------------------------
template <class P, bool VEC16>
__global__ __launch_bounds__(kBlock) void row_short_kernel(RowArgs a)
{
  using acc_t     = typename P::acc_t;
  using H         = Held<P, VEC16>;
  constexpr int S = Loader<P, VEC16>::STEP;
  const int lane  = threadIdx.x & (kWave - 1);
  const i64 wid   = (i64)blockIdx.x * (kBlock / kWave) + (threadIdx.x >> 6);
  const int G     = a.G;
  const int R     = kWave >> a.logG;
  const int c     = lane & (G - 1);
  const int g     = lane >> a.logG;
  const bool incol = c < a.nvec;

  typename H::type x[kUnroll];
  i64 row[kUnroll];
#pragma unroll
  for (int t = 0; t < kUnroll; ++t) {
    row[t] = (wid * kUnroll + t) * R + g;
    if (incol && row[t] < a.n_out) x[t] = H::load(a.in, row[t] * a.nvec + c);
  }
  acc_t acc[kUnroll];
#pragma unroll
  for (int t = 0; t < kUnroll; ++t) {
    acc[t] = P::neutral();
    if (incol && row[t] < a.n_out) H::push(acc[t], x[t], (i64)c * S);
  }
#pragma unroll
  for (int t = 0; t < kUnroll; ++t)
    group_allreduce<P>(acc[t], G);

  // Every lane of a group now holds its row's result.  Hand the results to lanes
  // so that consecutive lanes own consecutive rows: the wave's kUnroll*R outputs
  // then leave as one contiguous run per store instead of R-element pieces.
  const i64 wave_row0 = wid * kUnroll * R;
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
// G lanes of one wave per row, looping over the row with kUnroll loads in
// flight per lane.
// ---------------------------------------------------------------------------
template <class P, bool VEC16>
__global__ __launch_bounds__(kBlock) void row_wave_kernel(RowArgs a)
{
  using acc_t     = typename P::acc_t;
  using H         = Held<P, VEC16>;
  constexpr int S = Loader<P, VEC16>::STEP;
  const int lane  = threadIdx.x & (kWave - 1);
  const i64 wid   = (i64)blockIdx.x * (kBlock / kWave) + (threadIdx.x >> 6);
  const int G     = a.G;
  const int R     = kWave >> a.logG;
  const int c     = lane & (G - 1);
  const i64 row   = wid * R + (lane >> a.logG);
  const i64 nvec  = a.nvec;

  acc_t acc = P::neutral();
  if (row < a.n_out) {
    const i64 base = row * nvec;
    i64 v          = c;
    for (; v + (kUnroll - 1) * G < nvec; v += kUnroll * G) {
      typename H::type x[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u)
        x[u] = H::load(a.in, base + v + u * G);
#pragma unroll
      for (int u = 0; u < kUnroll; ++u)
        H::push(acc, x[u], (v + u * G) * S);
    }
    if (v < nvec) {  // fewer than kUnroll lane-loads left for this lane
      typename H::type x[kUnroll - 1];
#pragma unroll
      for (int u = 0; u < kUnroll - 1; ++u)
        if (v + u * G < nvec) x[u] = H::load(a.in, base + v + u * G);
#pragma unroll
      for (int u = 0; u < kUnroll - 1; ++u)
        if (v + u * G < nvec) H::push(acc, x[u], (v + u * G) * S);
    }
  }
  group_allreduce<P>(acc, G);
  if (c == 0 && row < a.n_out) finish<P>(a.epi, row, acc);
}

// ---------------------------------------------------------------------------
// Teams of T = 64 << logT threads (1..16 waves); each team sweeps one chunk of
// one row with kTeamUnroll loads in flight per lane.  A workgroup holds
// blockDim.x / T teams.  B chunks per row: B == 1 writes outputs, B > 1 writes
// partials for the second pass.
// ---------------------------------------------------------------------------
template <class P, bool VEC16>
__global__ __launch_bounds__(1024) void row_block_kernel(RowArgs a)
{
  using acc_t     = typename P::acc_t;
  using H         = Held<P, VEC16>;
  constexpr int S = Loader<P, VEC16>::STEP;
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
    const i64 v0   = (i64)b * a.chunk;
    const i64 v1   = (v0 + a.chunk < a.nvec) ? (v0 + a.chunk) : a.nvec;
    const i64 base = row * a.nvec;
    i64 v          = v0 + t;
    for (; v + (U - 1) * (i64)T < v1; v += (i64)U * T) {
      typename H::type x[U];
#pragma unroll
      for (int u = 0; u < U; ++u)
        x[u] = H::load(a.in, base + v + (i64)u * T);
#pragma unroll
      for (int u = 0; u < U; ++u)
        H::push(acc, x[u], (v + (i64)u * T) * S);
    }
    if (v < v1) {  // fewer than U lane-loads left for this lane
      typename H::type x[U - 1];
#pragma unroll
      for (int u = 0; u < U - 1; ++u)
        if (v + (i64)u * T < v1) x[u] = H::load(a.in, base + v + (i64)u * T);
#pragma unroll
      for (int u = 0; u < U - 1; ++u)
        if (v + (i64)u * T < v1) H::push(acc, x[u], (v + (i64)u * T) * S);
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
    } else {
      static_cast<acc_t*>(a.partial)[row * a.B + b] = acc;
    }
  }
}

// ---------------------------------------------------------------------------
// Reduction along the strided dimension of a [len][n_out] row-major array.
// Thread (tx, ty): tx owns one lane-load wide group of adjacent columns for
// the whole kernel, ty strides over the rows of the tiles dealt to this block.
// ---------------------------------------------------------------------------
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

template <class P, bool VEC16>
__global__ __launch_bounds__(kBlock) void col_kernel(ColArgs a)
{
  using acc_t     = typename P::acc_t;
  using in_t      = typename P::in_t;
  constexpr int S = VEC16 ? P::VEC : 1;
  constexpr int W = kBlock / kWave;
  __shared__ acc_t sm[W * kWave * S];

  const int t    = threadIdx.x;
  const int TX   = a.TX;
  const int TY   = kBlock >> a.logTX;
  const int tx   = t & (TX - 1);
  const int ty   = t >> a.logTX;
  const i64 cv   = (i64)blockIdx.x * TX + tx;
  const bool live = cv < a.nvec;
  // Row tiles of TY*kColUnroll rows are dealt round-robin over blockIdx.y, so at any
  // moment the blocks of the grid read one compact, advancing window of the matrix.
  const i64 RT     = (i64)TY * kColUnroll;
  const i64 n_full = a.len / RT;

  acc_t acc[S];
#pragma unroll
  for (int j = 0; j < S; ++j)
    acc[j] = P::neutral();

  if (live) {
    if constexpr (VEC16) {
      const u32x4* p = static_cast<const u32x4*>(a.in) + cv;
      // two tiles in flight: the loads of the next tile are issued before the
      // current one is accumulated
      i64 tile = blockIdx.y;
      u32x4 x[kColUnroll];
      if (tile < n_full) {
#pragma unroll
        for (int u = 0; u < kColUnroll; ++u)
          x[u] = load16(p + (tile * RT + ty + (i64)u * TY) * a.nvec);
      }
      while (tile < n_full) {
        const i64 next = tile + a.B;
        u32x4 y[kColUnroll];
        if (next < n_full) {
#pragma unroll
          for (int u = 0; u < kColUnroll; ++u)
            y[u] = load16(p + (next * RT + ty + (i64)u * TY) * a.nvec);
        }
#pragma unroll
        for (int u = 0; u < kColUnroll; ++u)
          P::push_cols(acc, x[u], tile * RT + ty + (i64)u * TY);
#pragma unroll
        for (int u = 0; u < kColUnroll; ++u)
          x[u] = y[u];
        tile = next;
      }
      if ((i64)blockIdx.y == n_full % a.B) {  // the rows past the last whole tile
        for (i64 r = n_full * RT + ty; r < a.len; r += TY)
          P::push_cols(acc, load16(p + r * a.nvec), r);
      }
    } else {
      const in_t* p = static_cast<const in_t*>(a.in) + cv;
      for (i64 tile = blockIdx.y; tile < n_full; tile += a.B) {
        const i64 r = tile * RT + ty;
        typename In<in_t>::nat x[kColUnroll];
#pragma unroll
        for (int u = 0; u < kColUnroll; ++u)
          x[u] = In<in_t>::ld(p + (r + (i64)u * TY) * a.nvec);
#pragma unroll
        for (int u = 0; u < kColUnroll; ++u)
          P::push(acc[0], x[u], r + (i64)u * TY);
      }
      if ((i64)blockIdx.y == n_full % a.B) {
        for (i64 r = n_full * RT + ty; r < a.len; r += TY)
          P::push(acc[0], In<in_t>::ld(p + r * a.nvec), r);
      }
    }
  }

  // lanes of one wave that share tx sit TX, 2*TX, ... apart
  for (int m = TX; m < kWave; m <<= 1) {
#pragma unroll
    for (int j = 0; j < S; ++j)
      P::merge(acc[j], bperm_acc<P>(acc[j], m));
  }
  // one value per (wave, tx, j) through LDS, folded by the block's first TX threads
  const int lane = t & (kWave - 1);
  const int wave = t >> 6;
  constexpr int NW = W;  // every wave covers its own set of ty
  if (lane < TX) {
#pragma unroll
    for (int j = 0; j < S; ++j)
      sm[(wave * kWave + lane) * S + j] = acc[j];
  }
  __syncthreads();
  if (t < TX && live) {
#pragma unroll
    for (int j = 0; j < S; ++j) {
      acc_t r = sm[(0 * kWave + t) * S + j];
      for (int w = 1; w < NW; ++w)
        P::merge(r, sm[(w * kWave + t) * S + j]);
      const i64 col = cv * S + j;
      if (a.B == 1) {
        finish<P>(a.epi, col, r);
      } else {
        static_cast<acc_t*>(a.partial)[col * a.B + blockIdx.y] = r;
      }
    }
  }
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
  if (o < a.n_out) {
    const acc_t* p = static_cast<const acc_t*>(a.partial) + o * a.B;
    int b          = lb;
    for (; b + (kUnroll - 1) * a.LB < a.B; b += kUnroll * a.LB) {
      acc_t x[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u)
        x[u] = p[b + u * a.LB];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u)
        P::merge(acc, x[u]);
    }
    for (; b < a.B; b += a.LB)
      P::merge(acc, p[b]);
  }
  group_allreduce<P>(acc, a.LB);
  if (lb == 0 && o < a.n_out) finish<P>(a.epi, o, acc);
}

}  // namespace rmi
