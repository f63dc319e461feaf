// native_layer_norm over the last N elements of M dense rows: returns y, mean, rstd.
//
//   sub    rows of at most 32 vectors: 1 .. 32 lanes per row, several rows per wave;
//   tile   row fits the registers of 1, 2 or 4 cooperating waves: one HBM read; mean by
//          all-reduce, then the centred second moment from the same registers (exact
//          two-step statistics at single-pass traffic); y written once;
//   block  longer rows: per-thread Welford accumulation, Chan's pairwise merge across
//          lanes (shuffles) and waves (LDS), then the row is re-read (L2) to normalise.
#include <type_traits>

#include "rowtile.h"

namespace mi355 {

constexpr int kLnBlock = kRowBlock;

// BLOCK = 1024 (many rows): gamma and beta are staged once per block in LDS (dynamic,
// 2 * n * sizeof(Wt) bytes) and serve the 1024 / (64 W) rows of the block.  Fetching them from
// L2 for every row makes every wave of the launch hammer the same 16 KB — the few L2 channels
// that hold them — and cost ~15 % of the kernel's time.  BLOCK = 256 (few rows) reads them
// straight from L2 and keeps more blocks in flight.
// SHIFT: rows do not start on 16-byte boundaries (odd row length); see RowTile::load_shifted.
// gamma / beta are then indexed element by element (their vectors do not line up with the row's).
template <typename T, typename Wt, typename S, int NV, bool VEC, int W, int BLOCK, bool SHIFT = false>
__global__ __launch_bounds__(BLOCK) void layernorm_tile_kernel(const T* __restrict__ x, const Wt* __restrict__ w,
                                                              const Wt* __restrict__ b, T* __restrict__ y,
                                                              S* __restrict__ mean_out, S* __restrict__ rstd_out,
                                                              int64_t rows, int64_t n, float eps) {
  using Tile = RowTile<T, NV, VEC, W, BLOCK>;
  constexpr int V = Tile::V;
  constexpr bool STAGE = VEC && !SHIFT && BLOCK > kLnBlock && W <= 4;  // rows over 8 / 16 waves: one row per block, nothing to share
  extern __shared__ __attribute__((aligned(32))) unsigned char ln_smem[];
  __shared__ float red_a[BLOCK / kWave], red_b[BLOCK / kWave];
  const Wt* gs = w;
  const Wt* bs = b;
  const int t = threadIdx.x % Tile::GROUP;
  int64_t row = (int64_t)blockIdx.x * Tile::ROWS_PER_BLOCK + threadIdx.x / Tile::GROUP;
  const bool active = row < rows;  // inactive groups still walk through the barriers
  if (!active) row = rows - 1;
  Tile tile;
  int a = 0;
  if constexpr (SHIFT) {
    a = row_misalignment<T, V>(x + row * n);
    tile.load_shifted(x + row * n, n, a, t, 0.f);
  } else {
    tile.load(x + row * n, n, t, 0.f);
  }
  if constexpr (STAGE) {
    Wt* gl = reinterpret_cast<Wt*>(ln_smem);
    Wt* bl = gl + n;
    constexpr int WV = 16 / sizeof(Wt);
    for (int64_t c = (int64_t)threadIdx.x * WV; c < n; c += (int64_t)BLOCK * WV) {
      if (w) st<Wt, WV>(gl + c, ld<Wt, WV>(w + c));
      if (b) st<Wt, WV>(bl + c, ld<Wt, WV>(b + c));
    }
    gs = gl;
    bs = bl;  // visible after the barrier inside the first group_allreduce (W > 1) or the one below
    if constexpr (W == 1) __syncthreads();
  }
  float s = 0.f;
#pragma unroll
  for (int k = 0; k < NV; ++k)
#pragma unroll
    for (int j = 0; j < V; ++j) s += tile.v[k][j];
  const float inv_n = 1.f / (float)n;
  const float mean = group_allreduce<W>(s, SumOp(), red_a) * inv_n;
  // Centre the tile in place (the output needs v - mean again) and accumulate the second moment.
  // In the vector layout a 128-bit slab is wholly inside or wholly outside the row, so the
  // padding test is made once per slab, not per element.
  float q = 0.f;
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    if constexpr (SHIFT) {
#pragma unroll
      for (int j = 0; j < V; ++j) {
        const int64_t c = Tile::col(k, j, t) - a;  // window position -> column of the row
        const float d = (c >= 0 && c < n) ? tile.v[k][j] - mean : 0.f;
        tile.v[k][j] = d;
        q += d * d;
      }
    } else if constexpr (VEC) {
      if (Tile::col(k, 0, t) < n) {
#pragma unroll
        for (int j = 0; j < V; ++j) {
          const float d = tile.v[k][j] - mean;
          tile.v[k][j] = d;
          q += d * d;
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < V; ++j) {
        const float d = Tile::col(k, j, t) < n ? tile.v[k][j] - mean : 0.f;
        tile.v[k][j] = d;
        q += d * d;
      }
    }
  }
  const float var = group_allreduce<W>(q, SumOp(), red_b) * inv_n;
  const float rstd = rsqrtf(var + eps);
  if (!active) return;
  if (t == 0) {
    mean_out[row] = static_cast<S>(mean);
    rstd_out[row] = static_cast<S>(rstd);
  }
  T* out = y + row * n;
  if constexpr (SHIFT) {
    tile.store_shifted(out, n, a, t, [=](float d, int64_t c) {
      float r = d * rstd;
      if (w) r *= static_cast<float>(w[c]);
      if (b) r += static_cast<float>(b[c]);
      return r;
    });
  } else if constexpr (VEC) {
    // The weight / bias null tests are made once, outside the unrolled loops: inside, the
    // compiler turns them into a branch per element.
    auto emit = [&](auto has_w, auto has_b) {
      constexpr bool HW = decltype(has_w)::value, HB = decltype(has_b)::value;
#pragma unroll
      for (int k = 0; k < NV; ++k) {
        const int64_t c = Tile::col(k, 0, t);
        if (c < n) {
          VecN<Wt, V> g, be;
          if constexpr (HW) g = ld<Wt, V>(gs + c);
          if constexpr (HB) be = ld<Wt, V>(bs + c);
          VecN<T, V> r;
#pragma unroll
          for (int j = 0; j < V; ++j) {
            float f = tile.v[k][j] * rstd;
            if constexpr (HW && HB) f = f * static_cast<float>(g.v[j]) + static_cast<float>(be.v[j]);
            else if constexpr (HW) f *= static_cast<float>(g.v[j]);
            else if constexpr (HB) f += static_cast<float>(be.v[j]);
            r.v[j] = static_cast<T>(f);
          }
          st_nt<T, V>(out + c, r);
        }
      }
    };
    using std::true_type;
    using std::false_type;
    if (w && b) emit(true_type(), true_type());
    else if (w) emit(true_type(), false_type());
    else if (b) emit(false_type(), true_type());
    else emit(false_type(), false_type());
  } else {
    tile.store(out, n, t, [=](float d, int64_t c) {
      float r = d * rstd;
      if (w) r *= static_cast<float>(w[c]);
      if (b) r += static_cast<float>(b[c]);
      return r;
    });
  }
}

// Many rows that each fit one wave's registers (NV slabs of 64 lanes x one 128-bit vector:
// up to 4096 two-byte or 2048 four-byte elements): every wave walks rows wave, wave + waves, ...
// with the NEXT row's loads issued before the current row is reduced, so the memory system
// always holds a row per wave in flight while the reductions and the normalisation run.  One wave
// per row: both all-reduces stay inside the wave (DPP + bpermute), no barrier in the loop.
// gamma / beta are staged once per block in LDS (2 n elements of dynamic shared memory).  Same
// statistics as the tile kernel (mean, then the centred second moment from the registers).
template <typename T, typename S, int NV, bool HW, bool HB>
__global__ __launch_bounds__(kLnBlock) __attribute__((amdgpu_waves_per_eu(4, 8))) void layernorm_stream_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                                   const T* __restrict__ b, T* __restrict__ y,
                                                                   S* __restrict__ mean_out, S* __restrict__ rstd_out,
                                                                   int64_t rows, int64_t n, float eps) {
  constexpr int V = Vec<T>::N;
  extern __shared__ __attribute__((aligned(32))) unsigned char ln_smem[];  // gamma, then beta: 2 n elements
  T* gl = reinterpret_cast<T*>(ln_smem);
  T* bl = gl + n;
  const int lane = threadIdx.x % kWave;
  const int64_t waves = (int64_t)gridDim.x * (kLnBlock / kWave);
  int64_t row = (int64_t)blockIdx.x * (kLnBlock / kWave) + threadIdx.x / kWave;
  bool in[NV];
  VecN<T, V> nxt[NV];
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int64_t c = ((int64_t)k * kWave + lane) * V;
    in[k] = c < n;  // n % V == 0: a vector is inside the row or past it
    if (in[k] && row < rows) nxt[k] = ld_nt<T, V>(x + row * n + c);
  }
  // gamma / beta once per block into LDS, behind the first row's loads
  if constexpr (HW || HB) {
    for (int64_t c = (int64_t)threadIdx.x * V; c < n; c += (int64_t)kLnBlock * V) {
      if constexpr (HW) st<T, V>(gl + c, ld<T, V>(w + c));
      if constexpr (HB) st<T, V>(bl + c, ld<T, V>(b + c));
    }
    __syncthreads();
  }
  const float inv_n = 1.f / (float)n;
  for (; row < rows; row += waves) {
    float v[NV][V];
#pragma unroll
    for (int k = 0; k < NV; ++k)
#pragma unroll
      for (int j = 0; j < V; ++j) v[k][j] = in[k] ? static_cast<float>(nxt[k].v[j]) : 0.f;
    const int64_t ahead = row + waves;
    if (ahead < rows) {
#pragma unroll
      for (int k = 0; k < NV; ++k)
        if (in[k]) nxt[k] = ld_nt<T, V>(x + ahead * n + ((int64_t)k * kWave + lane) * V);
    }
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < NV; ++k)
#pragma unroll
      for (int j = 0; j < V; ++j) s += v[k][j];
    const float mean = wave_allreduce(s, SumOp()) * inv_n;
    float q = 0.f;
#pragma unroll
    for (int k = 0; k < NV; ++k)
      if (in[k]) {
#pragma unroll
        for (int j = 0; j < V; ++j) {
          const float d = v[k][j] - mean;
          v[k][j] = d;
          q += d * d;
        }
      }
    const float rstd = rsqrtf(wave_allreduce(q, SumOp()) * inv_n + eps);
    if (lane == 0) {
      mean_out[row] = static_cast<S>(mean);
      rstd_out[row] = static_cast<S>(rstd);
    }
    T* out = y + row * n;
#pragma unroll
    for (int k = 0; k < NV; ++k)
      if (in[k]) {
        const int64_t c = ((int64_t)k * kWave + lane) * V;
        VecN<T, V> g, be, r;
        if constexpr (HW) g = ld<T, V>(gl + c);
        if constexpr (HB) be = ld<T, V>(bl + c);
#pragma unroll
        for (int j = 0; j < V; ++j) {
          float f = v[k][j] * rstd;
          if constexpr (HW && HB) f = f * static_cast<float>(g.v[j]) + static_cast<float>(be.v[j]);
          else if constexpr (HW) f *= static_cast<float>(g.v[j]);
          else if constexpr (HB) f += static_cast<float>(be.v[j]);
          r.v[j] = static_cast<T>(f);
        }
        st_nt<T, V>(out + c, r);
      }
  }
}

// Rows of at most 32 vectors: G = 1 .. 32 lanes per row, 64 / G rows per wave (per-head q/k
// norms over 64 or 128 elements).  A lane holds one 16-byte vector of its row, or V single
// elements (column t + G j) when rows are not vector-aligned, and loads the gamma / beta of its
// columns once; sums meet by DPP exchanges among the lanes of the row.
template <typename T, typename Wt, typename S, int G, bool VEC>
__global__ __launch_bounds__(kLnBlock) void layernorm_sub_kernel(const T* __restrict__ x, const Wt* __restrict__ w,
                                                                const Wt* __restrict__ b, T* __restrict__ y,
                                                                S* __restrict__ mean_out, S* __restrict__ rstd_out,
                                                                int64_t rows, int64_t n, float eps) {
  constexpr int V = Vec<T>::N;
  static_assert(kLnBlock % G == 0, "groups must not straddle blocks");
  const int t = threadIdx.x % G;
  int64_t row = ((int64_t)blockIdx.x * kLnBlock + threadIdx.x) / G;
  const bool active = row < rows;  // lanes past the last row still take part in the exchanges
  if (!active) row = rows - 1;
  const T* p = x + row * n;
  float v[V], gw[V], gb[V];
  bool in[V];
  if constexpr (VEC) {
    const bool inside = (int64_t)t * V < n;  // n % V == 0: a vector is inside the row or past it
    VecN<T, V> xv;
    VecN<Wt, V> wv, bv;
    if (inside) {
      xv = ld_nt<T, V>(p + t * V);
      if (w) wv = ld<Wt, V>(w + t * V);
      if (b) bv = ld<Wt, V>(b + t * V);
    }
#pragma unroll
    for (int j = 0; j < V; ++j) {
      in[j] = inside;
      v[j] = inside ? static_cast<float>(xv.v[j]) : 0.f;
      gw[j] = inside && w ? static_cast<float>(wv.v[j]) : 1.f;
      gb[j] = inside && b ? static_cast<float>(bv.v[j]) : 0.f;
    }
  } else {
#pragma unroll
    for (int j = 0; j < V; ++j) {
      const int c = t + G * j;
      in[j] = c < n;
      v[j] = in[j] ? static_cast<float>(p[c]) : 0.f;
      gw[j] = in[j] && w ? static_cast<float>(w[c]) : 1.f;
      gb[j] = in[j] && b ? static_cast<float>(b[c]) : 0.f;
    }
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < V; ++j) s += v[j];
  const float inv_n = 1.f / (float)n;
  const float mean = sub_allreduce<G>(s, SumOp()) * inv_n;
  float q = 0.f;
#pragma unroll
  for (int j = 0; j < V; ++j) {
    const float d = in[j] ? v[j] - mean : 0.f;
    v[j] = d;
    q += d * d;
  }
  const float var = sub_allreduce<G>(q, SumOp()) * inv_n;
  const float rstd = rsqrtf(var + eps);
  if (!active) return;
  if (t == 0) {
    mean_out[row] = static_cast<S>(mean);
    rstd_out[row] = static_cast<S>(rstd);
  }
  T* out = y + row * n;
  if constexpr (VEC) {
    if (in[0]) {
      VecN<T, V> r;
#pragma unroll
      for (int j = 0; j < V; ++j) r.v[j] = static_cast<T>(v[j] * rstd * gw[j] + gb[j]);
      st_nt<T, V>(out + t * V, r);
    }
  } else {
#pragma unroll
    for (int j = 0; j < V; ++j)
      if (in[j]) out[t + G * j] = static_cast<T>(v[j] * rstd * gw[j] + gb[j]);
  }
}

// Welford state and Chan's merge, in the accumulation type A (float; double for f64 input).
template <typename T> struct LnAcc { using type = float; };
template <> struct LnAcc<double> { using type = double; };
template <typename A> struct WF {
  A n, mean, m2;
};
template <typename A> __device__ __forceinline__ void wf_update(WF<A>& a, A x) {
  a.n += A(1);
  const A d = x - a.mean;
  a.mean += d / a.n;
  a.m2 += d * (x - a.mean);
}
template <typename A> __device__ __forceinline__ WF<A> wf_merge(WF<A> a, WF<A> b) {
  const A n = a.n + b.n;
  if (n == A(0)) return a;
  const A d = b.mean - a.mean;
  const A fb = b.n / n;
  return {n, a.mean + d * fb, a.m2 + b.m2 + d * d * a.n * fb};
}
template <typename A> __device__ __forceinline__ WF<A> wf_wave_reduce(WF<A> a) {
#pragma unroll
  for (int k = 1; k < kWave; k <<= 1) {
    WF<A> o{__shfl_xor(a.n, k, kWave), __shfl_xor(a.mean, k, kWave), __shfl_xor(a.m2, k, kWave)};
    a = wf_merge(a, o);
  }
  return a;
}

template <typename T, typename W, typename S, bool VEC>
__global__ __launch_bounds__(kLnBlock) void layernorm_block_kernel(const T* __restrict__ x, const W* __restrict__ w,
                                                                  const W* __restrict__ b, T* __restrict__ y,
                                                                  S* __restrict__ mean_out, S* __restrict__ rstd_out,
                                                                  int64_t n, float eps) {
  using A = typename LnAcc<T>::type;
  constexpr int V = Vec<T>::N;
  __shared__ WF<A> smem[kLnBlock / kWave];
  const T* row = x + (int64_t)blockIdx.x * n;
  T* out = y + (int64_t)blockIdx.x * n;
  WF<A> a{A(0), A(0), A(0)};
  if constexpr (VEC) {
    for (int64_t c = (int64_t)threadIdx.x * V; c < n; c += (int64_t)kLnBlock * V) {
      const Vec<T> t = load_vec(row + c);
#pragma unroll
      for (int j = 0; j < V; ++j) wf_update(a, static_cast<A>(t.v[j]));
    }
  } else {
    for (int64_t c = threadIdx.x; c < n; c += kLnBlock) wf_update(a, static_cast<A>(row[c]));
  }
  a = wf_wave_reduce(a);
  if (threadIdx.x % kWave == 0) smem[threadIdx.x / kWave] = a;
  __syncthreads();
  a = smem[0];
#pragma unroll
  for (int k = 1; k < kLnBlock / kWave; ++k) a = wf_merge(a, smem[k]);
  const A mean = a.mean;
  A rstd;
  if constexpr (std::is_same<A, double>::value) rstd = 1.0 / sqrt(a.m2 / (double)n + (double)eps);
  else rstd = rsqrtf(a.m2 / (float)n + eps);
  if (threadIdx.x == 0) {
    mean_out[blockIdx.x] = static_cast<S>(mean);
    rstd_out[blockIdx.x] = static_cast<S>(rstd);
  }
  for (int64_t c = threadIdx.x; c < n; c += kLnBlock) {
    A r = (static_cast<A>(row[c]) - mean) * rstd;
    if (w) r *= static_cast<A>(w[c]);
    if (b) r += static_cast<A>(b[c]);
    out[c] = static_cast<T>(r);
  }
}

// Few, very long rows (plan_row_split): blockIdx.x = chunk, blockIdx.y = row.  Pass 1 leaves the
// Welford state of every chunk in the workspace; pass 2 merges the states of its row (Chan),
// writes mean / rstd (chunk 0) and normalises its chunk.  VEC: x and y rows 16-byte aligned and
// N a multiple of the vector width; gamma / beta are indexed by element (they stay in cache).
template <typename T, bool VEC>
__global__ __launch_bounds__(kLnBlock) void layernorm_split_partial_kernel(const T* __restrict__ x, unsigned char* __restrict__ ws,
                                                                          int64_t n, int64_t chunk) {
  using A = typename LnAcc<T>::type;
  constexpr int V = Vec<T>::N;
  __shared__ WF<A> smem[kLnBlock / kWave];
  const T* row = x + (int64_t)blockIdx.y * n;
  const int64_t c0 = (int64_t)blockIdx.x * chunk, c1 = c0 + chunk < n ? c0 + chunk : n;
  WF<A> a{A(0), A(0), A(0)};
  if constexpr (VEC) {
    for (int64_t c = c0 + (int64_t)threadIdx.x * V; c < c1; c += (int64_t)kLnBlock * V) {
      const Vec<T> t = load_vec(row + c);
#pragma unroll
      for (int j = 0; j < V; ++j) wf_update(a, static_cast<A>(t.v[j]));
    }
  } else {
    for (int64_t c = c0 + threadIdx.x; c < c1; c += kLnBlock) wf_update(a, static_cast<A>(row[c]));
  }
  a = wf_wave_reduce(a);
  if (threadIdx.x % kWave == 0) smem[threadIdx.x / kWave] = a;
  __syncthreads();
  if (threadIdx.x == 0) {
    a = smem[0];
#pragma unroll
    for (int k = 1; k < kLnBlock / kWave; ++k) a = wf_merge(a, smem[k]);
    *reinterpret_cast<WF<A>*>(ws + ((int64_t)blockIdx.y * gridDim.x + blockIdx.x) * kRowPartialBytes) = a;
  }
}

template <typename T, typename W, typename S, bool VEC>
__global__ __launch_bounds__(kLnBlock) void layernorm_split_finish_kernel(const T* __restrict__ x, const W* __restrict__ w,
                                                                         const W* __restrict__ b, T* __restrict__ y,
                                                                         S* __restrict__ mean_out, S* __restrict__ rstd_out,
                                                                         const unsigned char* __restrict__ ws, int64_t n,
                                                                         int64_t chunk, float eps) {
  using A = typename LnAcc<T>::type;
  constexpr int V = Vec<T>::N;
  __shared__ WF<A> smem[kLnBlock / kWave];
  WF<A> a{A(0), A(0), A(0)};
  for (int sp = threadIdx.x; sp < (int)gridDim.x; sp += kLnBlock)
    a = wf_merge(a, *reinterpret_cast<const WF<A>*>(ws + ((int64_t)blockIdx.y * gridDim.x + sp) * kRowPartialBytes));
  a = wf_wave_reduce(a);
  if (threadIdx.x % kWave == 0) smem[threadIdx.x / kWave] = a;
  __syncthreads();
  a = smem[0];
#pragma unroll
  for (int k = 1; k < kLnBlock / kWave; ++k) a = wf_merge(a, smem[k]);
  const A mean = a.mean;
  A rstd;
  if constexpr (std::is_same<A, double>::value) rstd = 1.0 / sqrt(a.m2 / (double)n + (double)eps);
  else rstd = rsqrtf(a.m2 / (float)n + eps);
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    mean_out[blockIdx.y] = static_cast<S>(mean);
    rstd_out[blockIdx.y] = static_cast<S>(rstd);
  }
  const T* row = x + (int64_t)blockIdx.y * n;
  T* out = y + (int64_t)blockIdx.y * n;
  const int64_t c0 = (int64_t)blockIdx.x * chunk, c1 = c0 + chunk < n ? c0 + chunk : n;
  auto norm = [&](A v, int64_t c) {
    A r = (v - mean) * rstd;
    if (w) r *= static_cast<A>(w[c]);
    if (b) r += static_cast<A>(b[c]);
    return r;
  };
  if constexpr (VEC) {
    for (int64_t c = c0 + (int64_t)threadIdx.x * V; c < c1; c += (int64_t)kLnBlock * V) {
      const Vec<T> t = load_vec(row + c);
      VecN<T, V> r;
#pragma unroll
      for (int j = 0; j < V; ++j) r.v[j] = static_cast<T>(norm(static_cast<A>(t.v[j]), c + j));
      st<T, V>(out + c, r);
    }
  } else {
    for (int64_t c = c0 + threadIdx.x; c < c1; c += kLnBlock) out[c] = static_cast<T>(norm(static_cast<A>(row[c]), c));
  }
}

template <typename T, typename W, typename S>
static int run_ln(const void* xv, const void* wv, const void* bv, void* yv, void* mv, void* rv, int64_t M,
                  int64_t N, double eps, void* ws, int64_t ws_bytes, hipStream_t st) {
  const T* x = static_cast<const T*>(xv);
  const W* w = static_cast<const W*>(wv);
  const W* b = static_cast<const W*>(bv);
  T* y = static_cast<T*>(yv);
  S* mean = static_cast<S*>(mv);
  S* rstd = static_cast<S*>(rv);
  constexpr int V = Vec<T>::N;
  const bool has_params = w != nullptr || b != nullptr;
  const bool vec = N % V == 0 && aligned16(x) && aligned16(y) &&
                   reinterpret_cast<uintptr_t>(w) % (sizeof(W) * V) == 0 &&
                   reinterpret_cast<uintptr_t>(b) % (sizeof(W) * V) == 0 && N % (16 / sizeof(W)) == 0;
  MI355_REQUIRE(M < (int64_t(1) << 31), "mi355_layer_norm: too many rows (%lld)", (long long)M);
  const size_t param_bytes = 2 * (size_t)N * sizeof(W);
  bool done = false;
  // few, very long rows: two launches over (row, chunk) when the caller brought the scratch for it
  {
    const RowSplit sp = plan_row_split(M, N, sizeof(T));
    if (sp.nsplit > 1 && ws != nullptr && ws_bytes >= M * sp.nsplit * kRowPartialBytes && reinterpret_cast<uintptr_t>(ws) % 8 == 0) {
      unsigned char* wsp = static_cast<unsigned char*>(ws);
      const dim3 grid((unsigned)sp.nsplit, (unsigned)M);
      const bool xv16 = N % V == 0 && aligned16(x) && aligned16(y);
      if (xv16) {
        hipLaunchKernelGGL((layernorm_split_partial_kernel<T, true>), grid, dim3(kLnBlock), 0, st, x, wsp, N, sp.chunk);
        hipLaunchKernelGGL((layernorm_split_finish_kernel<T, W, S, true>), grid, dim3(kLnBlock), 0, st, x, w, b, y, mean, rstd, wsp, N, sp.chunk, (float)eps);
      } else {
        hipLaunchKernelGGL((layernorm_split_partial_kernel<T, false>), grid, dim3(kLnBlock), 0, st, x, wsp, N, sp.chunk);
        hipLaunchKernelGGL((layernorm_split_finish_kernel<T, W, S, false>), grid, dim3(kLnBlock), 0, st, x, w, b, y, mean, rstd, wsp, N, sp.chunk, (float)eps);
      }
      return check_launch("mi355_layer_norm(split rows)");
    }
  }
  if constexpr (!std::is_same<T, double>::value)
  if (N <= 32 * V) {  // short rows: several per wave
    const int64_t need = (N + V - 1) / V;
#define MI355_LN_SUB(G_)                                                                                  \
  if (!done && need <= G_) {                                                                              \
    const unsigned nblk = (unsigned)((M * G_ + kLnBlock - 1) / kLnBlock);                                   \
    if (vec) hipLaunchKernelGGL((layernorm_sub_kernel<T, W, S, G_, true>), dim3(nblk), dim3(kLnBlock), 0, st, x, w, b, y, mean, rstd, M, N, (float)eps); \
    else hipLaunchKernelGGL((layernorm_sub_kernel<T, W, S, G_, false>), dim3(nblk), dim3(kLnBlock), 0, st, x, w, b, y, mean, rstd, M, N, (float)eps);    \
    done = true;                                                                                          \
  }
    MI355_LN_SUB(1) MI355_LN_SUB(2) MI355_LN_SUB(4) MI355_LN_SUB(8) MI355_LN_SUB(16) MI355_LN_SUB(32)
#undef MI355_LN_SUB
  }
  // Thousands of aligned rows of one wave's worth of registers each, gamma / beta of the input's
  // dtype: the streaming kernel (rows prefetched one ahead, no LDS, no barrier).
  if constexpr (std::is_same<T, W>::value && !std::is_same<T, double>::value)
  if (!done && vec && N > 32 * V && N <= 8 * kWave * V && M >= 4 * kNumCU) {
    // Grid: the blocks that are resident at once (the register tile decides how many), cut so
    // that every wave gets the same number of rows when M allows it.
    auto launch = [&](auto nv) {
      constexpr int NV = decltype(nv)::value;
      auto go = [&](auto hw, auto hb) {
        constexpr bool HW_ = decltype(hw)::value, HB_ = decltype(hb)::value;
        const void* kern = (const void*)layernorm_stream_kernel<T, S, NV, HW_, HB_>;
        static thread_local int resident = 0;  // blocks per CU, per instantiation
        if (resident == 0) {
          int nb = 0;
          if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, kern, kLnBlock, has_params ? param_bytes : 0) != hipSuccess || nb < 1) nb = 2;
          resident = nb;
        }
        const int64_t max_waves = (int64_t)kNumCU * resident * (kLnBlock / kWave);
        const int64_t per_wave = (M + max_waves - 1) / max_waves;
        const int64_t nwaves = (M + per_wave - 1) / per_wave;
        const unsigned nblk = (unsigned)((nwaves + kLnBlock / kWave - 1) / (kLnBlock / kWave));
        hipLaunchKernelGGL((layernorm_stream_kernel<T, S, NV, HW_, HB_>), dim3(nblk), dim3(kLnBlock), has_params ? param_bytes : 0, st, x,
                           reinterpret_cast<const T*>(w), reinterpret_cast<const T*>(b), y, mean, rstd, M, N, (float)eps);
      };
      using std::true_type;
      using std::false_type;
      if (w && b) go(true_type(), true_type());
      else if (w) go(true_type(), false_type());
      else if (b) go(false_type(), true_type());
      else go(false_type(), false_type());
    };
    if (N <= 4 * kWave * V) launch(std::integral_constant<int, 4>());
    else launch(std::integral_constant<int, 8>());
    done = true;
  }
  // Rows that start off a 16-byte boundary (odd N) still take the vector layout, shifted per
  // row, when input and output rows are misaligned by the same number of elements.  Rows under
  // 4000 bytes stay on the single-element layout: there the element-wise gamma / beta indexing of the
  // shifted form costs more than its vector accesses save.
  const bool shift = !vec && V > 1 && N * sizeof(T) >= 4000 &&
                     (reinterpret_cast<uintptr_t>(x) / sizeof(T)) % V == (reinterpret_cast<uintptr_t>(y) / sizeof(T)) % V;
  if constexpr (!std::is_same<T, double>::value)  // f64 rows take the block kernel (double accumulation)
  if (!done)
  done = dispatch_row_tile<T>(shift ? N + V - 1 : N, vec || shift, [&](auto nv, auto wv, auto v) {
    constexpr int NV = decltype(nv)::value, WG = decltype(wv)::value;
    constexpr bool VEC = decltype(v)::value;
    if constexpr (WG >= 8) {  // rows of 8 K - 64 K elements: a 512- or 1024-thread block per row
      constexpr int BLK = kWave * WG;
      if constexpr (VEC) {
        if (shift) {
          hipLaunchKernelGGL((layernorm_tile_kernel<T, W, S, NV, true, WG, BLK, true>), dim3((unsigned)M), dim3(BLK), 0, st, x, w, b, y, mean, rstd, M, N, (float)eps);
          return;
        }
      }
      hipLaunchKernelGGL((layernorm_tile_kernel<T, W, S, NV, VEC, WG, BLK>), dim3((unsigned)M), dim3(BLK), 0, st, x, w, b, y, mean, rstd, M, N, (float)eps);
      return;
    }
    constexpr int BIG = 1024;
    constexpr int rpb_big = WG >= 8 ? 1 : BIG / (kWave * WG), rpb = WG >= 8 ? 1 : kLnBlock / (kWave * WG);
    if constexpr (VEC) {
      if (shift) {
        const unsigned nblk = (unsigned)((M + rpb - 1) / rpb);
        hipLaunchKernelGGL((layernorm_tile_kernel<T, W, S, NV, true, WG, kLnBlock, true>), dim3(nblk), dim3(kLnBlock), 0, st, x, w, b, y, mean, rstd, M, N, (float)eps);
        return;
      }
    }
    // Enough rows to fill the chip with 1024-thread blocks: share gamma/beta through LDS.
    if (VEC && has_params && param_bytes <= 48 * 1024 && M >= (int64_t)rpb_big * 2 * kNumCU) {
      const unsigned nblk = (unsigned)((M + rpb_big - 1) / rpb_big);
      hipLaunchKernelGGL((layernorm_tile_kernel<T, W, S, NV, VEC, WG, BIG>), dim3(nblk), dim3(BIG), param_bytes, st, x, w, b, y, mean, rstd, M, N, (float)eps);
    } else {
      const unsigned nblk = (unsigned)((M + rpb - 1) / rpb);
      hipLaunchKernelGGL((layernorm_tile_kernel<T, W, S, NV, VEC, WG, kLnBlock>), dim3(nblk), dim3(kLnBlock), 0, st, x, w, b, y, mean, rstd, M, N, (float)eps);
    }
  }, 16);
  if (!done) {
    if (vec) hipLaunchKernelGGL((layernorm_block_kernel<T, W, S, true>), dim3((unsigned)M), dim3(kLnBlock), 0, st, x, w, b, y, mean, rstd, N, (float)eps);
    else hipLaunchKernelGGL((layernorm_block_kernel<T, W, S, false>), dim3((unsigned)M), dim3(kLnBlock), 0, st, x, w, b, y, mean, rstd, N, (float)eps);
  }
  return check_launch("mi355_layer_norm");
}

static thread_local void* g_ln_ws = nullptr;
static thread_local int64_t g_ln_ws_bytes = 0;

template <typename T, typename W>
static int run_ln_stat(int stat_dtype, int dtype, const void* x, const void* w, const void* b, void* y, void* m,
                       void* r, int64_t M, int64_t N, double eps, hipStream_t st) {
  if (stat_dtype == MI355_F32) return run_ln<T, W, float>(x, w, b, y, m, r, M, N, eps, g_ln_ws, g_ln_ws_bytes, st);
  if (stat_dtype == dtype) return run_ln<T, W, T>(x, w, b, y, m, r, M, N, eps, g_ln_ws, g_ln_ws_bytes, st);
  return set_error(MI355_ERR_UNSUPPORTED, "mi355_layer_norm: stat dtype must be f32 or the input dtype");
}

}  // namespace mi355

using namespace mi355;

extern "C" int mi355_layer_norm(const void* x, int dtype, const void* weight, const void* bias, int w_dtype,
                                void* y, void* mean, void* rstd, int stat_dtype, int64_t M, int64_t N, double eps,
                                void* workspace, int64_t workspace_bytes, void* stream) {
  g_ln_ws = workspace;
  g_ln_ws_bytes = workspace_bytes;
  MI355_REQUIRE(M >= 0 && N > 0, "mi355_layer_norm: bad extents M=%lld N=%lld", (long long)M, (long long)N);
  if (M == 0) return MI355_OK;
  MI355_REQUIRE(x && y && mean && rstd, "mi355_layer_norm: NULL data pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool has_w = weight != nullptr || bias != nullptr;
  if (!has_w) w_dtype = dtype;
  switch (dtype) {
    case MI355_F32:
      if (w_dtype == MI355_F32) return run_ln_stat<float, float>(stat_dtype, dtype, x, weight, bias, y, mean, rstd, M, N, eps, st);
      break;
    case MI355_F16:
      if (w_dtype == MI355_F16) return run_ln_stat<f16_t, f16_t>(stat_dtype, dtype, x, weight, bias, y, mean, rstd, M, N, eps, st);
      if (w_dtype == MI355_F32) return run_ln_stat<f16_t, float>(stat_dtype, dtype, x, weight, bias, y, mean, rstd, M, N, eps, st);
      break;
    case MI355_F64:
      if (w_dtype == MI355_F64) return run_ln_stat<double, double>(stat_dtype, dtype, x, weight, bias, y, mean, rstd, M, N, eps, st);
      break;
    case MI355_BF16:
      if (w_dtype == MI355_BF16) return run_ln_stat<bf16_t, bf16_t>(stat_dtype, dtype, x, weight, bias, y, mean, rstd, M, N, eps, st);
      if (w_dtype == MI355_F32) return run_ln_stat<bf16_t, float>(stat_dtype, dtype, x, weight, bias, y, mean, rstd, M, N, eps, st);
      break;
    default: break;
  }
  return set_error(MI355_ERR_UNSUPPORTED, "mi355_layer_norm: no kernel for x %s with weight %s", dtype_name(dtype),
                   dtype_name(w_dtype));
}
