// _softmax / _log_softmax over the middle axis of a dense [outer, dim, inner] view, fp32 math
// (fp64 for f64 input, on the block and cols kernels only).
//
//   sub    inner == 1, rows of at most 32 vectors: 1 .. 32 lanes per row, several rows per wave;
//   tile   inner == 1, row fits the registers of 1, 2 or 4 cooperating waves: one HBM read,
//          max and sum by wave all-reduce (+ one LDS exchange between waves), one HBM write;
//   block  inner == 1, longer rows: 256 threads keep an online (max, sum) pair in one
//          pass, combine through LDS, then re-read the row (L2) to normalise;
//   cols   inner > 1: lanes along inner (128-bit accesses and the softmax axis split over 8
//          row groups when inner allows, else one thread per column), online pass then
//          normalise pass.
// exp(x - max) carries the special values: a +inf or NaN in the row, or a row of -inf,
// turns the whole row into NaN, as ATen does.
#include <type_traits>

#include "rowtile.h"

namespace mi355 {

constexpr int kSmBlock = kRowBlock;

// SHIFT: rows are not 16-byte aligned (odd row length); see RowTile::load_shifted.
constexpr int sm_tile_block(int w) { return w <= 4 ? kSmBlock : kWave * w; }  // rows over 8 / 16 waves: one row per block

template <typename T, typename O, int NV, bool VEC, int W, bool LOG, bool SHIFT, int VB>
__global__ __launch_bounds__(sm_tile_block(W)) void softmax_tile_kernel(const T* __restrict__ x, O* __restrict__ y,
                                                                       int64_t rows, int64_t n) {
  constexpr int BLOCK = sm_tile_block(W);
  using Tile = RowTile<T, NV, VEC, W, BLOCK, VB>;
  constexpr int V = Tile::V;
  __shared__ float red_max[BLOCK / kWave], red_sum[BLOCK / kWave];
  const int t = threadIdx.x % Tile::GROUP;
  int64_t row = (int64_t)blockIdx.x * Tile::ROWS_PER_BLOCK + threadIdx.x / Tile::GROUP;
  const bool active = row < rows;  // inactive groups still walk through the barriers
  if (!active) row = rows - 1;
  Tile tile;
  int a = 0;
  if constexpr (SHIFT) {
    a = row_misalignment<T, V>(x + row * n);
    tile.load_shifted(x + row * n, n, a, t, -INFINITY);
  } else {
    tile.load(x + row * n, n, t, -INFINITY);
  }
  float m = -INFINITY;
#pragma unroll
  for (int k = 0; k < NV; ++k)
#pragma unroll
    for (int j = 0; j < V; ++j) m = __builtin_fmaxf(m, tile.v[k][j]);  // v_max3_f32 takes two elements; a NaN is skipped here and poisons the sum below
  m = group_allreduce<W>(m, MaxOp(), red_max);
  float s = 0.f;
#pragma unroll
  for (int k = 0; k < NV; ++k)
#pragma unroll
    for (int j = 0; j < V; ++j) {
      const float d = tile.v[k][j] - m;
      const float e = __expf(d);
      tile.v[k][j] = LOG ? d : e;  // log-softmax keeps x - max and subtracts log(sum) at the end
      s += e;
    }
  // Padding lanes hold exp(-inf - m) = 0 unless m is -inf/NaN, where the row is NaN anyway.
  s = group_allreduce<W>(s, SumOp(), red_sum);
  if (!active) return;
  const float ls = __logf(s), inv = 1.f / s;
  auto fin = [ls, inv](float v, int64_t) { return LOG ? v - ls : v * inv; };
  if constexpr (SHIFT) tile.store_shifted(y + row * n, n, a, t, fin);
  else tile.store(y + row * n, n, t, fin);
}

// Many aligned rows that each fit one wave's registers (NV slabs of 64 lanes x one 128-bit
// vector: up to 4096 two-byte or 2048 four-byte elements), output of the input's dtype: a wave
// walks rows wave, wave + waves, ... and issues the next row's loads before it reduces the
// current one.  One wave per row: max and sum stay inside the wave, no LDS, no barrier.
template <typename T, int NV, bool LOG>
__global__ __launch_bounds__(kSmBlock) __attribute__((amdgpu_waves_per_eu(4, 8))) void softmax_stream_kernel(
    const T* __restrict__ x, T* __restrict__ y, int64_t rows, int64_t n) {
  constexpr int V = Vec<T>::N;
  const int lane = threadIdx.x % kWave;
  const int64_t waves = (int64_t)gridDim.x * (kSmBlock / kWave);
  int64_t row = (int64_t)blockIdx.x * (kSmBlock / kWave) + threadIdx.x / kWave;
  bool in[NV];
  VecN<T, V> nxt[NV];
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int64_t c = ((int64_t)k * kWave + lane) * V;
    in[k] = c < n;  // n % V == 0: a vector is inside the row or past it
    if (in[k] && row < rows) nxt[k] = ld_nt<T, V>(x + row * n + c);
  }
  for (; row < rows; row += waves) {
    float v[NV][V];
#pragma unroll
    for (int k = 0; k < NV; ++k)
#pragma unroll
      for (int j = 0; j < V; ++j) v[k][j] = in[k] ? static_cast<float>(nxt[k].v[j]) : -INFINITY;
    const int64_t ahead = row + waves;
    if (ahead < rows) {
#pragma unroll
      for (int k = 0; k < NV; ++k)
        if (in[k]) nxt[k] = ld_nt<T, V>(x + ahead * n + ((int64_t)k * kWave + lane) * V);
    }
    float m = -INFINITY;
#pragma unroll
    for (int k = 0; k < NV; ++k)
#pragma unroll
      for (int j = 0; j < V; ++j) m = __builtin_fmaxf(m, v[k][j]);  // a NaN is skipped here and poisons the sum below
    m = wave_allreduce(m, MaxOp());
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < NV; ++k)
#pragma unroll
      for (int j = 0; j < V; ++j) {
        const float d = v[k][j] - m;
        const float e = __expf(d);
        v[k][j] = LOG ? d : e;
        s += e;
      }
    s = wave_allreduce(s, SumOp());
    const float ls = __logf(s), inv = 1.f / s;
    T* out = y + row * n;
#pragma unroll
    for (int k = 0; k < NV; ++k)
      if (in[k]) {
        VecN<T, V> r;
#pragma unroll
        for (int j = 0; j < V; ++j) r.v[j] = static_cast<T>(LOG ? v[k][j] - ls : v[k][j] * inv);
        st_nt<T, V>(out + ((int64_t)k * kWave + lane) * V, r);
      }
  }
}

// Rows of at most 32 vectors: G = 1 .. 32 lanes per row (the smallest power of two whose lanes,
// at one 16-byte vector or V single elements each, cover the row), 64 / G rows per wave.  Max
// and sum meet by DPP inside the 16-lane rows (G = 32: one more exchange across them), so a
// [1M, 8] softmax runs 32 rows per wave instead of one.
template <typename T, typename O, bool LOG, int G, bool VEC>
__global__ __launch_bounds__(kSmBlock) void softmax_sub_kernel(const T* __restrict__ x, O* __restrict__ y,
                                                              int64_t rows, int64_t n) {
  constexpr int V = Vec<T>::N;
  static_assert(kSmBlock % G == 0, "groups must not straddle blocks");
  const int t = threadIdx.x % G;
  int64_t row = ((int64_t)blockIdx.x * kSmBlock + threadIdx.x) / G;
  const bool active = row < rows;  // the lanes of a group past the end still take part in the exchanges
  if (!active) row = rows - 1;
  const T* p = x + row * n;
  float v[V];
  if constexpr (VEC) {
    if ((int64_t)t * V < n) {  // n % V == 0: a vector is inside the row or past it
      const Vec<T> in = load_vec(p + t * V);
#pragma unroll
      for (int j = 0; j < V; ++j) v[j] = static_cast<float>(in.v[j]);
    } else {
#pragma unroll
      for (int j = 0; j < V; ++j) v[j] = -INFINITY;
    }
  } else {
#pragma unroll
    for (int j = 0; j < V; ++j) v[j] = t + G * j < n ? static_cast<float>(p[t + G * j]) : -INFINITY;
  }
  float m = -INFINITY;
#pragma unroll
  for (int j = 0; j < V; ++j) m = __builtin_fmaxf(m, v[j]);
  m = sub_allreduce<G>(m, MaxOp());
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < V; ++j) {
    const float d = v[j] - m;
    const float e = __expf(d);
    v[j] = LOG ? d : e;
    s += e;
  }
  s = sub_allreduce<G>(s, SumOp());
  if (!active) return;
  const float ls = __logf(s), inv = 1.f / s;
  O* q = y + row * n;
  if constexpr (VEC) {
    if ((int64_t)t * V < n) {
      VecN<O, V> r;
#pragma unroll
      for (int j = 0; j < V; ++j) r.v[j] = static_cast<O>(LOG ? v[j] - ls : v[j] * inv);
      st<O, V>(q + t * V, r);
    }
  } else {
#pragma unroll
    for (int j = 0; j < V; ++j)
      if (t + G * j < n) q[t + G * j] = static_cast<O>(LOG ? v[j] - ls : v[j] * inv);
  }
}

// Online (max, sum) pair in the accumulation type A (float; double for f64 input); see the
// file header for the special-value rules.
template <typename A> __device__ __forceinline__ A sm_exp(A x) {
  if constexpr (std::is_same<A, double>::value) return exp(x);
  else return __expf(x);
}
template <typename A> __device__ __forceinline__ A sm_log(A x) {
  if constexpr (std::is_same<A, double>::value) return log(x);
  else return __logf(x);
}
template <typename T> struct SmAcc { using type = float; };
template <> struct SmAcc<double> { using type = double; };

template <typename A> struct MS {
  A m, s;
};
template <typename A> __device__ __forceinline__ void ms_update(MS<A>& a, A x) {
  if (x > a.m) {
    a.s = a.s * sm_exp(a.m - x) + sm_exp(x - x);  // x - x is NaN for +inf
    a.m = x;
  } else if (x == -INFINITY) {
    // contributes exactly zero
  } else {
    a.s += sm_exp(x - a.m);  // NaN x lands here and poisons the sum
  }
}
template <typename A> __device__ __forceinline__ MS<A> ms_combine(MS<A> a, MS<A> b) {
  const A m = a.m > b.m ? a.m : b.m;
  const A sa = a.m == -INFINITY ? a.s * A(0) : a.s * sm_exp(a.m - m);
  const A sb = b.m == -INFINITY ? b.s * A(0) : b.s * sm_exp(b.m - m);
  return {m, sa + sb};
}
template <typename A> __device__ __forceinline__ MS<A> ms_wave_reduce(MS<A> a) {
#pragma unroll
  for (int k = 1; k < kWave; k <<= 1) {
    MS<A> o{__shfl_xor(a.m, k, kWave), __shfl_xor(a.s, k, kWave)};
    a = ms_combine(a, o);
  }
  return a;
}

// MODE 0: scalar accesses; 1: rows 16-byte aligned, vector accesses; 2: vector accesses over the
// aligned window around a misaligned row (as RowTile::load_shifted): interior vectors whole,
// the two end vectors element by element.
template <typename T, typename O, int MODE, bool LOG, int BLOCK>
__global__ __launch_bounds__(BLOCK) void softmax_block_kernel(const T* __restrict__ x, O* __restrict__ y,
                                                             int64_t n) {
  using A = typename SmAcc<T>::type;
  constexpr int V = Vec<T>::N;
  __shared__ MS<A> smem[BLOCK / kWave];
  const T* row = x + (int64_t)blockIdx.x * n;
  O* out = y + (int64_t)blockIdx.x * n;
  const int a = MODE == 2 ? row_misalignment(row) : 0;
  const T* win = row - a;
  O* owin = out - a;
  const int64_t total = n + a;  // window extent in elements
  MS<A> acc{-INFINITY, A(0)};
  if constexpr (MODE != 0) {
    for (int64_t w = (int64_t)threadIdx.x * V; w < total; w += (int64_t)BLOCK * V) {
      const Vec<T> t = load_vec(win + w);
      if (MODE == 1 || (w >= a && w + V <= total)) {
#pragma unroll
        for (int j = 0; j < V; ++j) ms_update(acc, static_cast<A>(t.v[j]));
      } else {
#pragma unroll
        for (int j = 0; j < V; ++j)
          if (w + j >= a && w + j < total) ms_update(acc, static_cast<A>(t.v[j]));
      }
    }
  } else {
    for (int64_t c = threadIdx.x; c < n; c += BLOCK) ms_update(acc, static_cast<A>(row[c]));
  }
  acc = ms_wave_reduce(acc);
  if (threadIdx.x % kWave == 0) smem[threadIdx.x / kWave] = acc;
  __syncthreads();
  acc = smem[0];
#pragma unroll
  for (int w = 1; w < BLOCK / kWave; ++w) acc = ms_combine(acc, smem[w]);
  const A m = acc.m, inv = A(1) / acc.s, ls = sm_log(acc.s);
  auto fin = [=](A v) { return LOG ? (v - m) - ls : sm_exp(v - m) * inv; };
  if constexpr (MODE != 0) {
    for (int64_t w = (int64_t)threadIdx.x * V; w < total; w += (int64_t)BLOCK * V) {
      const Vec<T> t = load_vec(win + w);
      if (MODE == 1 || (w >= a && w + V <= total)) {
        VecN<O, V> r;
#pragma unroll
        for (int j = 0; j < V; ++j) r.v[j] = static_cast<O>(fin(static_cast<A>(t.v[j])));
        st<O, V>(owin + w, r);
      } else {
#pragma unroll
        for (int j = 0; j < V; ++j)
          if (w + j >= a && w + j < total) owin[w + j] = static_cast<O>(fin(static_cast<A>(t.v[j])));
      }
    }
  } else {
    for (int64_t c = threadIdx.x; c < n; c += BLOCK)
      out[c] = static_cast<O>(fin(static_cast<A>(row[c])));
  }
}

// Few, very long rows (plan_row_split): blockIdx.x = chunk, blockIdx.y = row.  Pass 1 leaves the
// (max, sum) pair of every chunk in the workspace; pass 2 combines the pairs of its row and writes
// its chunk.  VEC: rows 16-byte aligned and n a multiple of the vector width.
template <typename T, bool VEC>
__global__ __launch_bounds__(kSmBlock) void softmax_split_partial_kernel(const T* __restrict__ x, unsigned char* __restrict__ ws,
                                                                        int64_t n, int64_t chunk) {
  using A = typename SmAcc<T>::type;
  constexpr int V = Vec<T>::N;
  __shared__ MS<A> smem[kSmBlock / kWave];
  const T* row = x + (int64_t)blockIdx.y * n;
  const int64_t c0 = (int64_t)blockIdx.x * chunk, c1 = c0 + chunk < n ? c0 + chunk : n;
  MS<A> acc{-INFINITY, A(0)};
  if constexpr (VEC) {
    for (int64_t c = c0 + (int64_t)threadIdx.x * V; c < c1; c += (int64_t)kSmBlock * V) {
      const Vec<T> t = load_vec(row + c);
#pragma unroll
      for (int j = 0; j < V; ++j) ms_update(acc, static_cast<A>(t.v[j]));
    }
  } else {
    for (int64_t c = c0 + threadIdx.x; c < c1; c += kSmBlock) ms_update(acc, static_cast<A>(row[c]));
  }
  acc = ms_wave_reduce(acc);
  if (threadIdx.x % kWave == 0) smem[threadIdx.x / kWave] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    acc = smem[0];
#pragma unroll
    for (int w = 1; w < kSmBlock / kWave; ++w) acc = ms_combine(acc, smem[w]);
    *reinterpret_cast<MS<A>*>(ws + ((int64_t)blockIdx.y * gridDim.x + blockIdx.x) * kRowPartialBytes) = acc;
  }
}

template <typename T, typename O, bool VEC, bool LOG>
__global__ __launch_bounds__(kSmBlock) void softmax_split_finish_kernel(const T* __restrict__ x, O* __restrict__ y,
                                                                       const unsigned char* __restrict__ ws, int64_t n,
                                                                       int64_t chunk) {
  using A = typename SmAcc<T>::type;
  constexpr int V = Vec<T>::N;
  __shared__ MS<A> smem[kSmBlock / kWave];
  MS<A> acc{-INFINITY, A(0)};
  for (int sp = threadIdx.x; sp < (int)gridDim.x; sp += kSmBlock)
    acc = ms_combine(acc, *reinterpret_cast<const MS<A>*>(ws + ((int64_t)blockIdx.y * gridDim.x + sp) * kRowPartialBytes));
  acc = ms_wave_reduce(acc);
  if (threadIdx.x % kWave == 0) smem[threadIdx.x / kWave] = acc;
  __syncthreads();
  acc = smem[0];
#pragma unroll
  for (int w = 1; w < kSmBlock / kWave; ++w) acc = ms_combine(acc, smem[w]);
  const A m = acc.m, inv = A(1) / acc.s, ls = sm_log(acc.s);
  auto fin = [=](A v) { return LOG ? (v - m) - ls : sm_exp(v - m) * inv; };
  const T* row = x + (int64_t)blockIdx.y * n;
  O* out = y + (int64_t)blockIdx.y * n;
  const int64_t c0 = (int64_t)blockIdx.x * chunk, c1 = c0 + chunk < n ? c0 + chunk : n;
  if constexpr (VEC) {
    for (int64_t c = c0 + (int64_t)threadIdx.x * V; c < c1; c += (int64_t)kSmBlock * V) {
      const Vec<T> t = load_vec(row + c);
      VecN<O, V> r;
#pragma unroll
      for (int j = 0; j < V; ++j) r.v[j] = static_cast<O>(fin(static_cast<A>(t.v[j])));
      st<O, V>(out + c, r);
    }
  } else {
    for (int64_t c = c0 + threadIdx.x; c < c1; c += kSmBlock) out[c] = static_cast<O>(fin(static_cast<A>(row[c])));
  }
}

template <typename T, typename O, bool LOG>
__global__ __launch_bounds__(kSmBlock) void softmax_cols_kernel(const T* __restrict__ x, O* __restrict__ y,
                                                               int64_t outer, int64_t n, int64_t inner) {
  using A = typename SmAcc<T>::type;
  const int64_t total = outer * inner;
  const int64_t stride = (int64_t)gridDim.x * kSmBlock;
  for (int64_t e = (int64_t)blockIdx.x * kSmBlock + threadIdx.x; e < total; e += stride) {
    const int64_t o = e / inner, c = e - o * inner;
    const T* p = x + o * n * inner + c;
    O* q = y + o * n * inner + c;
    MS<A> a{-INFINITY, A(0)};
    for (int64_t r = 0; r < n; ++r) ms_update(a, static_cast<A>(p[r * inner]));
    const A inv = A(1) / a.s, ls = sm_log(a.s);
    for (int64_t r = 0; r < n; ++r) {
      const A v = static_cast<A>(p[r * inner]);
      q[r * inner] = static_cast<O>(LOG ? (v - a.m) - ls : sm_exp(v - a.m) * inv);
    }
  }
}

// inner > 1: block = (64, R).  Lane tx owns V consecutive columns (one 128-bit access; V = 1:
// single elements, for an inner extent or alignment that allows no vectors), the R row groups
// split the softmax axis; their online (max, sum) pairs meet in LDS, then every thread
// normalises the rows it read (second read from L2).  V > 1 needs inner % V == 0 and 16-byte
// aligned operands.  grid = (ceil(inner / (64 V)), outer).
constexpr int kSmColsR = 8;
template <typename T, typename O, bool LOG, int V>
__global__ __launch_bounds__(kWave * kSmColsR) void softmax_cols_vec_kernel(const T* __restrict__ x, O* __restrict__ y,
                                                                          int64_t n, int64_t inner) {
  using A = typename SmAcc<T>::type;
  constexpr int R = kSmColsR;
  struct Vals { T v[V]; };
  auto load = [](const T* ptr) {
    if constexpr (V == 1) {
      return Vals{{*ptr}};
    } else {
      const Vec<T> t = load_vec(ptr);
      Vals r;
#pragma unroll
      for (int j = 0; j < V; ++j) r.v[j] = t.v[j];
      return r;
    }
  };
  __shared__ MS<A> smem[R][V][kWave];
  const int tx = threadIdx.x, ty = threadIdx.y;
  const int64_t col = ((int64_t)blockIdx.x * kWave + tx) * V;
  const bool live = col < inner;
  const T* p = x + (int64_t)blockIdx.y * n * inner + col;
  O* q = y + (int64_t)blockIdx.y * n * inner + col;
  MS<A> acc[V];
#pragma unroll
  for (int j = 0; j < V; ++j) acc[j] = {-INFINITY, A(0)};
  if (live) {
    for (int64_t r = ty; r < n; r += R) {
      const Vals t = load(p + r * inner);
#pragma unroll
      for (int j = 0; j < V; ++j) ms_update(acc[j], static_cast<A>(t.v[j]));
    }
  }
#pragma unroll
  for (int j = 0; j < V; ++j) smem[ty][j][tx] = acc[j];
  __syncthreads();
  if (!live) return;
  A m[V], inv[V], ls[V];
#pragma unroll
  for (int j = 0; j < V; ++j) {
    MS<A> a = smem[0][j][tx];
#pragma unroll
    for (int k = 1; k < R; ++k) a = ms_combine(a, smem[k][j][tx]);
    m[j] = a.m;
    inv[j] = A(1) / a.s;
    ls[j] = sm_log(a.s);
  }
  for (int64_t r = ty; r < n; r += R) {
    const Vals t = load(p + r * inner);
    VecN<O, V> o;
#pragma unroll
    for (int j = 0; j < V; ++j) {
      const A v = static_cast<A>(t.v[j]);
      o.v[j] = static_cast<O>(LOG ? (v - m[j]) - ls[j] : sm_exp(v - m[j]) * inv[j]);
    }
    st<O, V>(q + r * inner, o);
  }
}

template <typename T, typename O, bool LOG>
static int run_softmax(const void* xv, void* yv, int64_t outer, int64_t n, int64_t inner, void* ws, int64_t ws_bytes,
                       hipStream_t st) {
  const T* x = static_cast<const T*>(xv);
  O* y = static_cast<O*>(yv);
  constexpr int V = Vec<T>::N;
  if (inner > 1) {
    // vectors along inner unless that leaves most of the chip without a block (a softmax over the
    // first dim of a matrix): single columns per lane then give V times the blocks
    const bool enough_blocks = ((inner + kWave * V - 1) / (kWave * V)) * outer >= kNumCU;
    if (V > 1 && inner % V == 0 && n >= 4 * kSmColsR && aligned16(x) && enough_blocks &&
        reinterpret_cast<uintptr_t>(y) % (sizeof(O) * V) == 0 && outer < 65536) {
      const int64_t xb = (inner + kWave * V - 1) / (kWave * V);
      MI355_REQUIRE(xb < (int64_t(1) << 31), "mi355_softmax: inner extent too large");
      hipLaunchKernelGGL((softmax_cols_vec_kernel<T, O, LOG, V>), dim3((unsigned)xb, (unsigned)outer), dim3(kWave, kSmColsR), 0, st, x, y, n, inner);
      return check_launch("mi355_softmax(cols, vector)");
    }
    if (n >= 4 * kSmColsR && outer < 65536) {  // no vectors along inner (odd extent, misaligned): the same shape on single elements
      const int64_t xb = (inner + kWave - 1) / kWave;
      MI355_REQUIRE(xb < (int64_t(1) << 31), "mi355_softmax: inner extent too large");
      hipLaunchKernelGGL((softmax_cols_vec_kernel<T, O, LOG, 1>), dim3((unsigned)xb, (unsigned)outer), dim3(kWave, kSmColsR), 0, st, x, y, n, inner);
      return check_launch("mi355_softmax(cols, split rows)");
    }
    const int grid = grid_for(outer * inner, kSmBlock, kNumCU * 16);
    hipLaunchKernelGGL((softmax_cols_kernel<T, O, LOG>), dim3(grid), dim3(kSmBlock), 0, st, x, y, outer, n, inner);
    return check_launch("mi355_softmax(cols)");
  }
  const bool vec = n % V == 0 && aligned16(x) && (reinterpret_cast<uintptr_t>(y) % (sizeof(O) * V)) == 0;
  // Rows that start off a 16-byte boundary (odd n, offset views) still take the vector layout,
  // shifted per row, when input and output rows are misaligned by the same number of elements.
  const bool shift = !vec && V > 1 &&
                     (reinterpret_cast<uintptr_t>(x) / sizeof(T)) % V == (reinterpret_cast<uintptr_t>(y) / sizeof(O)) % V;
  // Register tiles.  When the output element is wider than the input element (half_to_float)
  // a lane takes 8 input bytes per access, so that its output is one 16-byte piece and every
  // store instruction of a wave covers whole lines.
  constexpr int VB = sizeof(O) > sizeof(T) ? 8 : 16;
  constexpr int TV = VB / sizeof(T);
  const bool tvec = TV == V ? vec : (n % TV == 0 && reinterpret_cast<uintptr_t>(x) % VB == 0 && aligned16(y));
  const bool tshift = TV == V ? shift
                              : (!tvec && (reinterpret_cast<uintptr_t>(x) / sizeof(T)) % TV ==
                                              (reinterpret_cast<uintptr_t>(y) / sizeof(O)) % TV);
  bool done = false;
  // few, very long rows: two launches over (row, chunk) when the caller brought the scratch for it
  {
    const RowSplit sp = plan_row_split(outer, n, sizeof(T));
    if (sp.nsplit > 1 && ws != nullptr && ws_bytes >= outer * sp.nsplit * kRowPartialBytes && reinterpret_cast<uintptr_t>(ws) % 8 == 0) {
      unsigned char* w = static_cast<unsigned char*>(ws);
      const dim3 grid((unsigned)sp.nsplit, (unsigned)outer);
      if (vec) {
        hipLaunchKernelGGL((softmax_split_partial_kernel<T, true>), grid, dim3(kSmBlock), 0, st, x, w, n, sp.chunk);
        hipLaunchKernelGGL((softmax_split_finish_kernel<T, O, true, LOG>), grid, dim3(kSmBlock), 0, st, x, y, w, n, sp.chunk);
      } else {
        hipLaunchKernelGGL((softmax_split_partial_kernel<T, false>), grid, dim3(kSmBlock), 0, st, x, w, n, sp.chunk);
        hipLaunchKernelGGL((softmax_split_finish_kernel<T, O, false, LOG>), grid, dim3(kSmBlock), 0, st, x, y, w, n, sp.chunk);
      }
      return check_launch("mi355_softmax(split rows)");
    }
  }
  if constexpr (!std::is_same<T, double>::value)
  if (n <= 32 * V && outer < (int64_t(1) << 31)) {
    // short rows: several per wave
    const int64_t need = (n + V - 1) / V;
#define MI355_SM_SUB(G_)                                                                                   \
  if (!done && need <= G_) {                                                                               \
    const unsigned nblk = (unsigned)((outer * G_ + kSmBlock - 1) / kSmBlock);                                \
    if (vec) hipLaunchKernelGGL((softmax_sub_kernel<T, O, LOG, G_, true>), dim3(nblk), dim3(kSmBlock), 0, st, x, y, outer, n); \
    else hipLaunchKernelGGL((softmax_sub_kernel<T, O, LOG, G_, false>), dim3(nblk), dim3(kSmBlock), 0, st, x, y, outer, n);    \
    done = true;                                                                                           \
  }
    MI355_SM_SUB(1) MI355_SM_SUB(2) MI355_SM_SUB(4) MI355_SM_SUB(8) MI355_SM_SUB(16) MI355_SM_SUB(32)
#undef MI355_SM_SUB
  }
  // Thousands of aligned rows of one wave's worth of registers each, same dtype out: the streaming kernel
  if constexpr (std::is_same<T, O>::value && !std::is_same<T, double>::value)
  if (!done && vec && n > 32 * V && n <= 8 * kWave * V && outer >= 4 * kNumCU) {
    auto go = [&](auto nv) {
      constexpr int NV = decltype(nv)::value;
      const void* kern = (const void*)softmax_stream_kernel<T, NV, LOG>;
      static thread_local int resident = 0;  // blocks per CU, per instantiation
      if (resident == 0) {
        int nb = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, kern, kSmBlock, 0) != hipSuccess || nb < 1) nb = 2;
        resident = nb;
      }
      const int64_t max_waves = (int64_t)kNumCU * resident * (kSmBlock / kWave);
      const int64_t per_wave = (outer + max_waves - 1) / max_waves;
      const int64_t nwaves = (outer + per_wave - 1) / per_wave;
      const unsigned nblk = (unsigned)((nwaves + kSmBlock / kWave - 1) / (kSmBlock / kWave));
      hipLaunchKernelGGL((softmax_stream_kernel<T, NV, LOG>), dim3(nblk), dim3(kSmBlock), 0, st, x, reinterpret_cast<T*>(y), outer, n);
    };
    if (n <= 4 * kWave * V) go(std::integral_constant<int, 4>());
    else go(std::integral_constant<int, 8>());
    done = true;
  }
  if constexpr (!std::is_same<T, double>::value)  // f64 rows take the block kernel (double accumulation)
  if (!done && outer < (int64_t(1) << 31)) {
    done = dispatch_row_tile<T>(tshift ? n + TV - 1 : n, tvec || tshift, [&](auto nv, auto w, auto v) {
      constexpr int NV = decltype(nv)::value, W = decltype(w)::value;
      constexpr bool VEC = decltype(v)::value;
      constexpr int block = sm_tile_block(W);
      constexpr int rpb = block / (kWave * W);
      const unsigned nblk = (unsigned)((outer + rpb - 1) / rpb);
      if constexpr (VEC) {
        if (tshift) {
          hipLaunchKernelGGL((softmax_tile_kernel<T, O, NV, true, W, LOG, true, VB>), dim3(nblk), dim3(block), 0, st, x, y, outer, n);
          return;
        }
      }
      hipLaunchKernelGGL((softmax_tile_kernel<T, O, NV, VEC, W, LOG, false, VB>), dim3(nblk), dim3(block), 0, st, x, y, outer, n);
    }, 16, std::integral_constant<int, VB>());
  }
  if (!done) {
    MI355_REQUIRE(outer < (int64_t(1) << 31), "mi355_softmax: too many rows (%lld)", (long long)outer);
    // Rows this long get a 1024-thread block each: more loads in flight per row.
    const bool big = n >= 32768;
#define MI355_SM_BLOCK(MODE_)                                                                                         \
  if (big) hipLaunchKernelGGL((softmax_block_kernel<T, O, MODE_, LOG, 1024>), dim3((unsigned)outer), dim3(1024), 0, st, x, y, n); \
  else hipLaunchKernelGGL((softmax_block_kernel<T, O, MODE_, LOG, kSmBlock>), dim3((unsigned)outer), dim3(kSmBlock), 0, st, x, y, n);
    if (vec) { MI355_SM_BLOCK(1) }
    else if (shift) { MI355_SM_BLOCK(2) }
    else { MI355_SM_BLOCK(0) }
#undef MI355_SM_BLOCK
  }
  return check_launch("mi355_softmax");
}

}  // namespace mi355

using namespace mi355;

// File-scope so that the dispatch below stays one line per dtype pair.
static thread_local void* g_sm_ws = nullptr;
static thread_local int64_t g_sm_ws_bytes = 0;

template <typename T, typename O>
static int run_softmax_any(int log_softmax, const void* x, void* y, int64_t outer, int64_t dim, int64_t inner, hipStream_t st) {
  return log_softmax ? run_softmax<T, O, true>(x, y, outer, dim, inner, g_sm_ws, g_sm_ws_bytes, st)
                     : run_softmax<T, O, false>(x, y, outer, dim, inner, g_sm_ws, g_sm_ws_bytes, st);
}

extern "C" int64_t mi355_row_workspace_bytes(int64_t rows, int64_t n, int dtype) {
  const int es = dtype_size(dtype);
  if (es == 0 || rows <= 0 || n <= 0) return 0;
  const RowSplit sp = plan_row_split(rows, n, es);
  return sp.nsplit > 1 ? rows * sp.nsplit * kRowPartialBytes : 0;
}

extern "C" int mi355_softmax(const void* x, int in_dtype, void* y, int out_dtype, int64_t outer, int64_t dim,
                             int64_t inner, int log_softmax, void* workspace, int64_t workspace_bytes, void* stream) {
  g_sm_ws = inner == 1 ? workspace : nullptr;
  g_sm_ws_bytes = workspace_bytes;
  MI355_REQUIRE(outer >= 0 && dim >= 0 && inner >= 0, "mi355_softmax: negative extent");
  if (outer == 0 || dim == 0 || inner == 0) return MI355_OK;
  MI355_REQUIRE(x != nullptr && y != nullptr, "mi355_softmax: NULL data pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (out_dtype == in_dtype) {
    switch (in_dtype) {
      case MI355_F32: return run_softmax_any<float, float>(log_softmax, x, y, outer, dim, inner, st);
      case MI355_F16: return run_softmax_any<f16_t, f16_t>(log_softmax, x, y, outer, dim, inner, st);
      case MI355_BF16: return run_softmax_any<bf16_t, bf16_t>(log_softmax, x, y, outer, dim, inner, st);
      case MI355_F64: return run_softmax_any<double, double>(log_softmax, x, y, outer, dim, inner, st);
      default: break;
    }
  } else if (out_dtype == MI355_F32) {  // half_to_float
    switch (in_dtype) {
      case MI355_F16: return run_softmax_any<f16_t, float>(log_softmax, x, y, outer, dim, inner, st);
      case MI355_BF16: return run_softmax_any<bf16_t, float>(log_softmax, x, y, outer, dim, inner, st);
      default: break;
    }
  }
  return set_error(MI355_ERR_UNSUPPORTED, "mi355_softmax: no kernel for %s -> %s", dtype_name(in_dtype),
                   dtype_name(out_dtype));
}
