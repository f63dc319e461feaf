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
// gamma / beta are staged once per block in LDS (2 n elements of dynamic shared memory, as floats
// for bf16).  Same statistics as the tile kernel (mean, then the centred second moment of the
// same values).
// Both rows stay in the registers as loaded (NV 16-byte vectors each) and are widened to fp32
// anew in each pass: 2 x 4 NV registers of row data instead of 4 NV + NV V floats, which keeps a
// 4096-element row with gamma and beta under 96 registers - five waves per SIMD and nothing
// spilled to scratch memory (the fp32 register tile spilled two to five registers per lane, 3 %
// extra HBM traffic).  The row sum takes v_dot2_f32_{bf16,f16} against (1, 1); FULL (the row
// fills all NV slabs) drops the per-slab masks.
typedef uint32_t ln_raw16 __attribute__((ext_vector_type(4)));
typedef __bf16 ln_bf2 __attribute__((ext_vector_type(2)));
typedef _Float16 ln_h2 __attribute__((ext_vector_type(2)));

// Sum of the V elements of one 16-byte vector, accumulated in fp32 onto `acc`.  Two-byte types take
// v_dot2_f32_{bf16,f16} against (1, 1): two elements per instruction, no widening first.
template <typename T> __device__ __forceinline__ float ln_vec_sum(ln_raw16 r, float acc) {
  if constexpr (std::is_same<T, bf16_t>::value) {
    const ln_bf2 one = {(__bf16)1.0f, (__bf16)1.0f};
#pragma unroll
    for (int i = 0; i < 4; ++i) { const uint32_t wd = r[i]; acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(ln_bf2, wd), one, acc, false); }
  } else if constexpr (std::is_same<T, f16_t>::value) {
    const ln_h2 one = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
    for (int i = 0; i < 4; ++i) { const uint32_t wd = r[i]; acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(ln_h2, wd), one, acc, false); }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) { const uint32_t wd = r[i]; acc += __builtin_bit_cast(float, wd); }
  }
  return acc;
}
// The V elements of a 16-byte vector as floats.
template <typename T, int V> __device__ __forceinline__ void ln_widen(ln_raw16 r, float (&f)[V]) {
  if constexpr (std::is_same<T, bf16_t>::value) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __builtin_bit_cast(float, r[i] << 16);
      f[2 * i + 1] = __builtin_bit_cast(float, r[i] & 0xffff0000u);
    }
  } else {
    const VecN<T, V> xv = __builtin_bit_cast(VecN<T, V>, r);
#pragma unroll
    for (int j = 0; j < V; ++j) f[j] = static_cast<float>(xv.v[j]);
  }
}

// Half h (0, 1) of a 16-byte vector as H = V / 2 floats.
template <typename T, int H> __device__ __forceinline__ void ln_widen_half(ln_raw16 r, int h, float (&f)[H]) {
  const uint32_t w0 = h ? r[2] : r[0], w1 = h ? r[3] : r[1];
  if constexpr (std::is_same<T, bf16_t>::value) {
    f[0] = __builtin_bit_cast(float, w0 << 16);
    f[1] = __builtin_bit_cast(float, w0 & 0xffff0000u);
    f[2] = __builtin_bit_cast(float, w1 << 16);
    f[3] = __builtin_bit_cast(float, w1 & 0xffff0000u);
  } else if constexpr (std::is_same<T, f16_t>::value) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    const h2 a = __builtin_bit_cast(h2, w0), b = __builtin_bit_cast(h2, w1);
    f[0] = static_cast<float>(a[0]); f[1] = static_cast<float>(a[1]);
    f[2] = static_cast<float>(b[0]); f[3] = static_cast<float>(b[1]);
  } else {
    f[0] = __builtin_bit_cast(float, w0);
    f[1] = __builtin_bit_cast(float, w1);
  }
}

// gamma / beta in LDS (widened to P when P is wider than T), in two planes: plane h holds half h (H = V / 2
// elements) of every V-element vector, vector after vector.  A wave's read of one half of its lanes' vectors
// is then one contiguous stretch of LDS - with the vectors stored whole, the halves sit 2 H elements apart
// and every such read met a two-way bank conflict (SQ_LDS_BANK_CONFLICT: 48 % of the LDS cycles).
template <typename T, typename P, int V> __device__ __forceinline__ void ln_stage(P* planes, int64_t half_elems, int64_t c, const T* src) {
  constexpr int H = V / 2;
  const VecN<T, V> v = ld<T, V>(src + c);
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    VecN<P, H> o;
#pragma unroll
    for (int j = 0; j < H; ++j) o.v[j] = static_cast<P>(v.v[h * H + j]);
    st<P, H>(planes + h * half_elems + (c / V) * H, o);
  }
}
// H consecutive staged parameters as floats (one LDS read of H * sizeof(P) bytes).
template <typename P, int H> __device__ __forceinline__ void ln_params_half(const P* p, float (&f)[H]) {
  const VecN<P, H> v = ld<P, H>(p);
#pragma unroll
  for (int j = 0; j < H; ++j) f[j] = static_cast<float>(v.v[j]);
}

template <typename T, typename S, int NV, bool HW, bool HB, bool FULL>
__global__ __launch_bounds__(kLnBlock) void layernorm_stream_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                                   const T* __restrict__ b, T* __restrict__ y,
                                                                   S* __restrict__ mean_out, S* __restrict__ rstd_out,
                                                                   int64_t rows, int64_t n, float eps) {
  constexpr int V = Vec<T>::N;
  static_assert(sizeof(T) * V == 16, "one 16-byte vector per lane and slab");
  extern __shared__ __attribute__((aligned(32))) unsigned char ln_smem[];  // gamma, then beta: 2 n elements
  // bf16 has no mixed-precision FMA (f16 has v_fma_mix_f32): its gamma / beta are widened once, when
  // they are staged, instead of once per row and element.
  using P = typename std::conditional<std::is_same<T, bf16_t>::value, float, T>::type;
  P* gl = reinterpret_cast<P*>(ln_smem);
  P* bl = gl + n;
  const int lane = threadIdx.x % kWave;
  const int64_t waves = (int64_t)gridDim.x * (kLnBlock / kWave);
  int64_t row = (int64_t)blockIdx.x * (kLnBlock / kWave) + __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  bool in[NV];
  ln_raw16 ra[NV], rb[NV];
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int64_t c = ((int64_t)k * kWave + lane) * V;
    in[k] = FULL || c < n;  // n % V == 0: a vector is inside the row or past it
    ra[k] = rb[k] = ln_raw16{0u, 0u, 0u, 0u};  // slabs past the row stay zeros (+0 in every float type)
    if (in[k] && row < rows) ra[k] = __builtin_nontemporal_load(reinterpret_cast<const ln_raw16*>(x + row * n + c));
  }
  if constexpr (HW || HB) {
    for (int64_t c = (int64_t)threadIdx.x * V; c < n; c += (int64_t)kLnBlock * V) {
      if constexpr (HW) ln_stage<T, P, V>(gl, n / 2, c, w);
      if constexpr (HB) ln_stage<T, P, V>(bl, n / 2, c, b);
    }
    __syncthreads();
  }
  const float inv_n = 1.f / (float)n;
  // One row: request the row after it into `nxt`, then three passes over `cur` as loaded.
  auto one_row = [&](ln_raw16 (&cur)[NV], ln_raw16 (&nxt)[NV]) {
    const int64_t ahead = row + waves;
    if (ahead < rows) {
#pragma unroll
      for (int k = 0; k < NV; ++k)
        if (in[k])
          nxt[k] = __builtin_nontemporal_load(reinterpret_cast<const ln_raw16*>(x + ahead * n + ((int64_t)k * kWave + lane) * V));
    }
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < NV; ++k) s = ln_vec_sum<T>(cur[k], s);
    const float mean = wave_allreduce(s, SumOp()) * inv_n;
#pragma unroll
    for (int k = 0; k < NV; ++k) asm volatile("" : "+v"(cur[k]));
    float q = 0.f;
#pragma unroll
    for (int k = 0; k < NV; ++k)
      if (in[k]) {
        float f[V];
        ln_widen<T, V>(cur[k], f);
#pragma unroll
        for (int j = 0; j < V; ++j) {
          const float d = f[j] - mean;
          q += d * d;
        }
      }
    const float rstd = rsqrtf(wave_allreduce(q, SumOp()) * inv_n + eps);
#pragma unroll
    for (int k = 0; k < NV; ++k) asm volatile("" : "+v"(cur[k]));
    if (lane == 0) {
      mean_out[row] = static_cast<S>(mean);
      rstd_out[row] = static_cast<S>(rstd);
    }
    const float shift = -mean * rstd;
    T* out = y + row * n;
#pragma unroll
    for (int k = 0; k < NV; ++k)
      if (in[k]) {
        const int64_t c = ((int64_t)k * kWave + lane) * V;
        // half a vector at a time: 4 + 4 + 4 widened values live instead of 3 V
        VecN<T, V> r;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          constexpr int H = V / 2;
          float f[H], g[H], be[H];
          ln_widen_half<T, H>(cur[k], h, f);
          if constexpr (HW) ln_params_half<P, H>(gl + h * (n / 2) + (c / V) * H, g);
          if constexpr (HB) ln_params_half<P, H>(bl + h * (n / 2) + (c / V) * H, be);
#pragma unroll
          for (int j = 0; j < H; ++j) {
            float t = __builtin_fmaf(f[j], rstd, shift);  // (x - mean) * rstd
            if constexpr (HW && HB) t = __builtin_fmaf(t, g[j], be[j]);
            else if constexpr (HW) t *= g[j];
            else if constexpr (HB) t += be[j];
            r.v[h * H + j] = static_cast<T>(t);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
        st_nt<T, V>(out + c, r);
        __builtin_amdgcn_sched_barrier(0);
      }
  };
  // Two rows per trip, the two register sets trading places, so no row is copied between them.
  while (row < rows) {
    one_row(ra, rb);
    row += waves;
    if (row >= rows) break;
    one_row(rb, ra);
    row += waves;
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
                                                                  int64_t n, double eps) {
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
  else rstd = rsqrtf(a.m2 / (float)n + (float)eps);
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
                                                                         int64_t chunk, double eps) {
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
  else rstd = rsqrtf(a.m2 / (float)n + (float)eps);
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
        hipLaunchKernelGGL((layernorm_split_finish_kernel<T, W, S, true>), grid, dim3(kLnBlock), 0, st, x, w, b, y, mean, rstd, wsp, N, sp.chunk, eps);
      } else {
        hipLaunchKernelGGL((layernorm_split_partial_kernel<T, false>), grid, dim3(kLnBlock), 0, st, x, wsp, N, sp.chunk);
        hipLaunchKernelGGL((layernorm_split_finish_kernel<T, W, S, false>), grid, dim3(kLnBlock), 0, st, x, w, b, y, mean, rstd, wsp, N, sp.chunk, eps);
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
      auto go = [&](auto hw, auto hb, auto full) {
        constexpr bool HW_ = decltype(hw)::value, HB_ = decltype(hb)::value, FULL_ = decltype(full)::value;
        const void* kern = (const void*)layernorm_stream_kernel<T, S, NV, HW_, HB_, FULL_>;
        // gamma and beta in LDS: as floats for bf16 (widened once at staging)
        const size_t smem = has_params ? 2 * (size_t)N * (std::is_same<T, bf16_t>::value ? sizeof(float) : sizeof(T)) : 0;
        static thread_local int resident = 0;  // blocks per CU, per instantiation
        static thread_local size_t resident_smem = 0;
        if (resident == 0 || resident_smem != smem) {
          int nb = 0;
          if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, kern, kLnBlock, smem) != hipSuccess || nb < 1) nb = 2;
          resident = nb;
          resident_smem = smem;
        }
        const int64_t max_waves = (int64_t)kNumCU * resident * (kLnBlock / kWave);
        const int64_t per_wave = (M + max_waves - 1) / max_waves;
        const int64_t nwaves = (M + per_wave - 1) / per_wave;
        const unsigned nblk = (unsigned)((nwaves + kLnBlock / kWave - 1) / (kLnBlock / kWave));
        hipLaunchKernelGGL((layernorm_stream_kernel<T, S, NV, HW_, HB_, FULL_>), dim3(nblk), dim3(kLnBlock), smem, st, x,
                           reinterpret_cast<const T*>(w), reinterpret_cast<const T*>(b), y, mean, rstd, M, N, (float)eps);
      };
      using std::true_type;
      using std::false_type;
      // Rows that fill every slab run without the per-slab masks (two-byte types; for fp32 the masked
      // form measured 2 % faster, 23.1 against 23.5 us on [8192, 2048]).
      auto pick = [&](auto full) {
        if (w && b) go(true_type(), true_type(), full);
        else if (w) go(true_type(), false_type(), full);
        else if (b) go(false_type(), true_type(), full);
        else go(false_type(), false_type(), full);
      };
      if (sizeof(T) == 2 && N == (int64_t)NV * kWave * V) pick(true_type());
      else pick(false_type());
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
    if (vec) hipLaunchKernelGGL((layernorm_block_kernel<T, W, S, true>), dim3((unsigned)M), dim3(kLnBlock), 0, st, x, w, b, y, mean, rstd, N, eps);
    else hipLaunchKernelGGL((layernorm_block_kernel<T, W, S, false>), dim3((unsigned)M), dim3(kLnBlock), 0, st, x, w, b, y, mean, rstd, N, eps);
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
