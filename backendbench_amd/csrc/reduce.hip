// sum / mean / amax / argmax over the middle axis of a dense [outer, red, inner] view.
//
// Kernel shapes (picked by plan_reduce):
//   rows_wave    inner == 1, many short rows: one wave64 per row, 128-bit loads, DPP +
//                bpermute all-reduce, no LDS, no barrier;
//   rows_block   inner == 1, long or few rows: one 256-thread block per (row, split),
//                wave reduce then LDS combine across the four waves;
//   rows_thread  inner == 1, red <= 32: one thread per row;
//   rows_sub     inner == 1, many rows of at most 64 vectors (pooling over a 7x7 map, a 197-wide
//                attention row): sixteen lanes per row, four rows per wave, DPP reduce inside the
//                16-lane row;
//   cols         inner > 1: 64 lanes along inner (coalesced, one 128-bit load each when inner
//                allows) x 4 along red, LDS combine;
//   final        second pass over per-split partial states when a launch was split
//                to fill the chip (few rows, long reduction).
#include "common.h"

#include <mutex>

#include <type_traits>

namespace mi355 {

// ---------------------------------------------------------------- reduction ops
template <typename A> struct SumR {
  using acc_t = A;
  struct State { A s; };
  static __device__ __forceinline__ State init() { return {A(0)}; }
  static __device__ __forceinline__ void acc(State& st, A v, int64_t) { st.s += v; }
  static __device__ __forceinline__ State combine(State a, State b) { return {a.s + b.s}; }
  static __device__ __forceinline__ State shfl_xor(State a, int m) { return {__shfl_xor(a.s, m, kWave)}; }
};
template <typename A> struct AmaxR {
  using acc_t = A;
  struct State { A s; };
  static __device__ __forceinline__ State init() {
    if constexpr (IsFloat<A>::value) return {-INFINITY};
    else if constexpr (sizeof(A) == 8) return {INT64_MIN};
    else return {INT32_MIN};
  }
  static __device__ __forceinline__ void acc(State& st, A v, int64_t) { st.s = MaxNanOp()(st.s, v); }
  static __device__ __forceinline__ State combine(State a, State b) { return {MaxNanOp()(a.s, b.s)}; }
  static __device__ __forceinline__ State shfl_xor(State a, int m) { return {__shfl_xor(a.s, m, kWave)}; }
};
// (value, index) with ATen's order: NaN is the maximum, the lower index wins ties.
template <typename A> struct ArgmaxR {
  using acc_t = A;
  struct State { A v; int64_t i; };
  static __device__ __forceinline__ State init() { return {AmaxR<A>::init().s, INT64_MAX}; }
  static __device__ __forceinline__ bool better(A v, int64_t i, A bv, int64_t bi) {
    if constexpr (IsFloat<A>::value) {
      const bool vn = v != v, bn = bv != bv;
      if (vn || bn) return vn && (!bn || i < bi);
    }
    return v > bv || (v == bv && i < bi);
  }
  // Every kernel feeds a lane its elements in increasing index order, so an element equal to the
  // held one never replaces it and the index needs no comparison here.  A lane (or a whole row)
  // whose elements all equal the initial value keeps i = INT64_MAX; write_final turns that into
  // index 0, the first of the all-equal row.
  static __device__ __forceinline__ void acc(State& st, A v, int64_t i) {
    bool take;
    if constexpr (IsFloat<A>::value) take = (v != v) ? (st.v == st.v) : (v > st.v);  // v > NaN is false: a held NaN stays
    else take = v > st.v;
    if (take) { st.v = v; st.i = i; }
  }
  static __device__ __forceinline__ State combine(State a, State b) {
    return better(b.v, b.i, a.v, a.i) ? b : a;
  }
  static __device__ __forceinline__ State shfl_xor(State a, int m) {
    return {__shfl_xor(a.v, m, kWave), (int64_t)__shfl_xor((long long)a.i, m, kWave)};
  }
};

template <typename R> __device__ __forceinline__ typename R::State wave_reduce_state(typename R::State s) {
#pragma unroll
  for (int m = 1; m < kWave; m <<= 1) s = R::combine(s, R::shfl_xor(s, m));
  return s;
}
// Scalar states take the DPP path.
template <typename A> __device__ __forceinline__ typename SumR<A>::State wave_reduce(typename SumR<A>::State s, SumR<A>*) {
  return {wave_allreduce(s.s, SumOp())};
}
template <typename A> __device__ __forceinline__ typename AmaxR<A>::State wave_reduce(typename AmaxR<A>::State s, AmaxR<A>*) {
  return {wave_allreduce(s.s, MaxNanOp())};
}
// (value, index) pairs: the four steps inside a 16-lane row move both halves by DPP, only the
// two steps across rows go through ds_bpermute.
template <typename A, int CTRL> __device__ __forceinline__ typename ArgmaxR<A>::State argmax_dpp_step(typename ArgmaxR<A>::State s) {
  const typename ArgmaxR<A>::State o{dpp<CTRL>(s.v), dpp<CTRL>(s.i)};
  return ArgmaxR<A>::combine(s, o);
}
template <typename A> __device__ __forceinline__ typename ArgmaxR<A>::State argmax_row16(typename ArgmaxR<A>::State s) {
  s = argmax_dpp_step<A, 0xB1>(s);
  s = argmax_dpp_step<A, 0x4E>(s);
  s = argmax_dpp_step<A, 0x124>(s);
  s = argmax_dpp_step<A, 0x128>(s);
  return s;
}
template <typename A> __device__ __forceinline__ typename ArgmaxR<A>::State wave_reduce(typename ArgmaxR<A>::State s, ArgmaxR<A>*) {
  s = argmax_row16<A>(s);
  s = ArgmaxR<A>::combine(s, ArgmaxR<A>::shfl_xor(s, 16));
  s = ArgmaxR<A>::combine(s, ArgmaxR<A>::shfl_xor(s, 32));
  return s;
}

// Reduce over the 16 lanes of a DPP row (lanes 16 g .. 16 g + 15): result in all of them.
template <typename T, typename Op> __device__ __forceinline__ T row16_allreduce(T v, Op op) {
  v = op(v, dpp<0xB1>(v));   // quad_perm [1,0,3,2]
  v = op(v, dpp<0x4E>(v));   // quad_perm [2,3,0,1]
  v = op(v, dpp<0x124>(v));  // row_ror:4
  v = op(v, dpp<0x128>(v));  // row_ror:8
  return v;
}
template <typename A> __device__ __forceinline__ typename SumR<A>::State row16_reduce(typename SumR<A>::State s, SumR<A>*) {
  return {row16_allreduce(s.s, SumOp())};
}
template <typename A> __device__ __forceinline__ typename AmaxR<A>::State row16_reduce(typename AmaxR<A>::State s, AmaxR<A>*) {
  return {row16_allreduce(s.s, MaxNanOp())};
}
template <typename A> __device__ __forceinline__ typename ArgmaxR<A>::State row16_reduce(typename ArgmaxR<A>::State s, ArgmaxR<A>*) {
  return argmax_row16<A>(s);
}

// Block reduce of a State (blockDim.x = 256): result valid in thread 0.
template <typename R>
__device__ __forceinline__ typename R::State block_reduce_state(typename R::State s, typename R::State* smem) {
  s = wave_reduce(s, (R*)nullptr);
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int nwaves = blockDim.x / kWave;
  if (lane == 0) smem[wave] = s;
  __syncthreads();
  if (threadIdx.x == 0)
    for (int w = 1; w < nwaves; ++w) s = R::combine(s, smem[w]);
  return s;
}

// How a final value leaves a kernel: SUM/AMAX write s, MEAN divides, ARGMAX writes i.
enum { FIN_VALUE = 0, FIN_MEAN = 1, FIN_INDEX = 2 };
template <typename R, typename O, int FIN>
__device__ __forceinline__ void write_final(O* out, int64_t at, const typename R::State& st, double divisor) {
  using A = typename R::acc_t;
  if constexpr (FIN == FIN_INDEX) {
    const int64_t i = ((const typename ArgmaxR<A>::State&)st).i;
    out[at] = (O)(i == INT64_MAX ? 0 : i);  // nothing beat the initial value: every element equals it
  } else {
    A v = *reinterpret_cast<const A*>(&st);
    if constexpr (FIN == FIN_MEAN) v = v / (A)divisor;
    out[at] = static_cast<O>(v);
  }
}

// ---------------------------------------------------------------- kernels
constexpr int kRedBlock = 256;

// Accumulate row[lo .. hi) striding by `nthr` lanes starting at `tid`.
//   MODE 0  scalar accesses;
//   MODE 1  row 16-byte aligned, lo and hi multiples of V (the planner guarantees it): vectors;
//   MODE 2  misaligned row (odd row length, offset view): vectors over the aligned window that
//           starts `a` elements before the row; [lo, hi) are window positions (multiples of V
//           except the last hi), elements outside the row are skipped.  The window may reach up
//           to 15 bytes outside the row, inside 16-byte pieces that also hold row bytes.
template <typename T, typename R, int MODE>
__device__ __forceinline__ void accumulate_span(typename R::State& st, const T* row, int64_t lo, int64_t hi,
                                                int tid, int nthr, int a = 0, int64_t red = 0) {
  using A = typename R::acc_t;
  if constexpr (MODE != 0) {
    constexpr int V = Vec<T>::N;
    const T* win = row - a;
    const int64_t total = red + a;  // MODE 2 only
    auto take = [&](const Vec<T>& v, int64_t w) {
      if (MODE == 1 || (w >= a && w + V <= total)) {
#pragma unroll
        for (int j = 0; j < V; ++j) R::acc(st, (A)v.v[j], w + j - a);
      } else {
#pragma unroll
        for (int j = 0; j < V; ++j)
          if (w + j >= a && w + j < total) R::acc(st, (A)v.v[j], w + j - a);
      }
    };
    int64_t i = lo + (int64_t)tid * V;
    const int64_t step = (int64_t)nthr * V;
    if (hi - lo <= 4 * step) {
      // A short span (at most four vectors per lane) is one batch under per-lane predicates: one
      // memory latency for the whole row, whatever its length.
      if (i < hi) {
        const bool k1 = i + step < hi, k2 = i + 2 * step < hi, k3 = i + 3 * step < hi;
        Vec<T> v0 = load_vec_nt(win + i), v1, v2, v3;
        if (k1) v1 = load_vec_nt(win + i + step);
        if (k2) v2 = load_vec_nt(win + i + 2 * step);
        if (k3) v3 = load_vec_nt(win + i + 3 * step);
        take(v0, i);
        if (k1) take(v1, i + step);
        if (k2) take(v2, i + 2 * step);
        if (k3) take(v3, i + 3 * step);
      }
      return;
    }
    // Batches of four vectors per lane, all loads of a batch issued before the first is used.
    for (; i + 3 * step < hi; i += 4 * step) {
      Vec<T> v0 = load_vec_nt(win + i), v1 = load_vec_nt(win + i + step), v2 = load_vec_nt(win + i + 2 * step),
             v3 = load_vec_nt(win + i + 3 * step);
      take(v0, i);
      take(v1, i + step);
      take(v2, i + 2 * step);
      take(v3, i + 3 * step);
    }
    // The last batch of a row may be partial (per-lane predicates); its loads go out together as
    // well, so a short row costs one memory latency, not one per leftover vector.
    if (i < hi) {
      const bool k1 = i + step < hi, k2 = i + 2 * step < hi;
      Vec<T> v0 = load_vec_nt(win + i), v1, v2;
      if (k1) v1 = load_vec_nt(win + i + step);
      if (k2) v2 = load_vec_nt(win + i + 2 * step);
      take(v0, i);
      if (k1) take(v1, i + step);
      if (k2) take(v2, i + 2 * step);
    }
  } else {
    for (int64_t i = lo + tid; i < hi; i += nthr) R::acc(st, (A)row[i], i);
  }
}

template <typename T> __device__ __forceinline__ int reduce_row_misalignment(const T* p) {
  return (int)((reinterpret_cast<uintptr_t>(p) / sizeof(T)) % Vec<T>::N);
}

template <typename T, typename O, typename R, int FIN, int MODE>
__global__ __launch_bounds__(kRedBlock) void rows_wave_kernel(const T* __restrict__ x, O* __restrict__ out,
                                                             int64_t outer, int64_t red, double divisor) {
  const int lane = threadIdx.x % kWave;
  const int64_t wave0 = (int64_t)blockIdx.x * (kRedBlock / kWave) + threadIdx.x / kWave;
  const int64_t nwaves = (int64_t)gridDim.x * (kRedBlock / kWave);
  for (int64_t row = wave0; row < outer; row += nwaves) {
    typename R::State st = R::init();
    const T* r = x + row * red;
    const int a = MODE == 2 ? reduce_row_misalignment(r) : 0;
    accumulate_span<T, R, MODE>(st, r, 0, red + a, lane, kWave, a, red);
    st = wave_reduce(st, (R*)nullptr);
    if (lane == 0) write_final<R, O, FIN>(out, row, st, divisor);
  }
}

// grid = (nsplit, outer).  PARTIAL: writes State to ws[row * nsplit + split].
template <typename T, typename O, typename R, int FIN, int MODE, bool PARTIAL>
__global__ __launch_bounds__(kRedBlock) void rows_block_kernel(const T* __restrict__ x, O* __restrict__ out,
                                                              typename R::State* __restrict__ ws, int64_t red,
                                                              int64_t chunk, double divisor) {
  __shared__ typename R::State smem[kRedBlock / kWave];
  const int64_t row = blockIdx.y;
  const T* r = x + row * red;
  const int a = MODE == 2 ? reduce_row_misalignment(r) : 0;
  const int64_t total = red + a;  // window extent (= red unless MODE 2)
  const int64_t lo = (int64_t)blockIdx.x * chunk;
  // the last split also takes the few window positions the misalignment adds
  const int64_t hi = (blockIdx.x + 1 == gridDim.x || lo + chunk > total) ? total : lo + chunk;
  typename R::State st = R::init();
  if (lo < hi) accumulate_span<T, R, MODE>(st, r, lo, hi, threadIdx.x, kRedBlock, a, red);
  st = block_reduce_state<R>(st, smem);
  if (threadIdx.x == 0) {
    if constexpr (PARTIAL) ws[row * gridDim.x + blockIdx.x] = st;
    else write_final<R, O, FIN>(out, row, st, divisor);
  }
}

// Sixteen lanes per row, four rows per wave (one contiguous span of memory); MODE as in
// accumulate_span: vectors for aligned rows, the aligned window around a misaligned row, or
// single elements.  All lanes of a wave stay in the loop (the DPP reduce is wave-wide); rows past
// the end accumulate nothing and write nothing.
template <typename T, typename O, typename R, int FIN, int MODE>
__global__ __launch_bounds__(kRedBlock) void rows_sub_kernel(const T* __restrict__ x, O* __restrict__ out,
                                                            int64_t outer, int64_t red, double divisor) {
  const int j = threadIdx.x & 15;
  const int64_t group0 = ((int64_t)blockIdx.x * kRedBlock + threadIdx.x) >> 4;
  const int64_t ngroups = (int64_t)gridDim.x * (kRedBlock / 16);
  const int64_t rounds = (outer + ngroups - 1) / ngroups;
  for (int64_t r = 0; r < rounds; ++r) {
    const int64_t row = group0 + r * ngroups;
    typename R::State st = R::init();
    if (row < outer) {
      const T* p = x + row * red;
      const int a = MODE == 2 ? reduce_row_misalignment(p) : 0;
      accumulate_span<T, R, MODE>(st, p, 0, red + a, j, 16, a, red);
    }
    st = row16_reduce(st, (R*)nullptr);
    if (j == 0 && row < outer) write_final<R, O, FIN>(out, row, st, divisor);
  }
}

template <typename T, typename O, typename R, int FIN>
__global__ __launch_bounds__(kRedBlock) void rows_thread_kernel(const T* __restrict__ x, O* __restrict__ out,
                                                               int64_t outer, int64_t red, double divisor) {
  using A = typename R::acc_t;
  const int64_t stride = (int64_t)gridDim.x * kRedBlock;
  for (int64_t row = (int64_t)blockIdx.x * kRedBlock + threadIdx.x; row < outer; row += stride) {
    typename R::State st = R::init();
    const T* p = x + row * red;
    for (int64_t i = 0; i < red; ++i) R::acc(st, (A)p[i], i);
    write_final<R, O, FIN>(out, row, st, divisor);
  }
}

// block = (64, 4); grid = (ceil(inner/64), nsplit, outer).
template <typename T, typename O, typename R, int FIN, bool PARTIAL>
__global__ __launch_bounds__(kRedBlock) void cols_kernel(const T* __restrict__ x, O* __restrict__ out,
                                                        typename R::State* __restrict__ ws, int64_t red,
                                                        int64_t inner, int64_t chunk, double divisor) {
  using A = typename R::acc_t;
  __shared__ typename R::State smem[4][kWave];
  const int tx = threadIdx.x, ty = threadIdx.y;
  const int64_t col = (int64_t)blockIdx.x * kWave + tx;
  const int64_t o = blockIdx.z;
  const int64_t lo = (int64_t)blockIdx.y * chunk;
  const int64_t hi = lo + chunk < red ? lo + chunk : red;
  typename R::State st = R::init();
  if (col < inner) {
    const T* p = x + o * red * inner + col;
    for (int64_t r = lo + ty; r < hi; r += 4) R::acc(st, (A)p[r * inner], r);
  }
  smem[ty][tx] = st;
  __syncthreads();
  if (ty == 0 && col < inner) {
    for (int k = 1; k < 4; ++k) st = R::combine(st, smem[k][tx]);
    if constexpr (PARTIAL) ws[(o * gridDim.y + blockIdx.y) * inner + col] = st;
    else write_final<R, O, FIN>(out, o * inner + col, st, divisor);
  }
}

// partials [outer][nsplit][inner] -> out [outer][inner]
template <typename O, typename R, int FIN>
__global__ __launch_bounds__(kRedBlock) void final_kernel(const typename R::State* __restrict__ ws,
                                                         O* __restrict__ out, int64_t outer, int64_t nsplit,
                                                         int64_t inner, double divisor) {
  const int64_t total = outer * inner;
  const int64_t stride = (int64_t)gridDim.x * kRedBlock;
  for (int64_t e = (int64_t)blockIdx.x * kRedBlock + threadIdx.x; e < total; e += stride) {
    const int64_t o = e / inner, c = e - o * inner;
    const typename R::State* p = ws + (o * nsplit) * inner + c;
    typename R::State st = R::init();
    int64_t s = 0;
    for (; s + 8 <= nsplit; s += 8) {  // eight independent loads in flight, then combine in order
      typename R::State part[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) part[k] = p[(s + k) * inner];
#pragma unroll
      for (int k = 0; k < 8; ++k) st = R::combine(st, part[k]);
    }
    for (; s < nsplit; ++s) st = R::combine(st, p[s * inner]);
    write_final<R, O, FIN>(out, e, st, divisor);
  }
}

// As cols_kernel with one 128-bit load per lane: lane tx owns V consecutive columns, so a wave
// reads 1 KB of every row it visits, and four row loads are in flight per thread.
// block = (64, 4); grid = (ceil(inner / (64 V)), nsplit, outer).  inner % V == 0, x 16-byte aligned.
template <typename T, typename O, typename R, int FIN, bool PARTIAL>
__global__ __launch_bounds__(kRedBlock) void cols_vec_kernel(const T* __restrict__ x, O* __restrict__ out,
                                                            typename R::State* __restrict__ ws, int64_t red,
                                                            int64_t inner, int64_t chunk, double divisor) {
  using A = typename R::acc_t;
  using State = typename R::State;
  constexpr int V = Vec<T>::N;
  __shared__ State smem[3][kWave][V];
  const int tx = threadIdx.x, ty = threadIdx.y;
  const int64_t col = ((int64_t)blockIdx.x * kWave + tx) * V;
  const int64_t o = blockIdx.z;
  const int64_t lo = (int64_t)blockIdx.y * chunk;
  const int64_t hi = lo + chunk < red ? lo + chunk : red;
  State st[V];
#pragma unroll
  for (int j = 0; j < V; ++j) st[j] = R::init();
  if (col < inner) {
    const T* p = x + o * red * inner + col;
    int64_t r = lo + ty;
    for (; r + 12 < hi; r += 16) {
      const Vec<T> v0 = load_vec_nt(p + r * inner), v1 = load_vec_nt(p + (r + 4) * inner),
                   v2 = load_vec_nt(p + (r + 8) * inner), v3 = load_vec_nt(p + (r + 12) * inner);
#pragma unroll
      for (int j = 0; j < V; ++j) {
        R::acc(st[j], (A)v0.v[j], r);
        R::acc(st[j], (A)v1.v[j], r + 4);
        R::acc(st[j], (A)v2.v[j], r + 8);
        R::acc(st[j], (A)v3.v[j], r + 12);
      }
    }
    for (; r < hi; r += 4) {
      const Vec<T> v = load_vec_nt(p + r * inner);
#pragma unroll
      for (int j = 0; j < V; ++j) R::acc(st[j], (A)v.v[j], r);
    }
  }
  if (ty > 0) {
#pragma unroll
    for (int j = 0; j < V; ++j) smem[ty - 1][tx][j] = st[j];
  }
  __syncthreads();
  if (ty == 0 && col < inner) {
#pragma unroll
    for (int j = 0; j < V; ++j) {
      for (int k = 0; k < 3; ++k) st[j] = R::combine(st[j], smem[k][tx][j]);
      if constexpr (PARTIAL) ws[(o * gridDim.y + blockIdx.y) * inner + col + j] = st[j];
      else write_final<R, O, FIN>(out, o * inner + col + j, st[j], divisor);
    }
  }
}

// Second pass for split rows (inner == 1): one wave per output, lanes stride over the row's
// nsplit partial states, then a wave reduce.  (A single thread walking a thousand partials
// one after the other costs several times the first pass.)
template <typename O, typename R, int FIN>
__global__ __launch_bounds__(kRedBlock) void final_rows_kernel(const typename R::State* __restrict__ ws,
                                                              O* __restrict__ out, int64_t outer, int64_t nsplit,
                                                              double divisor) {
  const int lane = threadIdx.x % kWave;
  const int64_t row = (int64_t)blockIdx.x * (kRedBlock / kWave) + threadIdx.x / kWave;
  if (row >= outer) return;  // whole waves leave together
  typename R::State st = R::init();
  for (int64_t s = lane; s < nsplit; s += kWave) st = R::combine(st, ws[row * nsplit + s]);
  st = wave_reduce(st, (R*)nullptr);
  if (lane == 0) write_final<R, O, FIN>(out, row, st, divisor);
}

// ---------------------------------------------------------------- planning
enum Kind { ROWS_WAVE, ROWS_BLOCK, ROWS_THREAD, ROWS_SUB, COLS };
struct Plan {
  Kind kind;
  int64_t nsplit, chunk;
};

static Plan plan_reduce(int64_t outer, int64_t red, int64_t inner, int elem_size) {
  Plan p{ROWS_BLOCK, 1, red};
  const int V = 16 / elem_size;
  const int64_t want_blocks = kNumCU * 4;
  if (inner == 1) {
    if (red <= 8 && outer >= 4096) { p.kind = ROWS_THREAD; return p; }
    if (red <= 64 * V && outer >= 8192) { p.kind = ROWS_SUB; return p; }  // up to four vectors per lane: one batch
    if (red <= 32 && outer >= 4096) { p.kind = ROWS_THREAD; return p; }
    if (outer >= 2048 && red <= 16384) { p.kind = ROWS_WAVE; return p; }
    p.kind = ROWS_BLOCK;
    if (outer < 512) {
      const int64_t unit = (int64_t)kRedBlock * V * 4;  // >= 4 vector loads per thread per split
      int64_t ns = (want_blocks + outer - 1) / outer;
      const int64_t max_ns = red / unit > 0 ? red / unit : 1;
      if (ns > max_ns) ns = max_ns;
      if (ns > 1) {
        int64_t chunk = (red + ns - 1) / ns;
        chunk = (chunk + kRedBlock * V - 1) / (kRedBlock * V) * (kRedBlock * V);
        p.chunk = chunk;
        p.nsplit = (red + chunk - 1) / chunk;
      }
    }
    return p;
  }
  p.kind = COLS;
  const int64_t per_block = inner % V == 0 ? (int64_t)kWave * V : kWave;  // columns per block (vector / scalar form)
  const int64_t base = outer * ((inner + per_block - 1) / per_block);
  if (base < want_blocks) {
    int64_t ns = (want_blocks + base - 1) / base;
    int64_t max_ns = red / 16 > 0 ? red / 16 : 1;  // >= 4 rows per thread per split
    if (max_ns > 64) max_ns = 64;                    // keeps the second pass short
    if (ns > max_ns) ns = max_ns;
    if (ns > 1) {
      p.chunk = (red + ns - 1) / ns;
      p.nsplit = (red + p.chunk - 1) / p.chunk;
    }
  }
  return p;
}

template <typename T, typename O, typename R, int FIN>
static int run_reduce(const void* xv, int64_t outer, int64_t red, int64_t inner, void* outv, void* wsv,
                      int64_t ws_bytes, hipStream_t st) {
  const T* x = static_cast<const T*>(xv);
  O* out = static_cast<O*>(outv);
  using State = typename R::State;
  State* ws = static_cast<State*>(wsv);
  const Plan p = plan_reduce(outer, red, inner, sizeof(T));
  const double divisor = (double)red;
  constexpr int V = Vec<T>::N;
  if (p.nsplit > 1) {
    const int64_t need = outer * p.nsplit * inner * (int64_t)sizeof(State);
    MI355_REQUIRE(ws != nullptr && ws_bytes >= need,
                  "mi355_reduce: workspace of %lld bytes needed, %lld given", (long long)need, (long long)ws_bytes);
  }
  switch (p.kind) {
    case ROWS_THREAD: {
      const int grid = grid_for(outer, kRedBlock, kNumCU * 16);
      hipLaunchKernelGGL((rows_thread_kernel<T, O, R, FIN>), dim3(grid), dim3(kRedBlock), 0, st, x, out, outer, red, divisor);
      break;
    }
    case ROWS_SUB: {
      const int grid = grid_for(outer, kRedBlock / 16, kNumCU * 16);
      if (aligned16(x) && red % V == 0)
        hipLaunchKernelGGL((rows_sub_kernel<T, O, R, FIN, 1>), dim3(grid), dim3(kRedBlock), 0, st, x, out, outer, red, divisor);
      else if (V > 1 && red > 128)  // shorter misaligned rows: single elements beat the masked window
        hipLaunchKernelGGL((rows_sub_kernel<T, O, R, FIN, 2>), dim3(grid), dim3(kRedBlock), 0, st, x, out, outer, red, divisor);
      else
        hipLaunchKernelGGL((rows_sub_kernel<T, O, R, FIN, 0>), dim3(grid), dim3(kRedBlock), 0, st, x, out, outer, red, divisor);
      break;
    }
    case ROWS_WAVE: {
      const bool vec = aligned16(x) && red % V == 0;
      const int grid = grid_for(outer, kRedBlock / kWave, kNumCU * 16);
      if (vec) hipLaunchKernelGGL((rows_wave_kernel<T, O, R, FIN, 1>), dim3(grid), dim3(kRedBlock), 0, st, x, out, outer, red, divisor);
      else if (V > 1) hipLaunchKernelGGL((rows_wave_kernel<T, O, R, FIN, 2>), dim3(grid), dim3(kRedBlock), 0, st, x, out, outer, red, divisor);
      else hipLaunchKernelGGL((rows_wave_kernel<T, O, R, FIN, 0>), dim3(grid), dim3(kRedBlock), 0, st, x, out, outer, red, divisor);
      break;
    }
    case ROWS_BLOCK: {
      const bool vec = aligned16(x) && red % V == 0;
      // grid.y carries rows: split oversize row counts over several launches.
      for (int64_t r0 = 0; r0 < outer; r0 += 65535) {
        const int64_t nr = outer - r0 < 65535 ? outer - r0 : 65535;
        dim3 grid((unsigned)p.nsplit, (unsigned)nr);
        const T* xr = x + r0 * red;
        O* outr = out + r0;
        State* wsr = ws ? ws + r0 * p.nsplit : nullptr;
#define MI355_ROWS_BLOCK(MODE_)                                                                                          \
  if (p.nsplit > 1) hipLaunchKernelGGL((rows_block_kernel<T, O, R, FIN, MODE_, true>), grid, dim3(kRedBlock), 0, st, xr, outr, wsr, red, p.chunk, divisor); \
  else hipLaunchKernelGGL((rows_block_kernel<T, O, R, FIN, MODE_, false>), grid, dim3(kRedBlock), 0, st, xr, outr, wsr, red, p.chunk, divisor);
        if (vec) { MI355_ROWS_BLOCK(1) }
        else if (V > 1) { MI355_ROWS_BLOCK(2) }
        else { MI355_ROWS_BLOCK(0) }
#undef MI355_ROWS_BLOCK
      }
      break;
    }
    case COLS: {
      const bool vec = V > 1 && inner % V == 0 && aligned16(x);
      const int64_t xb = vec ? (inner + kWave * V - 1) / (kWave * V) : (inner + kWave - 1) / kWave;
      MI355_REQUIRE(xb < (int64_t(1) << 31) && p.nsplit < 65536, "mi355_reduce: inner extent too large");
      for (int64_t o0 = 0; o0 < outer; o0 += 65535) {
        const int64_t no = outer - o0 < 65535 ? outer - o0 : 65535;
        dim3 grid((unsigned)xb, (unsigned)p.nsplit, (unsigned)no);
        const T* xo = x + o0 * red * inner;
        O* outo = out + o0 * inner;
        State* wso = ws ? ws + o0 * p.nsplit * inner : nullptr;
        if (vec) {
          if (p.nsplit > 1) hipLaunchKernelGGL((cols_vec_kernel<T, O, R, FIN, true>), grid, dim3(kWave, 4), 0, st, xo, outo, wso, red, inner, p.chunk, divisor);
          else hipLaunchKernelGGL((cols_vec_kernel<T, O, R, FIN, false>), grid, dim3(kWave, 4), 0, st, xo, outo, wso, red, inner, p.chunk, divisor);
        } else {
          if (p.nsplit > 1) hipLaunchKernelGGL((cols_kernel<T, O, R, FIN, true>), grid, dim3(kWave, 4), 0, st, xo, outo, wso, red, inner, p.chunk, divisor);
          else hipLaunchKernelGGL((cols_kernel<T, O, R, FIN, false>), grid, dim3(kWave, 4), 0, st, xo, outo, wso, red, inner, p.chunk, divisor);
        }
      }
      break;
    }
  }
  int rc = check_launch("mi355_reduce");
  if (rc) return rc;
  if (p.nsplit > 1) {
    if (inner == 1) {
      const int grid = (int)((outer + kRedBlock / kWave - 1) / (kRedBlock / kWave));  // outer < 512 on this path
      hipLaunchKernelGGL((final_rows_kernel<O, R, FIN>), dim3(grid), dim3(kRedBlock), 0, st, ws, out, outer, p.nsplit, divisor);
    } else {
      const int grid = grid_for(outer * inner, kRedBlock, kNumCU * 8);
      hipLaunchKernelGGL((final_kernel<O, R, FIN>), dim3(grid), dim3(kRedBlock), 0, st, ws, out, outer, p.nsplit, inner, divisor);
    }
    rc = check_launch("mi355_reduce(final)");
  }
  return rc;
}

template <typename T, typename O>
static int run_op(int op, const void* x, int64_t outer, int64_t red, int64_t inner, void* out, void* ws,
                  int64_t ws_bytes, hipStream_t st) {
  using A = typename OpMath<T>::type;
  using Acc = typename std::conditional<IsFloat<T>::value, A, int64_t>::type;  // ints sum in int64
  switch (op) {
    case MI355_SUM: return run_reduce<T, O, SumR<Acc>, FIN_VALUE>(x, outer, red, inner, out, ws, ws_bytes, st);
    case MI355_MEAN:
      if constexpr (IsFloat<T>::value) return run_reduce<T, O, SumR<Acc>, FIN_MEAN>(x, outer, red, inner, out, ws, ws_bytes, st);
      else return set_error(MI355_ERR_UNSUPPORTED, "mi355_reduce: mean needs a floating dtype");
    case MI355_AMAX: return run_reduce<T, O, AmaxR<A>, FIN_VALUE>(x, outer, red, inner, out, ws, ws_bytes, st);
    default: return set_error(MI355_ERR_INVALID, "mi355_reduce: unknown op %d", op);
  }
}

static size_t state_size(int op, int in_dtype) {
  const bool is_f64 = in_dtype == MI355_F64, is_int = in_dtype == MI355_I32 || in_dtype == MI355_I64;
  if (op == MI355_ARGMAX) return 16;
  if (op == MI355_AMAX) return (is_f64 || in_dtype == MI355_I64) ? 8 : 4;
  return (is_f64 || is_int) ? 8 : 4;
}

}  // namespace mi355

using namespace mi355;

// Bytes of scratch mi355_reduce needs for this problem (0 = single pass).
extern "C" int64_t mi355_reduce_workspace_bytes(int op, int in_dtype, int64_t outer, int64_t red,
                                                int64_t inner) {
  const int es = dtype_size(in_dtype);
  if (es == 0 || outer <= 0 || red <= 0 || inner <= 0) return 0;
  const Plan p = plan_reduce(outer, red, inner, es);
  if (p.nsplit <= 1) return 0;
  return outer * p.nsplit * inner * (int64_t)state_size(op, in_dtype);
}

extern "C" int mi355_reduce(int op, const void* x, int in_dtype, int64_t outer, int64_t red, int64_t inner,
                            void* out, int out_dtype, void* workspace, int64_t workspace_bytes, void* stream) {
  MI355_REQUIRE(outer >= 0 && inner >= 0 && red > 0, "mi355_reduce: bad extents outer=%lld red=%lld inner=%lld",
                (long long)outer, (long long)red, (long long)inner);
  if (outer == 0 || inner == 0) return MI355_OK;
  MI355_REQUIRE(x != nullptr && out != nullptr, "mi355_reduce: NULL data pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (op == MI355_ARGMAX) {
    MI355_REQUIRE(out_dtype == MI355_I64, "mi355_reduce(argmax): out dtype must be i64");
    switch (in_dtype) {
      case MI355_F32: return run_reduce<float, int64_t, ArgmaxR<float>, FIN_INDEX>(x, outer, red, inner, out, workspace, workspace_bytes, st);
      case MI355_F16: return run_reduce<f16_t, int64_t, ArgmaxR<float>, FIN_INDEX>(x, outer, red, inner, out, workspace, workspace_bytes, st);
      case MI355_BF16: return run_reduce<bf16_t, int64_t, ArgmaxR<float>, FIN_INDEX>(x, outer, red, inner, out, workspace, workspace_bytes, st);
      case MI355_F64: return run_reduce<double, int64_t, ArgmaxR<double>, FIN_INDEX>(x, outer, red, inner, out, workspace, workspace_bytes, st);
      case MI355_I32: return run_reduce<int32_t, int64_t, ArgmaxR<int32_t>, FIN_INDEX>(x, outer, red, inner, out, workspace, workspace_bytes, st);
      case MI355_I64: return run_reduce<int64_t, int64_t, ArgmaxR<int64_t>, FIN_INDEX>(x, outer, red, inner, out, workspace, workspace_bytes, st);
      default: return set_error(MI355_ERR_UNSUPPORTED, "mi355_reduce(argmax): unsupported dtype %s", dtype_name(in_dtype));
    }
  }
  const bool same = out_dtype == in_dtype;
  switch (in_dtype) {
    case MI355_F32:
      if (same) return run_op<float, float>(op, x, outer, red, inner, out, workspace, workspace_bytes, st);
      break;
    case MI355_F16:
      if (same) return run_op<f16_t, f16_t>(op, x, outer, red, inner, out, workspace, workspace_bytes, st);
      if (out_dtype == MI355_F32) return run_op<f16_t, float>(op, x, outer, red, inner, out, workspace, workspace_bytes, st);
      break;
    case MI355_BF16:
      if (same) return run_op<bf16_t, bf16_t>(op, x, outer, red, inner, out, workspace, workspace_bytes, st);
      if (out_dtype == MI355_F32) return run_op<bf16_t, float>(op, x, outer, red, inner, out, workspace, workspace_bytes, st);
      break;
    case MI355_F64:
      if (same) return run_op<double, double>(op, x, outer, red, inner, out, workspace, workspace_bytes, st);
      break;
    case MI355_I32:
      if (op == MI355_AMAX && same) return run_op<int32_t, int32_t>(op, x, outer, red, inner, out, workspace, workspace_bytes, st);
      if (op == MI355_SUM && out_dtype == MI355_I64) return run_op<int32_t, int64_t>(op, x, outer, red, inner, out, workspace, workspace_bytes, st);
      break;
    case MI355_I64:
      if (same && op != MI355_MEAN) return run_op<int64_t, int64_t>(op, x, outer, red, inner, out, workspace, workspace_bytes, st);
      break;
    default: break;
  }
  return set_error(MI355_ERR_UNSUPPORTED, "mi355_reduce: no kernel for op %d, %s -> %s", op,
                   dtype_name(in_dtype), dtype_name(out_dtype));
}

// ---------------------------------------------------------------- allocation-free form
// Scratch for callers that cannot allocate (HIP graph capture, serving loops): one array per
// GPU, held from library load until the process ends.  Host code never uses the array's name
// as an address: the per-device address comes from hipGetSymbolAddress once per device.
constexpr int64_t kStaticScratchBytes = 4 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static void* g_scratch_ptr[kMaxDevices];  // device address of `scratch`, per device; nullptr = not asked yet
static std::mutex g_scratch_mutex;

static int scratch_address(void** ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return set_error(MI355_ERR_LAUNCH, "mi355_reduce_static: hipGetDevice failed or device %d out of range: %s", dev,
                     hipGetErrorString(e));
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr)
      return set_error(MI355_ERR_LAUNCH, "mi355_reduce_static: hipGetSymbolAddress failed on device %d: %s", dev,
                       hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *ptr = g_scratch_ptr[dev];
  return MI355_OK;
}

// Called by mi355_init(): resolves the address on the current device ahead of the first call, so that
// a mi355_reduce_static recorded into a HIP graph does no runtime query during the capture.
namespace mi355 {
int reduce_static_init() {
  void* ptr = nullptr;
  return scratch_address(&ptr);
}
}  // namespace mi355

extern "C" int64_t mi355_reduce_static_max_bytes(void) { return kStaticScratchBytes; }

extern "C" int mi355_reduce_static(int op, const void* x, int in_dtype, int64_t outer, int64_t red, int64_t inner,
                                   void* out, int out_dtype, void* stream) {
  const int64_t need = mi355_reduce_workspace_bytes(op, in_dtype, outer, red, inner);
  if (need == 0) return mi355_reduce(op, x, in_dtype, outer, red, inner, out, out_dtype, nullptr, 0, stream);
  MI355_REQUIRE(need <= kStaticScratchBytes,
                "mi355_reduce_static: this reduction needs %lld bytes of scratch, the built-in buffer holds %lld; "
                "call mi355_reduce with a workspace of the caller's",
                (long long)need, (long long)kStaticScratchBytes);
  void* ptr = nullptr;
  const int rc = scratch_address(&ptr);
  if (rc) return rc;
  // Every partial result the second pass reads is written by the first pass of the same call:
  // nothing in the buffer has to start at zero.
  return mi355_reduce(op, x, in_dtype, outer, red, inner, out, out_dtype, ptr, need, stream);
}
