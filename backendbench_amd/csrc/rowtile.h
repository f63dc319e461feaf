// A row held in the registers of W cooperating wave64s (W = 1, 2 or 4 waves of one 256-thread
// block): NV slabs of 64*W lanes x V elements (V = one 128-bit load), converted to fp32 on
// load.  Used by the single-pass softmax and layer norm kernels: the row is read from HBM
// once (non-temporal 128-bit loads), reduced with wave all-reduces plus one LDS exchange when
// W > 1, and written once.  Spreading a row over more waves keeps the per-lane tile at <= 32
// values, so eight waves fit on a SIMD and all rows of a launch are resident at once.
// VEC = false keeps the same register shape with scalar, lane-interleaved accesses for rows
// whose base is not 16-byte aligned (W = 1 only).
#pragma once
#include <type_traits>

#include "common.h"
#include "elementwise.h"  // VecN / ld / st

namespace mi355 {

constexpr int kRowBlock = 256;  // threads per block of every row-tile kernel

// VB: bytes per lane and access (16; 8 when the output element is twice as wide as the input
// element, so that the output side still moves whole 16-byte pieces per lane).
template <typename T, int NV, bool VEC, int W, int BLOCK = kRowBlock, int VB = 16> struct RowTile {
  static constexpr int V = VB / sizeof(T);
  static constexpr int GROUP = kWave * W;        // lanes cooperating on one row
  static constexpr int ROWS_PER_BLOCK = BLOCK / GROUP;
  float v[NV][V];

  // Column of element (k, j) for lane `t` (0 .. GROUP-1) of the row group.
  static __device__ __forceinline__ int64_t col(int k, int j, int t) {
    if constexpr (VEC) return ((int64_t)k * GROUP + t) * V + j;
    else return ((int64_t)k * V + j) * GROUP + t;
  }

  __device__ __forceinline__ void load(const T* row, int64_t n, int t, float pad) {
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      if constexpr (VEC) {
        const int64_t c = col(k, 0, t);
        if (c < n) {  // n % V == 0 on this path: a vector is all-in or all-out
          const VecN<T, V> x = ld_nt<T, V>(row + c);
#pragma unroll
          for (int j = 0; j < V; ++j) v[k][j] = static_cast<float>(x.v[j]);
        } else {
#pragma unroll
          for (int j = 0; j < V; ++j) v[k][j] = pad;
        }
      } else {
#pragma unroll
        for (int j = 0; j < V; ++j) {
          const int64_t c = col(k, j, t);
          v[k][j] = c < n ? static_cast<float>(row[c]) : pad;
        }
      }
    }
  }

  // out[c] = f(v, c) for every in-range element, written in the slab layout.
  template <typename O, typename Fn>
  __device__ __forceinline__ void store(O* row, int64_t n, int t, Fn f) const {
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      if constexpr (VEC) {
        const int64_t c = col(k, 0, t);
        if (c < n) {
          VecN<O, V> x;
#pragma unroll
          for (int j = 0; j < V; ++j) x.v[j] = static_cast<O>(f(v[k][j], c + j));
          st_nt<O, V>(row + c, x);
        }
      } else {
#pragma unroll
        for (int j = 0; j < V; ++j) {
          const int64_t c = col(k, j, t);
          if (c < n) row[c] = static_cast<O>(f(v[k][j], c));
        }
      }
    }
  }

  // Shifted access (vector layout only) for rows that do not start on a 16-byte boundary: `a`
  // (0 <= a < V) is how many elements past the previous boundary the row begins.  The lanes
  // walk the aligned window that starts `a` elements before the row, so every load is a whole
  // aligned 128-bit vector; elements outside [0, n) — the tail of the previous row, the head
  // of the next one, or at most 15 bytes beyond either end of the tensor, inside 16-byte
  // chunks that also hold tensor bytes — are replaced by `pad`.  The row fits when
  // n + a <= NV * GROUP * V.
  __device__ __forceinline__ void load_shifted(const T* row, int64_t n, int a, int t, float pad) {
    static_assert(VEC, "shifted access uses the vector layout");
    const T* win = row - a;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int64_t w = ((int64_t)k * GROUP + t) * V;
      if (w < n + a) {
        const VecN<T, V> x = ld_nt<T, V>(win + w);
#pragma unroll
        for (int j = 0; j < V; ++j) {
          const int64_t c = w + j - a;
          v[k][j] = (c >= 0 && c < n) ? static_cast<float>(x.v[j]) : pad;
        }
      } else {
#pragma unroll
        for (int j = 0; j < V; ++j) v[k][j] = pad;
      }
    }
  }

  // Counterpart of load_shifted: whole vectors where all V elements belong to the row, single
  // elements at the two ends (the neighbouring rows are written by other waves).
  template <typename O, typename Fn>
  __device__ __forceinline__ void store_shifted(O* row, int64_t n, int a, int t, Fn f) const {
    O* win = row - a;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      const int64_t w = ((int64_t)k * GROUP + t) * V;
      if (w >= n + a) continue;
      if (w >= a && w + V <= n + a) {
        VecN<O, V> x;
#pragma unroll
        for (int j = 0; j < V; ++j) x.v[j] = static_cast<O>(f(v[k][j], w + j - a));
        st_nt<O, V>(win + w, x);
      } else {
#pragma unroll
        for (int j = 0; j < V; ++j) {
          const int64_t c = w + j - a;
          if (c >= 0 && c < n) row[c] = static_cast<O>(f(v[k][j], c));
        }
      }
    }
  }
};

// Elements between the previous V-element boundary and `p` (0 for aligned rows).
template <typename T, int V = 16 / sizeof(T)> __device__ __forceinline__ int row_misalignment(const T* p) {
  return (int)((reinterpret_cast<uintptr_t>(p) / sizeof(T)) % V);
}

// All-reduce over the W waves of a row group.  `smem` has one slot per wave of the block and
// must not be reused by the caller before the next __syncthreads().  Every thread of the
// block has to call this (it contains a barrier when W > 1).
template <int W, typename T, typename Op>
__device__ __forceinline__ T group_allreduce(T v, Op op, T* smem) {
  v = wave_allreduce(v, op);
  if constexpr (W == 1) {
    return v;
  } else {
    const int wave = threadIdx.x / kWave;
    if (threadIdx.x % kWave == 0) smem[wave] = v;
    __syncthreads();
    const int first = wave / W * W;
    T r = smem[first];
#pragma unroll
    for (int i = 1; i < W; ++i) r = op(r, smem[first + i]);
    return r;
  }
}

// All-reduce over the G = 1 .. 32 adjacent lanes that share a short row (G a power of two).
template <int G, typename Op> __device__ __forceinline__ float sub_allreduce(float v, Op op) {
  if constexpr (G >= 2) v = op(v, dpp<0xB1>(v));    // quad_perm [1,0,3,2]
  if constexpr (G >= 4) v = op(v, dpp<0x4E>(v));    // quad_perm [2,3,0,1]
  if constexpr (G >= 8) v = op(v, dpp<0x141>(v));   // row_half_mirror: the other quad of 8 lanes
  if constexpr (G >= 16) v = op(v, dpp<0x140>(v));  // row_mirror: the other half of 16 lanes
  if constexpr (G >= 32) v = op(v, __shfl_xor(v, 16, kWave));
  return v;
}
// Picks (NV, W) for rows of n elements of T and calls body(NV, W, VEC) with integral
// constants; false when the row does not fit (16 slabs over 4 waves, or 64 values per lane over
// max_w waves).  Aligned rows get at most
// 32 values per lane (W grows instead); unaligned rows use one wave and the scalar layout.
template <typename T, typename Body, int VB = 16>
inline bool dispatch_row_tile(int64_t n, bool vec, Body body, int max_w = 4, std::integral_constant<int, VB> = {}) {
  constexpr int V = VB / sizeof(T);
  using std::integral_constant;
#define MI355_ROW(NV_, W_, VEC_)                                                              \
  {                                                                                           \
    body(integral_constant<int, NV_>(), integral_constant<int, W_>(), integral_constant<bool, VEC_>()); \
    return true;                                                                              \
  }
  if (!vec) {
    const int64_t unit = V * kWave;
    if (n <= unit) MI355_ROW(1, 1, false)
    if (n <= 2 * unit) MI355_ROW(2, 1, false)
    if (n <= 4 * unit) MI355_ROW(4, 1, false)
    if (n <= 8 * unit) MI355_ROW(8, 1, false)
    if (n <= 16 * unit) MI355_ROW(16, 1, false)
    return false;
  }
  constexpr int NV32 = 32 / V;  // slabs that make 32 values per lane
  if (n <= 32 * kWave) {
    const int64_t unit = V * kWave;
    if (n <= unit) MI355_ROW(1, 1, true)
    if (n <= 2 * unit) MI355_ROW(2, 1, true)
    if (NV32 >= 4 && n <= 4 * unit) MI355_ROW(4, 1, true)
    MI355_ROW(NV32, 1, true)
  }
  if (n <= 32 * kWave * 2) MI355_ROW(NV32, 2, true)
  const int64_t unit4 = V * kWave * 4;
  if (n <= NV32 * unit4) MI355_ROW(NV32, 4, true)
  // Callers whose kernels take 512- and 1024-thread blocks (max_w 8 / 16) keep 32 values per
  // lane up to 32 K elements and go to 64 per lane only beyond that.
  if (max_w >= 8 && n <= 32 * kWave * 8) MI355_ROW(NV32, 8, true)
  if (max_w >= 16 && n <= 32 * kWave * 16) MI355_ROW(NV32, 16, true)
  if (max_w >= 16 && n <= 64 * kWave * 16) MI355_ROW(2 * NV32, 16, true)
  if (NV32 < 8 && n <= 8 * unit4) MI355_ROW(8, 4, true)
  if (n <= 16 * unit4) MI355_ROW(16, 4, true)
#undef MI355_ROW
  return false;
}

}  // namespace mi355
