// A row held in the registers of one wave64: NV slabs of 64 lanes x V elements (V = one
// 128-bit load), converted to fp32 on load.  Used by the single-pass softmax and layer
// norm kernels: the row is read from HBM once, reduced with wave all-reduces, and written
// once.  VEC=false keeps the same register shape with scalar, lane-interleaved accesses
// for rows whose base is not 16-byte aligned.
#pragma once
#include <type_traits>

#include "common.h"
#include "elementwise.h"  // VecN / ld / st

namespace mi355 {

template <typename T, int NV, bool VEC> struct RowTile {
  static constexpr int V = 16 / sizeof(T);
  static constexpr int CAP = NV * V * kWave;  // elements one wave can hold
  float v[NV][V];

  // Column of element (k, j) for this lane.
  static __device__ __forceinline__ int64_t col(int k, int j, int lane) {
    if constexpr (VEC) return ((int64_t)k * kWave + lane) * V + j;
    else return ((int64_t)k * V + j) * kWave + lane;
  }

  __device__ __forceinline__ void load(const T* row, int64_t n, int lane, float pad) {
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      if constexpr (VEC) {
        const int64_t c = col(k, 0, lane);
        if (c < n) {  // n % V == 0 on this path: a vector is all-in or all-out
          const Vec<T> t = load_vec(row + c);
#pragma unroll
          for (int j = 0; j < V; ++j) v[k][j] = static_cast<float>(t.v[j]);
        } else {
#pragma unroll
          for (int j = 0; j < V; ++j) v[k][j] = pad;
        }
      } else {
#pragma unroll
        for (int j = 0; j < V; ++j) {
          const int64_t c = col(k, j, lane);
          v[k][j] = c < n ? static_cast<float>(row[c]) : pad;
        }
      }
    }
  }

  // out[c] = f(v, c) for every in-range element, written in the slab layout.
  template <typename O, typename Fn>
  __device__ __forceinline__ void store(O* row, int64_t n, int lane, Fn f) const {
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      if constexpr (VEC) {
        const int64_t c = col(k, 0, lane);
        if (c < n) {
          VecN<O, V> t;
#pragma unroll
          for (int j = 0; j < V; ++j) t.v[j] = static_cast<O>(f(v[k][j], c + j));
          st<O, V>(row + c, t);
        }
      } else {
#pragma unroll
        for (int j = 0; j < V; ++j) {
          const int64_t c = col(k, j, lane);
          if (c < n) row[c] = static_cast<O>(f(v[k][j], c));
        }
      }
    }
  }
};

// Calls body(std::integral_constant<int, NV>) for the smallest NV in {1,2,4,8,16} whose
// tile holds n elements of T; returns false when the row is too long for registers.
template <typename T, typename Body> inline bool dispatch_row_tile(int64_t n, Body body) {
  constexpr int64_t unit = (16 / sizeof(T)) * kWave;
  if (n <= unit) { body(std::integral_constant<int, 1>()); return true; }
  if (n <= 2 * unit) { body(std::integral_constant<int, 2>()); return true; }
  if (n <= 4 * unit) { body(std::integral_constant<int, 4>()); return true; }
  if (n <= 8 * unit) { body(std::integral_constant<int, 8>()); return true; }
  if (n <= 16 * unit) { body(std::integral_constant<int, 16>()); return true; }
  return false;
}

}  // namespace mi355
