// Shared device/host helpers for the gfx950 kernels: dtype traits, 128-bit vector
// access, wave64 reductions (DPP inside 16-lane rows, bpermute across rows), dimension
// collapsing and the thread-local error string behind mi355_last_error().
#pragma once
#include <type_traits>

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <math.h>

#include "../../include/mi355_aten.h"

namespace mi355 {

// ---------------------------------------------------------------- error plumbing
int set_error(int code, const char* fmt, ...);
int check_launch(const char* what);

// Test and measurement knobs, read from the environment once per process (MI355_GEMM_TILE,
// MI355_GEMM_WAVES) and changed afterwards only through mi355_set_knob(): no entry point calls
// getenv on its way to a launch.
struct Knobs {
  char gemm_tile[16];   // "" = the planner decides; see mi355_set_knob in include/mi355_aten.h
  char gemm_waves[8];   // "" / "4" / "8"
  char gemm_split[12];  // "" = the planner decides how a split K meets; "launch2" a summing launch, "inlaunch" inside the one launch
  int x16_spin_limit;   // polls of the in-launch split-K's bounded wait before it gives up
  int gemm_prefetch;    // workgroups that only warm the last-level cache next to a 128x128-tile launch's tiles: -1 = the planner decides
};
const Knobs& knobs();
constexpr int kX16SpinLimitDefault = 1 << 21;  // about 1 us per poll

#define MI355_REQUIRE(cond, ...)                                  \
  do {                                                            \
    if (!(cond)) return ::mi355::set_error(MI355_ERR_INVALID, __VA_ARGS__); \
  } while (0)

// ---------------------------------------------------------------- scalar types
typedef __bf16 bf16_t;
typedef _Float16 f16_t;

constexpr int kWave = 64;
// Chip geometry the launch heuristics are sized for.
constexpr int kNumCU = 256;
constexpr int kNumXCD = 8;

template <typename T> struct OpMath { using type = T; };
template <> struct OpMath<bf16_t> { using type = float; };
template <> struct OpMath<f16_t> { using type = float; };

template <typename T> struct IsFloat { static constexpr bool value = false; };
template <> struct IsFloat<float> { static constexpr bool value = true; };
template <> struct IsFloat<double> { static constexpr bool value = true; };
template <> struct IsFloat<bf16_t> { static constexpr bool value = true; };
template <> struct IsFloat<f16_t> { static constexpr bool value = true; };

template <typename T> __device__ __forceinline__ bool is_nan(T) { return false; }
template <> __device__ __forceinline__ bool is_nan<float>(float v) { return v != v; }
template <> __device__ __forceinline__ bool is_nan<double>(double v) { return v != v; }

inline int dtype_size(int dt) {
  switch (dt) {
    case MI355_F32: case MI355_I32: return 4;
    case MI355_F16: case MI355_BF16: case MI355_I16: return 2;
    case MI355_F64: case MI355_I64: return 8;
    case MI355_I8: case MI355_U8: case MI355_BOOL: return 1;
    default: return 0;
  }
}
inline const char* dtype_name(int dt) {
  static const char* names[] = {"f32", "f16", "bf16", "f64", "i32", "i64", "i16", "i8", "u8", "bool"};
  return (dt >= 0 && dt < MI355_DTYPE_COUNT) ? names[dt] : "?";
}

// Calls f(T{}) with the C++ type of dtype `dt`; `return`s UNSUPPORTED for others.
#define MI355_DISPATCH_FLOAT(dt, NAME, ...)                                     \
  switch (dt) {                                                                 \
    case MI355_F32: { using T = float; __VA_ARGS__; break; }                    \
    case MI355_F16: { using T = ::mi355::f16_t; __VA_ARGS__; break; }           \
    case MI355_BF16: { using T = ::mi355::bf16_t; __VA_ARGS__; break; }         \
    case MI355_F64: { using T = double; __VA_ARGS__; break; }                   \
    default:                                                                    \
      return ::mi355::set_error(MI355_ERR_UNSUPPORTED, "%s: unsupported dtype %s", NAME, \
                                ::mi355::dtype_name(dt));                       \
  }

#define MI355_DISPATCH_NUMERIC(dt, NAME, ...)                                   \
  switch (dt) {                                                                 \
    case MI355_F32: { using T = float; __VA_ARGS__; break; }                    \
    case MI355_F16: { using T = ::mi355::f16_t; __VA_ARGS__; break; }           \
    case MI355_BF16: { using T = ::mi355::bf16_t; __VA_ARGS__; break; }         \
    case MI355_F64: { using T = double; __VA_ARGS__; break; }                   \
    case MI355_I32: { using T = int32_t; __VA_ARGS__; break; }                  \
    case MI355_I64: { using T = int64_t; __VA_ARGS__; break; }                  \
    case MI355_I16: { using T = int16_t; __VA_ARGS__; break; }                  \
    case MI355_I8: { using T = int8_t; __VA_ARGS__; break; }                    \
    case MI355_U8: { using T = uint8_t; __VA_ARGS__; break; }                   \
    default:                                                                    \
      return ::mi355::set_error(MI355_ERR_UNSUPPORTED, "%s: unsupported dtype %s", NAME, \
                                ::mi355::dtype_name(dt));                       \
  }

// ---------------------------------------------------------------- 128-bit access
// VecT<T>: as many T as fit in 16 bytes, loaded/stored with one dwordx4 instruction.
template <typename T> struct alignas(16) Vec {
  static constexpr int N = 16 / sizeof(T);
  T v[N];
};
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T> __device__ __forceinline__ Vec<T> load_vec(const T* p) {
  u32x4 raw = *reinterpret_cast<const u32x4*>(p);
  return __builtin_bit_cast(Vec<T>, raw);
}
// Streaming variants: data touched once, keep it out of the way of reused lines.
template <typename T> __device__ __forceinline__ Vec<T> load_vec_nt(const T* p) {
  u32x4 raw = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  return __builtin_bit_cast(Vec<T>, raw);
}
template <typename T> __device__ __forceinline__ void store_vec(T* p, const Vec<T>& v) {
  *reinterpret_cast<u32x4*>(p) = __builtin_bit_cast(u32x4, v);
}
template <typename T> __device__ __forceinline__ void store_vec_nt(T* p, const Vec<T>& v) {
  __builtin_nontemporal_store(__builtin_bit_cast(u32x4, v), reinterpret_cast<u32x4*>(p));
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---------------------------------------------------------------- wave64 reductions
// dpp_ctrl encodings (GCN3+/CDNA): quad_perm = 0x00..0xFF, row_ror:n = 0x120 + n.
template <int CTRL> __device__ __forceinline__ int dpp_i32(int v) {
  return __builtin_amdgcn_update_dpp(v, v, CTRL, 0xF, 0xF, false);
}
template <int CTRL> __device__ __forceinline__ float dpp(float v) {
  return __builtin_bit_cast(float, dpp_i32<CTRL>(__builtin_bit_cast(int, v)));
}
template <int CTRL> __device__ __forceinline__ int dpp(int v) { return dpp_i32<CTRL>(v); }
template <int CTRL> __device__ __forceinline__ double dpp(double v) {
  int2 p = __builtin_bit_cast(int2, v);
  p.x = dpp_i32<CTRL>(p.x);
  p.y = dpp_i32<CTRL>(p.y);
  return __builtin_bit_cast(double, p);
}
template <int CTRL> __device__ __forceinline__ int64_t dpp(int64_t v) {
  int2 p = __builtin_bit_cast(int2, v);
  p.x = dpp_i32<CTRL>(p.x);
  p.y = dpp_i32<CTRL>(p.y);
  return __builtin_bit_cast(int64_t, p);
}

// All-reduce over the 64 lanes of a wave with an associative, commutative `op`.
// Steps 1, 2 (quad_perm) and 4, 8 (row_ror) stay in the DPP path of the VALU; the two
// cross-row steps (16, 32) go through ds_bpermute via __shfl_xor.
template <typename T, typename Op> __device__ __forceinline__ T wave_allreduce(T v, Op op) {
  v = op(v, dpp<0xB1>(v));   // quad_perm [1,0,3,2]
  v = op(v, dpp<0x4E>(v));   // quad_perm [2,3,0,1]
  v = op(v, dpp<0x124>(v));  // row_ror:4
  v = op(v, dpp<0x128>(v));  // row_ror:8
  v = op(v, __shfl_xor(v, 16, kWave));
  v = op(v, __shfl_xor(v, 32, kWave));
  return v;
}

struct SumOp {
  template <typename T> __device__ __forceinline__ T operator()(T a, T b) const { return a + b; }
};
// NaN-propagating max (either operand NaN -> NaN), the ATen amax/maximum rule.
struct MaxNanOp {
  template <typename T> __device__ __forceinline__ T operator()(T a, T b) const {
    if constexpr (std::is_same<T, float>::value) {
      return __builtin_elementwise_maximum(a, b);  // v_maximum3_f32: IEEE 754-2019 maximum, one instruction
    } else if constexpr (IsFloat<T>::value) {
      return (is_nan(a) || a > b) ? a : b;  // b NaN: a > b false -> b
    } else {
      return a > b ? a : b;
    }
  }
};
// Plain max for values known NaN-free (softmax keeps a separate NaN-safe path).
struct MaxOp {
  template <typename T> __device__ __forceinline__ T operator()(T a, T b) const { return a > b ? a : b; }
};

// Block-wide all-reduce: wave reduce, one LDS slot per wave, every thread re-reduces
// the (<= 16) slots.  `smem` must hold blockDim.x / 64 elements of T.  Ends with the
// result in all threads; callers reusing `smem` must __syncthreads() first.
template <typename T, typename Op>
__device__ __forceinline__ T block_allreduce(T v, Op op, T* smem, T identity) {
  v = wave_allreduce(v, op);
  const int nwaves = blockDim.x / kWave;
  if (nwaves == 1) return v;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  if (lane == 0) smem[wave] = v;
  __syncthreads();
  T r = identity;
  for (int w = 0; w < nwaves; ++w) r = op(r, smem[w]);
  return r;
}

// ---------------------------------------------------------------- few, very long rows
// Softmax and layer norm over a handful of rows of tens of thousands of elements and more leave
// the chip idle at one block per row.  Such rows are cut into `nsplit` chunks of `chunk` elements
// (a multiple of 256 vectors): a first launch leaves one partial state per (row, chunk) in the
// caller's workspace (kRowPartialBytes each), a second combines a row's partials and writes its
// chunk of the output.  nsplit == 1: not worth splitting.
constexpr int kRowPartialBytes = 24;
struct RowSplit {
  int64_t nsplit, chunk;
};
inline RowSplit plan_row_split(int64_t rows, int64_t n, int elem_size) {
  RowSplit p{1, n};
  const int64_t unit = 256 * (16 / elem_size);  // one vector per thread of a 256-thread block
  if (rows <= 0 || rows >= 64 || n < 32768 || n < 8 * unit) return p;
  int64_t ns = (2 * kNumCU + rows - 1) / rows;
  const int64_t max_ns = n / (4 * unit);  // at least four vectors per thread and chunk
  if (ns > max_ns) ns = max_ns;
  if (ns > 256) ns = 256;
  if (ns <= 1) return p;
  int64_t chunk = (n + ns - 1) / ns;
  chunk = (chunk + unit - 1) / unit * unit;
  p.chunk = chunk;
  p.nsplit = (n + chunk - 1) / chunk;
  if (p.nsplit <= 1) p = RowSplit{1, n};
  return p;
}

// ---------------------------------------------------------------- strided views
// Up to MI355_MAX_DIMS collapsed dims shared by `NT` tensors; passed to kernels by value.
template <int NT> struct Dims {
  int32_t ndim;
  int64_t sizes[MI355_MAX_DIMS];
  int64_t strides[NT][MI355_MAX_DIMS];
};

// Merge adjacent dims that are jointly dense in every tensor and drop size-1 dims.
// Dim 0 is outermost.  Returns the collapsed view (ndim >= 1).
template <int NT>
inline Dims<NT> collapse_dims(int ndim, const int64_t* sizes, const int64_t* const strides[NT]) {
  Dims<NT> d;
  d.ndim = 0;
  for (int i = 0; i < ndim; ++i) {
    if (sizes[i] == 1) continue;
    if (d.ndim > 0) {
      bool mergeable = true;
      const int p = d.ndim - 1;
      for (int t = 0; t < NT; ++t)
        if (d.strides[t][p] != strides[t][i] * sizes[i]) mergeable = false;
      if (mergeable) {
        d.sizes[p] *= sizes[i];
        for (int t = 0; t < NT; ++t) d.strides[t][p] = strides[t][i];
        continue;
      }
    }
    d.sizes[d.ndim] = sizes[i];
    for (int t = 0; t < NT; ++t) d.strides[t][d.ndim] = strides[t][i];
    ++d.ndim;
  }
  if (d.ndim == 0) {
    d.ndim = 1;
    d.sizes[0] = 1;
    for (int t = 0; t < NT; ++t) d.strides[t][0] = 1;
  }
  for (int i = d.ndim; i < MI355_MAX_DIMS; ++i) {
    d.sizes[i] = 1;
    for (int t = 0; t < NT; ++t) d.strides[t][i] = 0;
  }
  return d;
}

inline int64_t numel(const mi355_tensor* t) {
  int64_t n = 1;
  for (int i = 0; i < t->ndim; ++i) n *= t->sizes[i];
  return n;
}
inline bool same_shape(const mi355_tensor* a, const mi355_tensor* b) {
  if (a->ndim != b->ndim) return false;
  for (int i = 0; i < a->ndim; ++i)
    if (a->sizes[i] != b->sizes[i]) return false;
  return true;
}
int check_tensor(const mi355_tensor* t, const char* op, const char* name);

// If every tensor has identical strides that tile memory densely in some dim order
// (a permuted-contiguous layout), the op is a flat 1-D pass over `numel` elements.
bool same_dense_layout(const mi355_tensor* const* ts, int nt);

inline int grid_for(int64_t work_items, int per_block, int max_blocks) {
  int64_t b = (work_items + per_block - 1) / per_block;
  if (b < 1) b = 1;
  if (b > max_blocks) b = max_blocks;
  return static_cast<int>(b);
}

}  // namespace mi355
