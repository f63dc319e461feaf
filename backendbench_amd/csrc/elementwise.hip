// add / mul / maximum / relu / clamp / where / copy-cast entry points.
#include "elementwise.h"

namespace mi355 {

struct Unused {};

// ---- binary ----------------------------------------------------------------------
template <typename T> struct AddF {
  using out_t = T; using in0_t = T; using in1_t = T; using in2_t = Unused;
  static constexpr int NIN = 2;
  using M = typename OpMath<T>::type;
  M alpha;
  __device__ __forceinline__ T operator()(T a, T b, Unused) const {
    return static_cast<T>(static_cast<M>(a) + alpha * static_cast<M>(b));
  }
};
template <typename T> struct MulF {
  using out_t = T; using in0_t = T; using in1_t = T; using in2_t = Unused;
  static constexpr int NIN = 2;
  using M = typename OpMath<T>::type;
  __device__ __forceinline__ T operator()(T a, T b, Unused) const {
    return static_cast<T>(static_cast<M>(a) * static_cast<M>(b));
  }
};
// fp32 result from one fp32 and one half-precision operand (type promotion of a mixed-precision
// residual add or scale): the narrow operand is widened in registers instead of by a separate
// cast pass over memory.
template <typename TA, typename TB> struct AddMixF {
  using out_t = float; using in0_t = TA; using in1_t = TB; using in2_t = Unused;
  static constexpr int NIN = 2;
  float alpha;
  __device__ __forceinline__ float operator()(TA a, TB b, Unused) const {
    return static_cast<float>(a) + alpha * static_cast<float>(b);
  }
};
template <typename TA, typename TB> struct MulMixF {
  using out_t = float; using in0_t = TA; using in1_t = TB; using in2_t = Unused;
  static constexpr int NIN = 2;
  __device__ __forceinline__ float operator()(TA a, TB b, Unused) const {
    return static_cast<float>(a) * static_cast<float>(b);
  }
};
// Floating point: IEEE 754-2019 maximum / minimum (a NaN operand gives NaN, -0 is below +0), which
// is ATen's rule.  In fp32 that is one instruction (v_maximum3_f32 / v_minimum3_f32); in fp64 the
// NaN-ignoring hardware max / min plus one unordered compare that puts the NaN back.  At two bytes
// per element a chain of compares and selects instead keeps these kernels off the memory roofline.
__device__ __forceinline__ float nan_max(float x, float y) { return __builtin_elementwise_maximum(x, y); }
__device__ __forceinline__ float nan_min(float x, float y) { return __builtin_elementwise_minimum(x, y); }
__device__ __forceinline__ double nan_max(double x, double y) {
  return __builtin_isunordered(x, y) ? x + y : __builtin_fmax(x, y);
}
__device__ __forceinline__ double nan_min(double x, double y) {
  return __builtin_isunordered(x, y) ? x + y : __builtin_fmin(x, y);
}

template <typename T> struct MaximumF {
  using out_t = T; using in0_t = T; using in1_t = T; using in2_t = Unused;
  static constexpr int NIN = 2;
  using M = typename OpMath<T>::type;
  static constexpr bool kPair = std::is_same<T, f16_t>::value;  // v_pk_maximum3_f16: IEEE 754-2019 maximum of two pairs
  __device__ __forceinline__ void pair(const T* a, const T* b, const Unused*, T* r) const {
    const f16x2_t m = __builtin_elementwise_maximum(f16x2_t{(_Float16)a[0], (_Float16)a[1]}, f16x2_t{(_Float16)b[0], (_Float16)b[1]});
    r[0] = (T)m[0];
    r[1] = (T)m[1];
  }
  __device__ __forceinline__ T operator()(T a, T b, Unused) const {
    const M x = static_cast<M>(a), y = static_cast<M>(b);
    if constexpr (IsFloat<T>::value) {
      return static_cast<T>(nan_max(x, y));
    } else {
      return x > y ? a : b;
    }
  }
};

template <typename T> struct MinimumF {
  using out_t = T; using in0_t = T; using in1_t = T; using in2_t = Unused;
  static constexpr int NIN = 2;
  using M = typename OpMath<T>::type;
  static constexpr bool kPair = std::is_same<T, f16_t>::value;
  __device__ __forceinline__ void pair(const T* a, const T* b, const Unused*, T* r) const {
    const f16x2_t m = __builtin_elementwise_minimum(f16x2_t{(_Float16)a[0], (_Float16)a[1]}, f16x2_t{(_Float16)b[0], (_Float16)b[1]});
    r[0] = (T)m[0];
    r[1] = (T)m[1];
  }
  __device__ __forceinline__ T operator()(T a, T b, Unused) const {
    const M x = static_cast<M>(a), y = static_cast<M>(b);
    if constexpr (IsFloat<T>::value) {
      return static_cast<T>(nan_min(x, y));
    } else {
      return x < y ? a : b;
    }
  }
};

// ---- unary -----------------------------------------------------------------------
template <typename T> struct ReluF {
  using out_t = T; using in0_t = T; using in1_t = Unused; using in2_t = Unused;
  static constexpr int NIN = 1;
  using M = typename OpMath<T>::type;
  __device__ __forceinline__ T operator()(T a, Unused, Unused) const {
    const M x = static_cast<M>(a);
    // NaN < 0 and -0.0 < 0 are false: both pass through unchanged, as on ATen's CPU kernel
    return x < M(0) ? static_cast<T>(M(0)) : a;
  }
};
template <typename T> struct ClampF {
  using out_t = T; using in0_t = T; using in1_t = Unused; using in2_t = Unused;
  static constexpr int NIN = 1;
  using M = typename OpMath<T>::type;
  M lo, hi;  // floating point: a missing bound is -inf / +inf, a NaN bound is kept (it makes everything NaN)
  bool has_lo, has_hi;
  // f16: the bounds rounded to f16 (as ATen rounds them to the tensor's dtype), then the NaN-propagating
  // packed pair - a NaN input or bound gives NaN, hi applied last
  static constexpr bool kPair = std::is_same<T, f16_t>::value;
  __device__ __forceinline__ void pair(const T* a, const Unused*, const Unused*, T* r) const {
    const _Float16 l = (_Float16)lo, h = (_Float16)hi;
    const f16x2_t m = __builtin_elementwise_minimum(
        __builtin_elementwise_maximum(f16x2_t{(_Float16)a[0], (_Float16)a[1]}, f16x2_t{l, l}), f16x2_t{h, h});
    r[0] = (T)m[0];
    r[1] = (T)m[1];
  }
  __device__ __forceinline__ T operator()(T a, Unused, Unused) const {
    M x = static_cast<M>(a);
    if constexpr (IsFloat<T>::value) {
      // the NaN-ignoring v_max / v_min and one select for a NaN input measured faster here than the
      // NaN-propagating pair (uniform bounds: their NaN tests are scalar)
      M r;
      if constexpr (sizeof(M) == 8) r = __builtin_fmin(__builtin_fmax(x, lo), hi);
      else r = __builtin_fminf(__builtin_fmaxf(x, lo), hi);  // hi applied last: lo > hi gives hi
      return static_cast<T>(x != x ? x : (lo != lo ? lo : (hi != hi ? hi : r)));
    } else {
      if (has_lo && x < lo) x = lo;
      if (has_hi && x > hi) x = hi;
      return static_cast<T>(x);
    }
  }
};

// ---- where: bit-exact select by element width ------------------------------------
template <typename U> struct WhereF {
  using out_t = U; using in0_t = uint8_t; using in1_t = U; using in2_t = U;
  static constexpr int NIN = 3;
  __device__ __forceinline__ U operator()(uint8_t c, U a, U b) const { return c ? a : b; }
};

// ---- copy / cast -------------------------------------------------------------------
struct Bool8 { uint8_t v; };

template <typename D, typename S> __device__ __forceinline__ D convert(S s) {
  if constexpr (__is_same(D, S)) {
    return s;
  } else if constexpr (__is_same(S, Bool8)) {
    return convert<D, uint8_t>(s.v ? 1 : 0);
  } else if constexpr (__is_same(D, Bool8)) {
    if constexpr (__is_same(S, bf16_t) || __is_same(S, f16_t)) return Bool8{(uint8_t)(static_cast<float>(s) != 0.f)};
    else return Bool8{(uint8_t)(s != S(0))};
  } else if constexpr (__is_same(S, bf16_t) || __is_same(S, f16_t)) {
    return convert<D, float>(static_cast<float>(s));
  } else if constexpr (__is_same(D, bf16_t) || __is_same(D, f16_t)) {
    return static_cast<D>(static_cast<float>(s));
  } else {
    return static_cast<D>(s);
  }
}
template <typename D, typename S> struct CastF {
  using out_t = D; using in0_t = S; using in1_t = Unused; using in2_t = Unused;
  static constexpr int NIN = 1;
  __device__ __forceinline__ D operator()(S a, Unused, Unused) const { return convert<D, S>(a); }
};

template <typename S> static int copy_from(const mi355_tensor* src, const mi355_tensor* dst, hipStream_t st) {
  const mi355_tensor* ins[1] = {src};
  switch (dst->dtype) {
    case MI355_F32: return launch_elementwise(CastF<float, S>{}, ins, dst, st, "mi355_copy");
    case MI355_F16: return launch_elementwise(CastF<f16_t, S>{}, ins, dst, st, "mi355_copy");
    case MI355_BF16: return launch_elementwise(CastF<bf16_t, S>{}, ins, dst, st, "mi355_copy");
    case MI355_F64: return launch_elementwise(CastF<double, S>{}, ins, dst, st, "mi355_copy");
    case MI355_I32: return launch_elementwise(CastF<int32_t, S>{}, ins, dst, st, "mi355_copy");
    case MI355_I64: return launch_elementwise(CastF<int64_t, S>{}, ins, dst, st, "mi355_copy");
    case MI355_I16: return launch_elementwise(CastF<int16_t, S>{}, ins, dst, st, "mi355_copy");
    case MI355_I8: return launch_elementwise(CastF<int8_t, S>{}, ins, dst, st, "mi355_copy");
    case MI355_U8: return launch_elementwise(CastF<uint8_t, S>{}, ins, dst, st, "mi355_copy");
    case MI355_BOOL: return launch_elementwise(CastF<Bool8, S>{}, ins, dst, st, "mi355_copy");
    default: return set_error(MI355_ERR_UNSUPPORTED, "mi355_copy: unsupported dst dtype %d", dst->dtype);
  }
}

// ---- transposing copy ------------------------------------------------------------
// dst[b][m][n] = src[b][n][m] for same-width elements when the source is unit-stride along m
// and the destination along n (a transposed view made dense, per batch).  64 x 64 tiles go
// through LDS so that both the reads and the writes of a wave are contiguous; the strided
// elementwise kernel reads such a source one scattered element per lane.
// grid = (ceil(N / 64), ceil(M / 64), batch), block = 256.
template <typename U>
__global__ __launch_bounds__(256) void transpose_copy_kernel(const U* __restrict__ src, U* __restrict__ dst, int64_t M,
                                                            int64_t N, int64_t src_n_stride, int64_t dst_m_stride,
                                                            int64_t src_b_stride, int64_t dst_b_stride) {
  __shared__ U tile[64][65];
  const int64_t n0 = (int64_t)blockIdx.x * 64, m0 = (int64_t)blockIdx.y * 64;
  const U* s = src + (int64_t)blockIdx.z * src_b_stride;
  U* d = dst + (int64_t)blockIdx.z * dst_b_stride;
  const int c = threadIdx.x % 64, r4 = threadIdx.x / 64;
#pragma unroll
  for (int p = 0; p < 16; ++p) {  // row n0 + r of the source view: 64 consecutive m
    const int r = p * 4 + r4;
    if (n0 + r < N && m0 + c < M) tile[r][c] = s[(n0 + r) * src_n_stride + m0 + c];
  }
  __syncthreads();
#pragma unroll
  for (int p = 0; p < 16; ++p) {  // row m0 + r of the destination: 64 consecutive n
    const int r = p * 4 + r4;
    if (m0 + r < M && n0 + c < N) d[(m0 + r) * dst_m_stride + n0 + c] = tile[c][r];
  }
}

// The same for 2- and 4-byte elements when both sides allow 16-byte accesses (M, N and both row
// pitches multiples of the vector length VL = 8 or 4, aligned bases): a thread moves VL elements
// per global access instead of one.  Source vectors (VL consecutive m of row n) land in an
// unpadded 64 x 64 tile whose 16-byte chunk index is XORed with n / VL; a destination vector (VL
// consecutive n of row m) is gathered with VL single-element LDS reads that, over a wave, touch
// distinct banks.
template <typename U>
__global__ __launch_bounds__(256) void transpose_copy_vec_kernel(const U* __restrict__ src, U* __restrict__ dst,
                                                                int64_t M, int64_t N, int64_t src_n_stride,
                                                                int64_t dst_m_stride, int64_t src_b_stride,
                                                                int64_t dst_b_stride) {
  constexpr int VL = 16 / sizeof(U), CH = 64 / VL, ROWS = 256 / CH;  // chunks per tile row, tile rows per pass
  __shared__ __attribute__((aligned(16))) U tile[64 * 64];
  const int64_t n0 = (int64_t)blockIdx.x * 64, m0 = (int64_t)blockIdx.y * 64;
  const U* s = src + (int64_t)blockIdx.z * src_b_stride;
  U* d = dst + (int64_t)blockIdx.z * dst_b_stride;
  const int ch = threadIdx.x % CH, r = threadIdx.x / CH;
#pragma unroll
  for (int p = 0; p < 64 / ROWS; ++p) {
    const int n = p * ROWS + r;
    if (n0 + n < N && m0 + ch * VL < M) {
      const u32x4 v = *reinterpret_cast<const u32x4*>(s + (n0 + n) * src_n_stride + m0 + ch * VL);
      *reinterpret_cast<u32x4*>(tile + n * 64 + ((ch ^ (n / VL)) * VL)) = v;
    }
  }
  __syncthreads();
#pragma unroll
  for (int p = 0; p < 64 / ROWS; ++p) {
    const int m = p * ROWS + r;
    if (m0 + m < M && n0 + ch * VL < N) {
      Vec<U> v;
#pragma unroll
      for (int j = 0; j < VL; ++j) v.v[j] = tile[(ch * VL + j) * 64 + (((m / VL) ^ ch) * VL) + (m % VL)];
      store_vec(d + (m0 + m) * dst_m_stride + n0 + ch * VL, v);
    }
  }
}

// True (and the copy enqueued) when src -> dst is such a transposition.
template <typename U>
static bool try_transpose_copy(const mi355_tensor* src, const mi355_tensor* dst, hipStream_t st, int* rc) {
  const int64_t* strides[2] = {src->strides, dst->strides};
  const Dims<2> d = collapse_dims<2>(dst->ndim, dst->sizes, strides);
  if (d.ndim != 2 && d.ndim != 3) return false;
  const int im = d.ndim - 2, in = d.ndim - 1;
  const int64_t M = d.sizes[im], N = d.sizes[in];
  // destination row-major over (m, n), source unit-stride along m
  if (d.strides[1][in] != 1 || d.strides[0][im] != 1 || d.strides[0][in] < M || d.strides[1][im] < N) return false;
  if (M < 16 || N < 16) return false;
  const int64_t batch = d.ndim == 3 ? d.sizes[0] : 1;
  if (batch > 65535 || (M + 63) / 64 > 65535) return false;
  const dim3 grid((unsigned)((N + 63) / 64), (unsigned)((M + 63) / 64), (unsigned)batch);
  const int64_t sb = d.ndim == 3 ? d.strides[0][0] : 0, db = d.ndim == 3 ? d.strides[1][0] : 0;
  if constexpr (sizeof(U) == 2 || sizeof(U) == 4) {
    constexpr int VL = 16 / sizeof(U);
    if (M % VL == 0 && N % VL == 0 && d.strides[0][in] % VL == 0 && d.strides[1][im] % VL == 0 && sb % VL == 0 &&
        db % VL == 0 && aligned16(src->data) && aligned16(dst->data)) {
      hipLaunchKernelGGL((transpose_copy_vec_kernel<U>), grid, dim3(256), 0, st, (const U*)src->data, (U*)dst->data, M, N,
                         d.strides[0][in], d.strides[1][im], sb, db);
      *rc = check_launch("mi355_copy(transpose, vectors)");
      return true;
    }
  }
  hipLaunchKernelGGL((transpose_copy_kernel<U>), grid, dim3(256), 0, st, (const U*)src->data, (U*)dst->data, M, N,
                     d.strides[0][in], d.strides[1][im], sb, db);
  *rc = check_launch("mi355_copy(transpose)");
  return true;
}

}  // namespace mi355

using namespace mi355;

extern "C" int mi355_binary(int op, const mi355_tensor* a, const mi355_tensor* b, double alpha_f,
                            int64_t alpha_i, const mi355_tensor* out, void* stream) {
  int rc;
  if ((rc = check_tensor(a, "mi355_binary", "a"))) return rc;
  if ((rc = check_tensor(b, "mi355_binary", "b"))) return rc;
  if ((rc = check_tensor(out, "mi355_binary", "out"))) return rc;
  const mi355_tensor* ins[2] = {a, b};
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (out->dtype == MI355_F32 && a->dtype != b->dtype && (op == MI355_ADD || op == MI355_MUL)) {
    // add / mul of an fp32 and an f16 / bf16 operand into fp32
    auto run = [&](auto ta, auto tb) -> int {
      using TA = decltype(ta);
      using TB = decltype(tb);
      if (op == MI355_ADD) {
        AddMixF<TA, TB> f;
        f.alpha = static_cast<float>(alpha_f);
        return launch_elementwise(f, ins, out, st, "mi355_binary(add, mixed)");
      }
      return launch_elementwise(MulMixF<TA, TB>{}, ins, out, st, "mi355_binary(mul, mixed)");
    };
    if (a->dtype == MI355_F32 && b->dtype == MI355_F16) return run(float{}, f16_t{});
    if (a->dtype == MI355_F32 && b->dtype == MI355_BF16) return run(float{}, bf16_t{});
    if (a->dtype == MI355_F16 && b->dtype == MI355_F32) return run(f16_t{}, float{});
    if (a->dtype == MI355_BF16 && b->dtype == MI355_F32) return run(bf16_t{}, float{});
  }
  MI355_REQUIRE(a->dtype == out->dtype && b->dtype == out->dtype,
                "mi355_binary: operands must already have the output dtype (%s, %s -> %s), except fp32 with f16 / bf16 for add and mul",
                dtype_name(a->dtype), dtype_name(b->dtype), dtype_name(out->dtype));
  MI355_DISPATCH_NUMERIC(out->dtype, "mi355_binary", {
    using M = typename OpMath<T>::type;
    switch (op) {
      case MI355_ADD: {
        AddF<T> f;
        f.alpha = IsFloat<T>::value ? static_cast<M>(alpha_f) : static_cast<M>(alpha_i);
        return launch_elementwise(f, ins, out, st, "mi355_binary(add)");
      }
      case MI355_MUL: return launch_elementwise(MulF<T>{}, ins, out, st, "mi355_binary(mul)");
      case MI355_MAXIMUM: return launch_elementwise(MaximumF<T>{}, ins, out, st, "mi355_binary(maximum)");
      case MI355_MINIMUM: return launch_elementwise(MinimumF<T>{}, ins, out, st, "mi355_binary(minimum)");
      default: return set_error(MI355_ERR_INVALID, "mi355_binary: unknown op %d", op);
    }
  });
  return MI355_OK;
}

extern "C" int mi355_unary(int op, const mi355_tensor* x, int bounds, double lo_f, double hi_f,
                           int64_t lo_i, int64_t hi_i, const mi355_tensor* out, void* stream) {
  int rc;
  if ((rc = check_tensor(x, "mi355_unary", "x"))) return rc;
  if ((rc = check_tensor(out, "mi355_unary", "out"))) return rc;
  MI355_REQUIRE(x->dtype == out->dtype, "mi355_unary: x and out dtypes differ (%s vs %s)",
                dtype_name(x->dtype), dtype_name(out->dtype));
  const mi355_tensor* ins[1] = {x};
  hipStream_t st = static_cast<hipStream_t>(stream);
  MI355_DISPATCH_NUMERIC(out->dtype, "mi355_unary", {
    using M = typename OpMath<T>::type;
    switch (op) {
      case MI355_RELU: return launch_elementwise(ReluF<T>{}, ins, out, st, "mi355_unary(relu)");
      case MI355_CLAMP: {
        MI355_REQUIRE((bounds & 3) != 0, "mi355_unary(clamp): at least one of lo, hi must be given");
        ClampF<T> f;
        f.has_lo = bounds & 1;
        f.has_hi = bounds & 2;
        f.lo = IsFloat<T>::value ? (f.has_lo ? static_cast<M>(lo_f) : static_cast<M>(-INFINITY)) : static_cast<M>(lo_i);
        f.hi = IsFloat<T>::value ? (f.has_hi ? static_cast<M>(hi_f) : static_cast<M>(INFINITY)) : static_cast<M>(hi_i);
        return launch_elementwise(f, ins, out, st, "mi355_unary(clamp)");
      }
      default: return set_error(MI355_ERR_INVALID, "mi355_unary: unknown op %d", op);
    }
  });
  return MI355_OK;
}

extern "C" int mi355_where(const mi355_tensor* cond, const mi355_tensor* a, const mi355_tensor* b,
                           const mi355_tensor* out, void* stream) {
  int rc;
  if ((rc = check_tensor(cond, "mi355_where", "cond"))) return rc;
  if ((rc = check_tensor(a, "mi355_where", "a"))) return rc;
  if ((rc = check_tensor(b, "mi355_where", "b"))) return rc;
  if ((rc = check_tensor(out, "mi355_where", "out"))) return rc;
  MI355_REQUIRE(cond->dtype == MI355_BOOL || cond->dtype == MI355_U8,
                "mi355_where: condition must be bool or u8, got %s", dtype_name(cond->dtype));
  MI355_REQUIRE(a->dtype == out->dtype && b->dtype == out->dtype,
                "mi355_where: a and b must already have the output dtype");
  const mi355_tensor* ins[3] = {cond, a, b};
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (dtype_size(out->dtype)) {
    case 1: return launch_elementwise(WhereF<uint8_t>{}, ins, out, st, "mi355_where");
    case 2: return launch_elementwise(WhereF<uint16_t>{}, ins, out, st, "mi355_where");
    case 4: return launch_elementwise(WhereF<uint32_t>{}, ins, out, st, "mi355_where");
    case 8: return launch_elementwise(WhereF<uint64_t>{}, ins, out, st, "mi355_where");
    default: return set_error(MI355_ERR_UNSUPPORTED, "mi355_where: unsupported dtype");
  }
}

// min(max(x, lo), hi) with the NaN and signed-zero rules of the two binary ops, in one pass.
template <typename T> struct ClampTensorF {
  using out_t = T; using in0_t = T; using in1_t = T; using in2_t = T;
  static constexpr int NIN = 3;
  static constexpr bool kPair = std::is_same<T, f16_t>::value;
  __device__ __forceinline__ void pair(const T* x, const T* lo, const T* hi, T* r) const {
    const f16x2_t m = __builtin_elementwise_minimum(
        __builtin_elementwise_maximum(f16x2_t{(_Float16)x[0], (_Float16)x[1]}, f16x2_t{(_Float16)lo[0], (_Float16)lo[1]}),
        f16x2_t{(_Float16)hi[0], (_Float16)hi[1]});
    r[0] = (T)m[0];
    r[1] = (T)m[1];
  }
  __device__ __forceinline__ T operator()(T x, T lo, T hi) const {
    if constexpr (IsFloat<T>::value) {
      using M = typename OpMath<T>::type;
      const M v = static_cast<M>(x), l = static_cast<M>(lo), h = static_cast<M>(hi);
      return static_cast<T>(nan_min(nan_max(v, l), h));
    } else {
      return MinimumF<T>{}(MaximumF<T>{}(x, lo, Unused{}), hi, Unused{});
    }
  }
};

extern "C" int mi355_clamp_tensor(const mi355_tensor* x, const mi355_tensor* lo, const mi355_tensor* hi,
                                  const mi355_tensor* out, void* stream) {
  int rc;
  if ((rc = check_tensor(x, "mi355_clamp_tensor", "x"))) return rc;
  if ((rc = check_tensor(lo, "mi355_clamp_tensor", "lo"))) return rc;
  if ((rc = check_tensor(hi, "mi355_clamp_tensor", "hi"))) return rc;
  if ((rc = check_tensor(out, "mi355_clamp_tensor", "out"))) return rc;
  MI355_REQUIRE(x->dtype == out->dtype && lo->dtype == out->dtype && hi->dtype == out->dtype,
                "mi355_clamp_tensor: x, lo and hi must already have the output dtype");
  const mi355_tensor* ins[3] = {x, lo, hi};
  hipStream_t st = static_cast<hipStream_t>(stream);
  MI355_DISPATCH_NUMERIC(out->dtype, "mi355_clamp_tensor",
                         { return launch_elementwise(ClampTensorF<T>{}, ins, out, st, "mi355_clamp_tensor"); });
  return MI355_OK;
}

extern "C" int mi355_copy(const mi355_tensor* src, const mi355_tensor* dst, void* stream) {
  int rc;
  if ((rc = check_tensor(src, "mi355_copy", "src"))) return rc;
  if ((rc = check_tensor(dst, "mi355_copy", "dst"))) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (src->dtype == dst->dtype) {  // same dtype: move raw bits by element width
    const mi355_tensor* ins[1] = {src};
    if (same_shape(src, dst) && numel(dst) > 0) {
      bool done = false;
      switch (dtype_size(src->dtype)) {
        case 1: done = try_transpose_copy<uint8_t>(src, dst, st, &rc); break;
        case 2: done = try_transpose_copy<uint16_t>(src, dst, st, &rc); break;
        case 4: done = try_transpose_copy<uint32_t>(src, dst, st, &rc); break;
        case 8: done = try_transpose_copy<uint64_t>(src, dst, st, &rc); break;
      }
      if (done) return rc;
    }
    switch (dtype_size(src->dtype)) {
      case 1: return launch_elementwise(CastF<uint8_t, uint8_t>{}, ins, dst, st, "mi355_copy");
      case 2: return launch_elementwise(CastF<uint16_t, uint16_t>{}, ins, dst, st, "mi355_copy");
      case 4: return launch_elementwise(CastF<uint32_t, uint32_t>{}, ins, dst, st, "mi355_copy");
      case 8: return launch_elementwise(CastF<uint64_t, uint64_t>{}, ins, dst, st, "mi355_copy");
    }
  }
  switch (src->dtype) {
    case MI355_F32: return copy_from<float>(src, dst, st);
    case MI355_F16: return copy_from<f16_t>(src, dst, st);
    case MI355_BF16: return copy_from<bf16_t>(src, dst, st);
    case MI355_F64: return copy_from<double>(src, dst, st);
    case MI355_I32: return copy_from<int32_t>(src, dst, st);
    case MI355_I64: return copy_from<int64_t>(src, dst, st);
    case MI355_I16: return copy_from<int16_t>(src, dst, st);
    case MI355_I8: return copy_from<int8_t>(src, dst, st);
    case MI355_U8: return copy_from<uint8_t>(src, dst, st);
    case MI355_BOOL: return copy_from<Bool8>(src, dst, st);
    default: return set_error(MI355_ERR_UNSUPPORTED, "mi355_copy: unsupported src dtype %d", src->dtype);
  }
}
