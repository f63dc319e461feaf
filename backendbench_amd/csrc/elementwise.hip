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
template <typename T> struct MaximumF {
  using out_t = T; using in0_t = T; using in1_t = T; using in2_t = Unused;
  static constexpr int NIN = 2;
  using M = typename OpMath<T>::type;
  __device__ __forceinline__ T operator()(T a, T b, Unused) const {
    const M x = static_cast<M>(a), y = static_cast<M>(b);
    if constexpr (IsFloat<T>::value) {
      if (x != x) return a;
      if (y != y) return b;
      if (x == y) return __builtin_signbit(x) ? b : a;  // IEEE 754-2019 maximum: +0 above -0
    }
    return x > y ? a : b;
  }
};

template <typename T> struct MinimumF {
  using out_t = T; using in0_t = T; using in1_t = T; using in2_t = Unused;
  static constexpr int NIN = 2;
  using M = typename OpMath<T>::type;
  __device__ __forceinline__ T operator()(T a, T b, Unused) const {
    const M x = static_cast<M>(a), y = static_cast<M>(b);
    if constexpr (IsFloat<T>::value) {
      if (x != x) return a;
      if (y != y) return b;
      if (x == y) return __builtin_signbit(x) ? a : b;  // IEEE 754-2019 minimum: -0 below +0
    }
    return x < y ? a : b;
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
  M lo, hi;
  bool has_lo, has_hi;
  __device__ __forceinline__ T operator()(T a, Unused, Unused) const {
    M x = static_cast<M>(a);
    if constexpr (IsFloat<T>::value) {
      if (x != x) return a;
      if (has_lo && lo != lo) return static_cast<T>(lo);  // a NaN bound makes everything NaN
      if (has_hi && hi != hi) return static_cast<T>(hi);
    }
    if (has_lo && x < lo) x = lo;
    if (has_hi && x > hi) x = hi;  // applied last: lo > hi gives hi
    return static_cast<T>(x);
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

}  // namespace mi355

using namespace mi355;

extern "C" int mi355_binary(int op, const mi355_tensor* a, const mi355_tensor* b, double alpha_f,
                            int64_t alpha_i, const mi355_tensor* out, void* stream) {
  int rc;
  if ((rc = check_tensor(a, "mi355_binary", "a"))) return rc;
  if ((rc = check_tensor(b, "mi355_binary", "b"))) return rc;
  if ((rc = check_tensor(out, "mi355_binary", "out"))) return rc;
  MI355_REQUIRE(a->dtype == out->dtype && b->dtype == out->dtype,
                "mi355_binary: operands must already have the output dtype (%s, %s -> %s)",
                dtype_name(a->dtype), dtype_name(b->dtype), dtype_name(out->dtype));
  const mi355_tensor* ins[2] = {a, b};
  hipStream_t st = static_cast<hipStream_t>(stream);
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
        f.lo = IsFloat<T>::value ? static_cast<M>(lo_f) : static_cast<M>(lo_i);
        f.hi = IsFloat<T>::value ? static_cast<M>(hi_f) : static_cast<M>(hi_i);
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

extern "C" int mi355_copy(const mi355_tensor* src, const mi355_tensor* dst, void* stream) {
  int rc;
  if ((rc = check_tensor(src, "mi355_copy", "src"))) return rc;
  if ((rc = check_tensor(dst, "mi355_copy", "dst"))) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (src->dtype == dst->dtype) {  // same dtype: move raw bits by element width
    const mi355_tensor* ins[1] = {src};
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
