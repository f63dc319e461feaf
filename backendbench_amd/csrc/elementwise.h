// Elementwise launch framework: one functor type F describes an op
//   F::out_t, F::in0_t, F::in1_t, F::in2_t, F::NIN, out_t operator()(in0_t, in1_t, in2_t)
// and three kernel shapes cover every layout:
//   flat      all operands share one dense (possibly permuted) layout: 1-D pass, one
//             contiguous 16 KB tile per operand per block, non-temporal 128-bit accesses;
//   strided   any strides/broadcast, index split with multiply-shift division; vectorised
//             along the innermost dim when every operand is unit-stride or broadcast there;
//   strided64 the same with 64-bit index math for > 2^31 work items.
#pragma once
#include <type_traits>
#include "common.h"

namespace mi355 {

template <typename T, int N> struct alignas(sizeof(T) * N) VecN { T v[N]; };

template <typename T, int N> __device__ __forceinline__ VecN<T, N> ld(const T* p) {
  return *reinterpret_cast<const VecN<T, N>*>(p);
}
template <typename T, int N> __device__ __forceinline__ void st(T* p, const VecN<T, N>& v) {
  *reinterpret_cast<VecN<T, N>*>(p) = v;
}
// Streaming (non-temporal) forms for data touched exactly once: measured on MI355X, a
// block-contiguous copy with non-temporal loads and stores runs at 5.8-6.4 TB/s against
// 5.3-5.8 TB/s with plain accesses.  Vectors wider than 16 bytes are moved in 16-byte pieces.
template <int BYTES> struct RawVec { typedef uint32_t type __attribute__((ext_vector_type(BYTES / 4))); };
template <> struct RawVec<1> { typedef uint8_t type; };
template <> struct RawVec<2> { typedef uint16_t type; };
template <typename T, int N> __device__ __forceinline__ VecN<T, N> ld_nt(const T* p) {
  constexpr int B = sizeof(T) * N;
  if constexpr (B > 16) {
    VecN<T, N> r;
    using R = typename RawVec<16>::type;
    R* dst = reinterpret_cast<R*>(&r);
#pragma unroll
    for (int i = 0; i < B / 16; ++i) dst[i] = __builtin_nontemporal_load(reinterpret_cast<const R*>(p) + i);
    return r;
  } else {
    using R = typename RawVec<B>::type;
    return __builtin_bit_cast(VecN<T, N>, __builtin_nontemporal_load(reinterpret_cast<const R*>(p)));
  }
}
template <typename T, int N> __device__ __forceinline__ void st_nt(T* p, const VecN<T, N>& v) {
  constexpr int B = sizeof(T) * N;
  if constexpr (B > 16) {
    using R = typename RawVec<16>::type;
    const R* src = reinterpret_cast<const R*>(&v);
#pragma unroll
    for (int i = 0; i < B / 16; ++i) __builtin_nontemporal_store(src[i], reinterpret_cast<R*>(p) + i);
  } else {
    using R = typename RawVec<B>::type;
    __builtin_nontemporal_store(__builtin_bit_cast(R, v), reinterpret_cast<R*>(p));
  }
}

template <typename F> struct EwTraits {
  static constexpr int NIN = F::NIN;
  static constexpr int NT = NIN + 1;
  static constexpr int max_size() {
    int m = sizeof(typename F::out_t);
    if (NIN > 0 && (int)sizeof(typename F::in0_t) > m) m = sizeof(typename F::in0_t);
    if (NIN > 1 && (int)sizeof(typename F::in1_t) > m) m = sizeof(typename F::in1_t);
    if (NIN > 2 && (int)sizeof(typename F::in2_t) > m) m = sizeof(typename F::in2_t);
    return m;
  }
  static constexpr int V = 16 / max_size();  // elements per thread-vector
};

struct EwPtrs {
  const void* in[3];
  void* out;
};

// A functor with `static constexpr bool kPair = true` also has pair(a, b, c, r): the same operation on two
// neighbouring elements at once (packed f16: v_pk_maximum3_f16 / v_pk_minimum3_f16 take two elements per
// instruction and no round trip through fp32).
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
template <typename F, typename = void> struct HasPair : std::false_type {};
template <typename F> struct HasPair<F, std::enable_if_t<F::kPair>> : std::true_type {};

template <typename F, int V, typename VA, typename VB, typename VC>
__device__ __forceinline__ VecN<typename F::out_t, V> ew_apply(const F& f, const VA& a, const VB& b,
                                                              const VC& c) {
  VecN<typename F::out_t, V> r;
  if constexpr (HasPair<F>::value && V % 2 == 0) {
#pragma unroll
    for (int j = 0; j < V; j += 2) f.pair(a.v + j, b.v + j, c.v + j, r.v + j);
  } else {
#pragma unroll
    for (int j = 0; j < V; ++j) r.v[j] = f(a.v[j], b.v[j], c.v[j]);
  }
  return r;
}

// ---------------------------------------------------------------- flat
constexpr int kEwBlock = 256;
constexpr int kEwUnroll = 4;

template <typename T, int V>
__device__ __forceinline__ VecN<T, V> ld_or_splat(const T* p, bool splat) {
  if (V == 1 || splat) {
    VecN<T, V> r;
    const T s = *p;
#pragma unroll
    for (int j = 0; j < V; ++j) r.v[j] = s;
    return r;
  }
  return ld<T, V>(p);
}

// One block = one contiguous tile of kEwUnroll x 256 vectors per operand (16 KB each for
// 128-bit vectors): all loads of the tile are issued before the first store, and the tile is a
// single DRAM-friendly span — a grid-stride walk with the same number of loads in flight
// measured 10-25 % slower on this chip.
// SC: some inputs are single values broadcast over the whole output (bit t of scalar_mask): they
// are read once per thread and never indexed.
template <typename F, bool SC>
__global__ __launch_bounds__(kEwBlock) void ew_flat_kernel(F f, EwPtrs p, int64_t n, uint32_t scalar_mask) {
  using TO = typename F::out_t;
  using T0 = typename F::in0_t;
  using T1 = typename F::in1_t;
  using T2 = typename F::in2_t;
  constexpr int V = EwTraits<F>::V;
  constexpr int NIN = F::NIN;
  const T0* a = static_cast<const T0*>(p.in[0]);
  const T1* b = static_cast<const T1*>(p.in[1]);
  const T2* c = static_cast<const T2*>(p.in[2]);
  TO* o = static_cast<TO*>(p.out);
  const bool sa = SC && (scalar_mask & 1u), sb = SC && NIN > 1 && (scalar_mask & 2u), sc = SC && NIN > 2 && (scalar_mask & 4u);
  VecN<T0, V> ka;
  VecN<T1, V> kb;
  VecN<T2, V> kc;
  if constexpr (SC) {
    if (sa) ka = ld_or_splat<T0, V>(a, true);
    if constexpr (NIN > 1) if (sb) kb = ld_or_splat<T1, V>(b, true);
    if constexpr (NIN > 2) if (sc) kc = ld_or_splat<T2, V>(c, true);
  }

  const int64_t nvec = n / V;
  constexpr int64_t TILE = (int64_t)kEwBlock * kEwUnroll;
  for (int64_t base = (int64_t)blockIdx.x * TILE; base < nvec; base += (int64_t)gridDim.x * TILE) {
    const int64_t i0 = base + threadIdx.x;
    if (base + TILE <= nvec) {
      VecN<T0, V> va[kEwUnroll];
      VecN<T1, V> vb[kEwUnroll];
      VecN<T2, V> vc[kEwUnroll];
#pragma unroll
      for (int u = 0; u < kEwUnroll; ++u) {
        const int64_t e = (i0 + u * kEwBlock) * V;
        va[u] = sa ? ka : ld_nt<T0, V>(a + e);
        if constexpr (NIN > 1) vb[u] = sb ? kb : ld_nt<T1, V>(b + e);
        if constexpr (NIN > 2) vc[u] = sc ? kc : ld_nt<T2, V>(c + e);
      }
#pragma unroll
      for (int u = 0; u < kEwUnroll; ++u) {
        const int64_t e = (i0 + u * kEwBlock) * V;
        st_nt<TO, V>(o + e, ew_apply<F, V>(f, va[u], vb[u], vc[u]));
      }
    } else {
      for (int64_t i = i0; i < nvec; i += kEwBlock) {
        const int64_t e = i * V;
        VecN<T0, V> va = sa ? ka : ld_nt<T0, V>(a + e);
        VecN<T1, V> vb;
        VecN<T2, V> vc;
        if constexpr (NIN > 1) vb = sb ? kb : ld_nt<T1, V>(b + e);
        if constexpr (NIN > 2) vc = sc ? kc : ld_nt<T2, V>(c + e);
        st_nt<TO, V>(o + e, ew_apply<F, V>(f, va, vb, vc));
      }
    }
  }
  // ragged tail (< V elements), first threads of block 0
  if (blockIdx.x == 0) {
    const int64_t e = nvec * V + threadIdx.x;
    if (e < n) {
      T1 tb{};
      T2 tc{};
      if constexpr (NIN > 1) tb = b[sb ? 0 : e];
      if constexpr (NIN > 2) tc = c[sc ? 0 : e];
      o[e] = f(a[sa ? 0 : e], tb, tc);
    }
  }
}

// Same pass with scalar accesses, for operands whose base is not vector-aligned.
template <typename F>
__global__ __launch_bounds__(kEwBlock) void ew_flat_scalar_kernel(F f, EwPtrs p, int64_t n) {
  using TO = typename F::out_t;
  using T0 = typename F::in0_t;
  using T1 = typename F::in1_t;
  using T2 = typename F::in2_t;
  constexpr int NIN = F::NIN;
  const T0* a = static_cast<const T0*>(p.in[0]);
  const T1* b = static_cast<const T1*>(p.in[1]);
  const T2* c = static_cast<const T2*>(p.in[2]);
  TO* o = static_cast<TO*>(p.out);
  const int64_t stride = (int64_t)gridDim.x * kEwBlock;
  for (int64_t e = (int64_t)blockIdx.x * kEwBlock + threadIdx.x; e < n; e += stride) {
    T1 sb{};
    T2 sc{};
    if constexpr (NIN > 1) sb = b[e];
    if constexpr (NIN > 2) sc = c[e];
    o[e] = f(a[e], sb, sc);
  }
}

// ---------------------------------------------------------------- strided
// n / d for n < 2^31 as (umulhi(n, m) + n) >> s.
struct FastDiv {
  uint32_t d, m, s;
};
inline FastDiv make_fastdiv(uint32_t d) {
  FastDiv f;
  f.d = d;
  f.s = 0;
  while ((1ull << f.s) < d) ++f.s;
  f.m = (uint32_t)(((1ull << 32) * ((1ull << f.s) - d)) / d + 1);
  return f;
}

template <int NT> struct StridedArgs {
  int32_t ndim;
  uint32_t splat_mask;  // bit t: input t is broadcast along the vectorised inner dim
  FastDiv div[MI355_MAX_DIMS];
  int64_t sizes[MI355_MAX_DIMS];
  int64_t strides[NT][MI355_MAX_DIMS];  // element strides; [NT-1] is the output
};


// One work item = V consecutive elements of the innermost dim (V == 1: one element).  A block
// takes U * kEwBlock consecutive work items, U per thread: the U index splits and loads are all
// issued before the first store, as in the flat kernel.
template <typename F, int NT, bool WIDE>
__device__ __forceinline__ void ew_split_index(const StridedArgs<NT>& a, int64_t lin, int64_t (&off)[NT]) {
#pragma unroll
  for (int t = 0; t < NT; ++t) off[t] = 0;
  if constexpr (WIDE) {
    int64_t rem = lin;
    for (int k = a.ndim - 1; k >= 0; --k) {
      const int64_t q = rem / a.sizes[k];
      const int64_t idx = rem - q * a.sizes[k];
      rem = q;
#pragma unroll
      for (int t = 0; t < NT; ++t) off[t] += idx * a.strides[t][k];
    }
  } else {
    uint32_t rem = (uint32_t)lin;
    for (int k = a.ndim - 1; k >= 0; --k) {
      const FastDiv d = a.div[k];
      const uint32_t q = (uint32_t)(((uint64_t)__umulhi(rem, d.m) + rem) >> d.s);
      const uint32_t idx = rem - q * d.d;
      rem = q;
#pragma unroll
      for (int t = 0; t < NT; ++t) off[t] += (int64_t)idx * a.strides[t][k];
    }
  }
}

template <typename F, int V, bool WIDE, int U>
__global__ __launch_bounds__(kEwBlock) void ew_strided_kernel(F f, EwPtrs p,
                                                               StridedArgs<F::NIN + 1> a,
                                                               int64_t total) {
  using TO = typename F::out_t;
  using T0 = typename F::in0_t;
  using T1 = typename F::in1_t;
  using T2 = typename F::in2_t;
  constexpr int NIN = F::NIN;
  constexpr int NT = NIN + 1;
  const int64_t stride = (int64_t)gridDim.x * kEwBlock * U;
  for (int64_t base = (int64_t)blockIdx.x * kEwBlock * U + threadIdx.x; base < total; base += stride) {
    VecN<T0, V> va[U];
    VecN<T1, V> vb[U];
    VecN<T2, V> vc[U];
    int64_t out_off[U];
#pragma unroll
    for (int j = 0; j < U; ++j) {
      const int64_t lin = base + (int64_t)j * kEwBlock;
      if (lin < total) {
        int64_t off[NT];
        ew_split_index<F, NT, WIDE>(a, lin, off);
        out_off[j] = off[NT - 1];
        va[j] = ld_or_splat<T0, V>(static_cast<const T0*>(p.in[0]) + off[0], a.splat_mask & 1u);
        if constexpr (NIN > 1)
          vb[j] = ld_or_splat<T1, V>(static_cast<const T1*>(p.in[1]) + off[1], a.splat_mask & 2u);
        if constexpr (NIN > 2)
          vc[j] = ld_or_splat<T2, V>(static_cast<const T2*>(p.in[2]) + off[2], a.splat_mask & 4u);
      }
    }
#pragma unroll
    for (int j = 0; j < U; ++j)
      if (base + (int64_t)j * kEwBlock < total)
        st_nt<TO, V>(static_cast<TO*>(p.out) + out_off[j], ew_apply<F, V>(f, va[j], vb[j], vc[j]));
  }
}

// Dense row-major output whose innermost extent is no multiple of the vector (a 197-token
// attention map plus a [B,1,1,197] mask): the strided kernel would fall back to single
// elements.  Here one work item is V consecutive elements of the flat output: inputs laid out
// like the output (flat_mask bit t) are read as one aligned vector, the others element by
// element along a coordinate walk (the innermost index steps, a carry into the outer dims
// re-splits the flat index: once per row), and the result leaves as one aligned vector store.
template <typename F, int V>
__global__ __launch_bounds__(kEwBlock) void ew_dense_out_kernel(F f, EwPtrs p, StridedArgs<F::NIN + 1> a, int64_t n,
                                                                 uint32_t flat_mask) {
  using TO = typename F::out_t;
  using T0 = typename F::in0_t;
  using T1 = typename F::in1_t;
  using T2 = typename F::in2_t;
  constexpr int NIN = F::NIN;
  constexpr int NT = NIN + 1;
  const int last = a.ndim - 1;
  const int64_t items = (n + V - 1) / V;
  const T0* in0 = static_cast<const T0*>(p.in[0]);
  const T1* in1 = static_cast<const T1*>(p.in[1]);
  const T2* in2 = static_cast<const T2*>(p.in[2]);
  for (int64_t item = (int64_t)blockIdx.x * kEwBlock + threadIdx.x; item < items; item += (int64_t)gridDim.x * kEwBlock) {
    const int64_t e0 = item * V;
    const bool full = e0 + V <= n;
    VecN<T0, V> va;
    VecN<T1, V> vb;
    VecN<T2, V> vc;
    if (full) {
      if (flat_mask & 1u) va = ld_nt<T0, V>(in0 + e0);
      if constexpr (NIN > 1) if (flat_mask & 2u) vb = ld_nt<T1, V>(in1 + e0);
      if constexpr (NIN > 2) if (flat_mask & 4u) vc = ld_nt<T2, V>(in2 + e0);
    }
    int64_t off[NT];
    ew_split_index<F, NT, false>(a, e0, off);
    int64_t inner = 0;  // index along the innermost dim = e0 % sizes[last]
    {
      const FastDiv d = a.div[last];
      const uint32_t q = (uint32_t)(((uint64_t)__umulhi((uint32_t)e0, d.m) + (uint32_t)e0) >> d.s);
      inner = (uint32_t)e0 - q * d.d;
    }
#pragma unroll
    for (int j = 0; j < V; ++j) {
      if (e0 + j < n) {
        if (!full || !(flat_mask & 1u)) va.v[j] = in0[off[0]];
        if constexpr (NIN > 1) if (!full || !(flat_mask & 2u)) vb.v[j] = in1[off[1]];
        if constexpr (NIN > 2) if (!full || !(flat_mask & 4u)) vc.v[j] = in2[off[2]];
      }
      if (j + 1 < V) {
        if (++inner == a.sizes[last]) {
          inner = 0;
          ew_split_index<F, NT, false>(a, e0 + j + 1, off);
        } else {
#pragma unroll
          for (int t = 0; t < NIN; ++t) off[t] += a.strides[t][last];
        }
      }
    }
    const VecN<TO, V> r = ew_apply<F, V>(f, va, vb, vc);
    TO* o = static_cast<TO*>(p.out) + e0;
    if (full) {
      st_nt<TO, V>(o, r);
    } else {
#pragma unroll
      for (int j = 0; j < V; ++j)
        if (e0 + j < n) o[j] = r.v[j];
    }
  }
}

// ---------------------------------------------------------------- host launcher
template <typename F>
int launch_elementwise(const F& f, const mi355_tensor* const* ins, const mi355_tensor* out,
                       hipStream_t stream, const char* name) {
  constexpr int NIN = F::NIN;
  constexpr int NT = NIN + 1;
  constexpr int V = EwTraits<F>::V;
  const size_t esz[4] = {sizeof(typename F::in0_t), sizeof(typename F::in1_t),
                         sizeof(typename F::in2_t), sizeof(typename F::out_t)};
  for (int t = 0; t < NIN; ++t)
    if (!same_shape(ins[t], out))
      return set_error(MI355_ERR_INVALID, "%s: operand %d shape differs from output shape", name, t);
  const int64_t n = numel(out);
  if (n == 0) return MI355_OK;

  const mi355_tensor* ts[NT];
  for (int t = 0; t < NIN; ++t) ts[t] = ins[t];
  ts[NIN] = out;
  EwPtrs p{};
  for (int t = 0; t < NIN; ++t) p.in[t] = ins[t]->data;
  p.out = out->data;
  const int max_blocks = kNumCU * 8;

  // Inputs that are one value broadcast over the whole output (0-d operands, expanded scalars)
  // do not constrain the layout: the flat kernel reads them once.
  uint32_t scalar_mask = 0;
  const mi355_tensor* laid[NT];
  int nlaid = 0;
  for (int t = 0; t < NIN; ++t) {
    bool scalar = n > 1;
    for (int i = 0; i < ins[t]->ndim && scalar; ++i)
      if (ins[t]->sizes[i] > 1 && ins[t]->strides[i] != 0) scalar = false;
    if (scalar) scalar_mask |= 1u << t;
    else laid[nlaid++] = ins[t];
  }
  laid[nlaid++] = out;
  if (same_dense_layout(laid, nlaid)) {
    bool vec_ok = (reinterpret_cast<uintptr_t>(out->data) % (esz[3] * V)) == 0;
    for (int t = 0; t < NIN; ++t)
      if (!(scalar_mask & (1u << t)))
        vec_ok = vec_ok && (reinterpret_cast<uintptr_t>(ins[t]->data) % (esz[t] * V)) == 0;
    if (vec_ok) {
      const int grid = grid_for((n + V - 1) / V, kEwBlock * kEwUnroll, 1 << 30);
      if (scalar_mask) hipLaunchKernelGGL((ew_flat_kernel<F, true>), dim3(grid), dim3(kEwBlock), 0, stream, f, p, n, scalar_mask);
      else hipLaunchKernelGGL((ew_flat_kernel<F, false>), dim3(grid), dim3(kEwBlock), 0, stream, f, p, n, 0u);
      return check_launch(name);
    }
    if (!scalar_mask) {
      const int grid = grid_for(n, kEwBlock, max_blocks);
      hipLaunchKernelGGL(ew_flat_scalar_kernel<F>, dim3(grid), dim3(kEwBlock), 0, stream, f, p, n);
      return check_launch(name);
    }
  }

  // Output stride for broadcast-free iteration must be real (no stride-0 output dims).
  for (int i = 0; i < out->ndim; ++i)
    if (out->sizes[i] > 1 && out->strides[i] == 0)
      return set_error(MI355_ERR_INVALID, "%s: output has a broadcast (stride 0) dim", name);

  // Walk the dims in the memory order of the output (largest stride first): a channels-last
  // output then has its channels innermost, where they are unit-stride, instead of its width.
  int order[MI355_MAX_DIMS];
  for (int i = 0; i < out->ndim; ++i) order[i] = i;
  auto key = [&](int i) { return out->sizes[i] > 1 ? out->strides[i] : INT64_MAX; };  // size-1 dims: anywhere (dropped later)
  for (int i = 1; i < out->ndim; ++i) {  // stable insertion sort by descending output stride
    const int v = order[i];
    int j = i;
    while (j > 0 && key(order[j - 1]) < key(v)) {
      order[j] = order[j - 1];
      --j;
    }
    order[j] = v;
  }
  int64_t psizes[MI355_MAX_DIMS];
  int64_t pstrides[NT][MI355_MAX_DIMS];
  for (int i = 0; i < out->ndim; ++i) {
    psizes[i] = out->sizes[order[i]];
    for (int t = 0; t < NT; ++t) pstrides[t][i] = ts[t]->strides[order[i]];
  }
  const int64_t* strides[NT];
  for (int t = 0; t < NT; ++t) strides[t] = pstrides[t];
  Dims<NT> d = collapse_dims<NT>(out->ndim, psizes, strides);

  // Vectorise along the innermost collapsed dim when every operand is unit-stride (or
  // broadcast) there and every vector stays aligned.
  const int last = d.ndim - 1;
  bool vec_ok = V > 1 && d.sizes[last] % V == 0 && d.strides[NT - 1][last] == 1;
  uint32_t splat = 0;
  for (int t = 0; t < NT && vec_ok; ++t) {
    const int64_t s = d.strides[t][last];
    if (t < NIN && s == 0) {
      splat |= 1u << t;
      continue;
    }
    if (s != 1) vec_ok = false;
    if (reinterpret_cast<uintptr_t>(ts[t]->data) % (esz[t == NIN ? 3 : t] * V)) vec_ok = false;
    for (int k = 0; k < last; ++k)
      if (d.strides[t][k] % V) vec_ok = false;
  }

  StridedArgs<NT> a{};
  a.ndim = d.ndim;
  a.splat_mask = vec_ok ? splat : 0u;
  for (int k = 0; k < MI355_MAX_DIMS; ++k) {
    a.sizes[k] = d.sizes[k];
    for (int t = 0; t < NT; ++t) a.strides[t][k] = d.strides[t][k];
  }
  int64_t total = n;
  if (vec_ok) {
    a.sizes[last] /= V;
    for (int t = 0; t < NT; ++t) a.strides[t][last] *= V;
    total = n / V;
  }
  const bool wide = total >= (int64_t(1) << 31);
  if (!wide)
    for (int k = 0; k < d.ndim; ++k) a.div[k] = make_fastdiv((uint32_t)a.sizes[k]);
  if (!vec_ok && V > 1 && !wide && n >= 4096) {
    // dense row-major output on a vector boundary: vector stores over the flat output
    bool dense_out = reinterpret_cast<uintptr_t>(out->data) % (esz[3] * V) == 0;
    int64_t expect = 1;
    for (int k = d.ndim - 1; k >= 0 && dense_out; --k) {
      dense_out = d.strides[NT - 1][k] == expect;
      expect *= d.sizes[k];
    }
    if (dense_out) {
      uint32_t flat_mask = 0;
      for (int t = 0; t < NIN; ++t) {
        bool same = reinterpret_cast<uintptr_t>(ts[t]->data) % (esz[t] * V) == 0;
        for (int k = 0; k < d.ndim && same; ++k) same = d.strides[t][k] == d.strides[NT - 1][k];
        if (same) flat_mask |= 1u << t;
      }
      const int grid = grid_for((n + V - 1) / V, kEwBlock, 1 << 30);
      hipLaunchKernelGGL((ew_dense_out_kernel<F, V>), dim3(grid), dim3(kEwBlock), 0, stream, f, p, a, n, flat_mask);
      return check_launch(name);
    }
  }
  // Large vectorised problems: four work items per thread, so that a block owns 4 * 256 vectors.
  constexpr int kStridedUnroll = 4;
  if (!wide && total >= (int64_t)kEwBlock * kStridedUnroll * kNumCU * 4) {
    const int grid = grid_for(total, kEwBlock * kStridedUnroll, 1 << 30);
    if (vec_ok)
      hipLaunchKernelGGL((ew_strided_kernel<F, V, false, kStridedUnroll>), dim3(grid), dim3(kEwBlock), 0, stream, f, p, a, total);
    else  // an innermost extent that is no multiple of the vector (197 tokens): elements, four in flight per thread
      hipLaunchKernelGGL((ew_strided_kernel<F, 1, false, kStridedUnroll>), dim3(grid), dim3(kEwBlock), 0, stream, f, p, a, total);
    return check_launch(name);
  }
  const int grid = grid_for(total, kEwBlock, 1 << 30);
  if (vec_ok) {
    if (wide)
      hipLaunchKernelGGL((ew_strided_kernel<F, V, true, 1>), dim3(grid), dim3(kEwBlock), 0, stream, f, p, a, total);
    else
      hipLaunchKernelGGL((ew_strided_kernel<F, V, false, 1>), dim3(grid), dim3(kEwBlock), 0, stream, f, p, a, total);
  } else {
    if (wide)
      hipLaunchKernelGGL((ew_strided_kernel<F, 1, true, 1>), dim3(grid), dim3(kEwBlock), 0, stream, f, p, a, total);
    else
      hipLaunchKernelGGL((ew_strided_kernel<F, 1, false, 1>), dim3(grid), dim3(kEwBlock), 0, stream, f, p, a, total);
  }
  return check_launch(name);
}

}  // namespace mi355
