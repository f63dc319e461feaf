// index_select / embedding (row gather) and gather (element gather).  Both move bits,
// never values, so every dtype of a given width shares a kernel and results are exact.
//
//   rows_wave   rows of >= 64 copy units: one wave64 per output row, 128-bit units when
//               alignment allows, four loads in flight per lane;
//   rows_elem   short rows: one thread per copy unit;
//   gather_rows gather along the last dim of dense operands: the source row is staged in LDS
//               with coalesced loads and the indices are resolved there;
//   gather      any other layout: one thread per output element (or per 4 consecutive 32-bit
//               elements when the index tensor is dense), index stream coalesced.
// An out-of-range index is never dereferenced: the output is zero-filled there and the
// device error flag is raised.
#include "elementwise.h"

namespace mi355 {

constexpr int kIxBlock = 256;
typedef u32x4 U128;  // 16-byte copy unit

template <typename I> __device__ __forceinline__ int64_t load_index(const void* p, int64_t j) {
  return (int64_t) static_cast<const I*>(p)[j];
}

template <typename U, typename I>
__global__ __launch_bounds__(kIxBlock) void index_rows_wave_kernel(const U* __restrict__ src, const void* __restrict__ index,
                                                                  U* __restrict__ out, int64_t outer, int64_t n_src,
                                                                  int64_t n_idx, int64_t row_units, int32_t* err) {
  const int lane = threadIdx.x % kWave;
  const int64_t wave0 = (int64_t)blockIdx.x * (kIxBlock / kWave) + threadIdx.x / kWave;
  const int64_t nwaves = (int64_t)gridDim.x * (kIxBlock / kWave);
  const int64_t rows = outer * n_idx;
  for (int64_t r = wave0; r < rows; r += nwaves) {
    const int64_t o = r / n_idx, j = r - o * n_idx;
    const int64_t idx = load_index<I>(index, j);
    U* dst = out + r * row_units;
    if (idx < 0 || idx >= n_src) {
      if (err && lane == 0) *err = 1;
      for (int64_t u = lane; u < row_units; u += kWave) dst[u] = U(0);
      continue;
    }
    const U* s = src + (o * n_src + idx) * row_units;
    // rows are read and written once: streaming (non-temporal) accesses, four loads in flight
    int64_t u = lane;
    if (row_units <= 4 * kWave) {  // a short row is one batch under per-lane predicates: one memory latency
      if (u < row_units) {
        const bool k1 = u + kWave < row_units, k2 = u + 2 * kWave < row_units, k3 = u + 3 * kWave < row_units;
        U a = __builtin_nontemporal_load(s + u), b, c, d;
        if (k1) b = __builtin_nontemporal_load(s + u + kWave);
        if (k2) c = __builtin_nontemporal_load(s + u + 2 * kWave);
        if (k3) d = __builtin_nontemporal_load(s + u + 3 * kWave);
        __builtin_nontemporal_store(a, dst + u);
        if (k1) __builtin_nontemporal_store(b, dst + u + kWave);
        if (k2) __builtin_nontemporal_store(c, dst + u + 2 * kWave);
        if (k3) __builtin_nontemporal_store(d, dst + u + 3 * kWave);
      }
      continue;
    }
    for (; u + 3 * kWave < row_units; u += 4 * kWave) {
      const U a = __builtin_nontemporal_load(s + u), b = __builtin_nontemporal_load(s + u + kWave),
              c = __builtin_nontemporal_load(s + u + 2 * kWave), d = __builtin_nontemporal_load(s + u + 3 * kWave);
      __builtin_nontemporal_store(a, dst + u);
      __builtin_nontemporal_store(b, dst + u + kWave);
      __builtin_nontemporal_store(c, dst + u + 2 * kWave);
      __builtin_nontemporal_store(d, dst + u + 3 * kWave);
    }
    for (; u < row_units; u += kWave) __builtin_nontemporal_store(__builtin_nontemporal_load(s + u), dst + u);
  }
}

// Long rows when the launch has many of them: one wave per 4 KB chunk of an output row (four
// 128-bit loads per lane, all issued before the first store, nothing else: no loop), the index
// read through the scalar cache.  The shape of the flat copy kernel, which moves the same bytes
// 5 % faster than a wave that walks a whole 8 KB row in two batches.
template <typename U, typename I>
__global__ __launch_bounds__(kIxBlock) void index_rows_chunk_kernel(const U* __restrict__ src, const void* __restrict__ index,
                                                                   U* __restrict__ out, int64_t outer, int64_t n_src,
                                                                   int64_t n_idx, int row_units, int chunks, int32_t* err) {
  const int lane = threadIdx.x % kWave;
  const int64_t w = (int64_t)blockIdx.x * (kIxBlock / kWave) + __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int64_t r = w / chunks;
  if (r >= outer * n_idx) return;
  const int u0 = (int)(w - r * chunks) * (4 * kWave) + lane;
  int64_t o = 0, j = r;
  if (outer != 1) {
    o = r / n_idx;
    j = r - o * n_idx;
  }
  const int64_t idx = load_index<I>(index, j);
  U* dst = out + r * row_units + u0;
  const bool k0 = u0 < row_units, k1 = u0 + kWave < row_units, k2 = u0 + 2 * kWave < row_units, k3 = u0 + 3 * kWave < row_units;
  if (idx < 0 || idx >= n_src) {
    if (err && lane == 0) *err = 1;
    if (k0) dst[0] = U(0);
    if (k1) dst[kWave] = U(0);
    if (k2) dst[2 * kWave] = U(0);
    if (k3) dst[3 * kWave] = U(0);
    return;
  }
  const U* s = src + (o * n_src + idx) * row_units + u0;
  U a, b, c, d;
  if (k0) a = __builtin_nontemporal_load(s);
  if (k1) b = __builtin_nontemporal_load(s + kWave);
  if (k2) c = __builtin_nontemporal_load(s + 2 * kWave);
  if (k3) d = __builtin_nontemporal_load(s + 3 * kWave);
  if (k0) __builtin_nontemporal_store(a, dst);
  if (k1) __builtin_nontemporal_store(b, dst + kWave);
  if (k2) __builtin_nontemporal_store(c, dst + 2 * kWave);
  if (k3) __builtin_nontemporal_store(d, dst + 3 * kWave);
}

template <typename U, typename I>
__global__ __launch_bounds__(kIxBlock) void index_rows_elem_kernel(const U* __restrict__ src, const void* __restrict__ index,
                                                                  U* __restrict__ out, int64_t outer, int64_t n_src,
                                                                  int64_t n_idx, int64_t row_units, int32_t* err) {
  const int64_t total = outer * n_idx * row_units;
  const int64_t stride = (int64_t)gridDim.x * kIxBlock;
  for (int64_t e = (int64_t)blockIdx.x * kIxBlock + threadIdx.x; e < total; e += stride) {
    const int64_t r = e / row_units, u = e - r * row_units;
    const int64_t o = r / n_idx, j = r - o * n_idx;
    const int64_t idx = load_index<I>(index, j);
    if (idx < 0 || idx >= n_src) {
      if (err) *err = 1;
      out[e] = U(0);
    } else {
      out[e] = src[(o * n_src + idx) * row_units + u];
    }
  }
}


template <typename U>
static int run_index_select(const void* src, const void* index, int idx_dtype, void* out, int64_t outer, int64_t n_src,
                            int64_t n_idx, int64_t row_units, int32_t* err, hipStream_t st) {
  const int64_t rows = outer * n_idx;
  const bool i64 = idx_dtype == MI355_I64;
  // 128-bit units, rows of more than 4 KB, enough of them to fill the chip: a wave per 4 KB chunk
  if constexpr (sizeof(U) == 16)
  if (row_units > 4 * kWave && row_units < (1 << 24) && rows >= (int64_t)kNumCU * 8) {
    const int chunks = (int)((row_units + 4 * kWave - 1) / (4 * kWave));
    const int64_t nwaves = rows * chunks;
    const int64_t grid = (nwaves + kIxBlock / kWave - 1) / (kIxBlock / kWave);
    if (grid < (int64_t(1) << 31)) {
      if (i64) hipLaunchKernelGGL((index_rows_chunk_kernel<U, int64_t>), dim3((unsigned)grid), dim3(kIxBlock), 0, st, (const U*)src, index, (U*)out, outer, n_src, n_idx, (int)row_units, chunks, err);
      else hipLaunchKernelGGL((index_rows_chunk_kernel<U, int32_t>), dim3((unsigned)grid), dim3(kIxBlock), 0, st, (const U*)src, index, (U*)out, outer, n_src, n_idx, (int)row_units, chunks, err);
      return check_launch("mi355_index_select");
    }
  }
  if (row_units >= 2 * kWave) {  // rows of 2 KB and more: a wave per row; shorter rows: a thread per 16-byte unit
    const int grid = grid_for(rows, kIxBlock / kWave, kNumCU * 32);
    if (i64) hipLaunchKernelGGL((index_rows_wave_kernel<U, int64_t>), dim3(grid), dim3(kIxBlock), 0, st, (const U*)src, index, (U*)out, outer, n_src, n_idx, row_units, err);
    else hipLaunchKernelGGL((index_rows_wave_kernel<U, int32_t>), dim3(grid), dim3(kIxBlock), 0, st, (const U*)src, index, (U*)out, outer, n_src, n_idx, row_units, err);
  } else {
    const int grid = grid_for(rows * row_units, kIxBlock, kNumCU * 32);
    if (i64) hipLaunchKernelGGL((index_rows_elem_kernel<U, int64_t>), dim3(grid), dim3(kIxBlock), 0, st, (const U*)src, index, (U*)out, outer, n_src, n_idx, row_units, err);
    else hipLaunchKernelGGL((index_rows_elem_kernel<U, int32_t>), dim3(grid), dim3(kIxBlock), 0, st, (const U*)src, index, (U*)out, outer, n_src, n_idx, row_units, err);
  }
  return check_launch("mi355_index_select");
}

// ---------------------------------------------------------------- gather
struct GatherArgs {
  int32_t ndim, dim;
  int64_t sizes[MI355_MAX_DIMS];        // index (= out) sizes
  int64_t idx_strides[MI355_MAX_DIMS];  // index strides
  int64_t src_strides[MI355_MAX_DIMS];
  int64_t src_dim_size;
};

// One thread per VEC consecutive output elements along the last dim (VEC == 4 needs a
// dense index tensor and a last-dim size divisible by 4).
template <typename U, int VEC>
__global__ __launch_bounds__(kIxBlock) void gather_kernel(const U* __restrict__ src, const int64_t* __restrict__ index,
                                                         U* __restrict__ out, GatherArgs a, int64_t total,
                                                         int32_t* err) {
  const int64_t stride = (int64_t)gridDim.x * kIxBlock;
  const int last = a.ndim - 1;
  for (int64_t w = (int64_t)blockIdx.x * kIxBlock + threadIdx.x; w < total; w += stride) {
    const int64_t e = w * VEC;
    int64_t rem = e, ioff = 0, soff = 0, last_coord = 0;
    for (int k = last; k >= 0; --k) {
      const int64_t q = rem / a.sizes[k];
      const int64_t c = rem - q * a.sizes[k];
      rem = q;
      ioff += c * a.idx_strides[k];
      if (k == last) last_coord = c;
      if (k != a.dim) soff += c * a.src_strides[k];
    }
    if constexpr (VEC == 1) {
      const int64_t idx = index[ioff];
      if (idx < 0 || idx >= a.src_dim_size) {
        if (err) *err = 1;
        out[e] = U{};
      } else {
        out[e] = src[soff + idx * a.src_strides[a.dim]];
      }
    } else {
      (void)last_coord;
      // dense index: the VEC indices are adjacent in memory and 16-byte aligned pairs
      const VecN<int64_t, 2> i01 = ld<int64_t, 2>(index + e);
      const VecN<int64_t, 2> i23 = ld<int64_t, 2>(index + e + 2);
      const int64_t ix[4] = {i01.v[0], i01.v[1], i23.v[0], i23.v[1]};
      VecN<U, 4> r;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (ix[j] < 0 || ix[j] >= a.src_dim_size) {
          if (err) *err = 1;
          r.v[j] = U{};
        } else {
          const int64_t extra = a.dim == last ? 0 : (int64_t)j * a.src_strides[last];
          r.v[j] = src[soff + extra + ix[j] * a.src_strides[a.dim]];
        }
      }
      st<U, 4>(out + e, r);
    }
  }
}

// Gather along the last dim of a dense [rows, len] source with a dense [rows, n_idx] index (or
// one [n_idx] index shared by all rows: index_select along the last dim):
// one block stages (its share of) the source row in LDS with coalesced 128-bit loads, then
// resolves four indices per thread per step from LDS — the index stream and the output stay
// fully coalesced and no random access leaves the CU.  grid = (splits, rows).
template <typename U>
__global__ __launch_bounds__(kIxBlock) void gather_rows_lds_kernel(const U* __restrict__ src, const int64_t* __restrict__ index,
                                                                  U* __restrict__ out, int64_t len, int64_t n_idx,
                                                                  int64_t idx_row_stride, int64_t per_split, int32_t* err) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  U* row = reinterpret_cast<U*>(smem_raw);
  const int64_t r = blockIdx.y;
  const U* s = src + r * len;
  constexpr int UV = 16 / sizeof(U);
  const int64_t j0 = (int64_t)blockIdx.x * per_split;
  const int64_t j1 = j0 + per_split < n_idx ? j0 + per_split : n_idx;
  const int64_t* ix = index + r * idx_row_stride;  // 0: every row uses the same indices (index_select)
  U* o = out + r * n_idx;
  const bool vec = n_idx % 4 == 0 && per_split % 4 == 0 && (reinterpret_cast<uintptr_t>(ix) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(o) % (4 * sizeof(U))) == 0;
  // The first indices of every thread are requested before the row is staged, and every later batch
  // one step ahead: the index stream (two thirds of the bytes) never waits behind the barrier.
  VecN<int64_t, 2> na{}, nb{};
  const int64_t jf = j0 + (int64_t)threadIdx.x * 4;
  if (vec && jf < j1) {
    na = ld_nt<int64_t, 2>(ix + jf);
    nb = ld_nt<int64_t, 2>(ix + jf + 2);
  }
  if (len % UV == 0 && (reinterpret_cast<uintptr_t>(s) & 15) == 0) {
    for (int64_t i = (int64_t)threadIdx.x * UV; i < len; i += (int64_t)kIxBlock * UV)
      st<U, UV>(row + i, ld_nt<U, UV>(s + i));
  } else {
    for (int64_t i = threadIdx.x; i < len; i += kIxBlock) row[i] = s[i];
  }
  __syncthreads();
  if (vec) {
    for (int64_t j = jf; j < j1; j += (int64_t)kIxBlock * 4) {
      const VecN<int64_t, 2> a = na, b = nb;
      const int64_t jn = j + (int64_t)kIxBlock * 4;
      if (jn < j1) {
        na = ld_nt<int64_t, 2>(ix + jn);
        nb = ld_nt<int64_t, 2>(ix + jn + 2);
      }
      const int64_t id[4] = {a.v[0], a.v[1], b.v[0], b.v[1]};
      VecN<U, 4> v;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const bool ok = id[e] >= 0 && id[e] < len;
        if (!ok && err) *err = 1;
        v.v[e] = ok ? row[id[e]] : U(0);
      }
      st_nt<U, 4>(o + j, v);
    }
  } else {
    for (int64_t j = j0 + threadIdx.x; j < j1; j += kIxBlock) {
      const int64_t id = ix[j];
      const bool ok = id >= 0 && id < len;
      if (!ok && err) *err = 1;
      o[j] = ok ? row[id] : U(0);
    }
  }
}

template <typename U>
static int run_gather(const mi355_tensor* src, int dim, const mi355_tensor* index, const mi355_tensor* out,
                      int32_t* err, hipStream_t st) {
  GatherArgs a{};
  a.ndim = index->ndim;
  a.dim = dim;
  a.src_dim_size = src->sizes[dim];
  bool idx_dense = true;
  int64_t expect = 1;
  for (int k = index->ndim - 1; k >= 0; --k) {
    a.sizes[k] = index->sizes[k];
    a.idx_strides[k] = index->strides[k];
    a.src_strides[k] = src->strides[k];
    if (index->sizes[k] != 1 && index->strides[k] != expect) idx_dense = false;
    expect *= index->sizes[k];
  }
  const int64_t n = numel(out);
  const int last = index->ndim - 1;
  // LDS-staged path: last-dim gather, dense source and index, matching outer extents.
  {
    bool ok = dim == last && idx_dense;
    int64_t expect_s = 1, rows = 1;
    for (int k = last; k >= 0 && ok; --k) {
      if (src->sizes[k] != 1 && src->strides[k] != expect_s) ok = false;
      expect_s *= src->sizes[k];
      if (k != last) {
        if (index->sizes[k] != src->sizes[k]) ok = false;
        rows *= index->sizes[k];
      }
    }
    const int64_t len = src->sizes[last], n_idx = index->sizes[last];
    if (ok && len > 0 && len * (int64_t)sizeof(U) <= 64 * 1024 && rows < 65536 && n_idx >= len / 8) {
      int64_t splits = 1;
      if (rows < 512) {
        splits = n_idx / 4096;
        if (splits < 1) splits = 1;
        if (splits > 64) splits = 64;
      }
      int64_t per_split = (n_idx + splits - 1) / splits;
      per_split = (per_split + 3) / 4 * 4;
      splits = (n_idx + per_split - 1) / per_split;
      hipLaunchKernelGGL((gather_rows_lds_kernel<U>), dim3((unsigned)splits, (unsigned)rows), dim3(kIxBlock),
                         (size_t)(len * sizeof(U)), st, (const U*)src->data, (const int64_t*)index->data,
                         (U*)out->data, len, n_idx, n_idx, per_split, err);
      return check_launch("mi355_gather(lds)");
    }
  }
  const bool vec = sizeof(U) == 4 && idx_dense && a.sizes[last] % 4 == 0 && aligned16(index->data) &&
                   aligned16(out->data);
  if (vec) {
    const int grid = grid_for(n / 4, kIxBlock, kNumCU * 32);
    hipLaunchKernelGGL((gather_kernel<U, 4>), dim3(grid), dim3(kIxBlock), 0, st, (const U*)src->data,
                       (const int64_t*)index->data, (U*)out->data, a, n / 4, err);
  } else {
    const int grid = grid_for(n, kIxBlock, kNumCU * 32);
    hipLaunchKernelGGL((gather_kernel<U, 1>), dim3(grid), dim3(kIxBlock), 0, st, (const U*)src->data,
                       (const int64_t*)index->data, (U*)out->data, a, n, err);
  }
  return check_launch("mi355_gather");
}

}  // namespace mi355

using namespace mi355;

extern "C" int mi355_index_select(const void* src, int elem_size, int64_t outer, int64_t n_src, int64_t inner,
                                  const void* index, int idx_dtype, int64_t n_idx, void* out, int32_t* err_flag,
                                  void* stream) {
  MI355_REQUIRE(outer >= 0 && n_src >= 0 && inner >= 0 && n_idx >= 0, "mi355_index_select: negative extent");
  MI355_REQUIRE(elem_size == 1 || elem_size == 2 || elem_size == 4 || elem_size == 8,
                "mi355_index_select: elem_size %d", elem_size);
  MI355_REQUIRE(idx_dtype == MI355_I32 || idx_dtype == MI355_I64, "mi355_index_select: index must be i32 or i64");
  if (outer == 0 || inner == 0 || n_idx == 0) return MI355_OK;
  MI355_REQUIRE(index != nullptr && out != nullptr, "mi355_index_select: NULL data pointer");
  MI355_REQUIRE(src != nullptr || n_src == 0, "mi355_index_select: NULL src");
  hipStream_t st = static_cast<hipStream_t>(stream);
  // Selecting single elements along the last dim: stage each source row in LDS and resolve the
  // (shared) indices there instead of issuing one scattered global read per element.
  if (inner == 1 && idx_dtype == MI355_I64 && n_src * elem_size <= 64 * 1024 && outer < 65536 && n_idx >= n_src / 8 &&
      n_src > 0) {
    int64_t splits = 1;
    if (outer < 512) {
      splits = n_idx / 4096;
      if (splits < 1) splits = 1;
      if (splits > 64) splits = 64;
    }
    int64_t per_split = (n_idx + splits - 1) / splits;
    per_split = (per_split + 3) / 4 * 4;
    splits = (n_idx + per_split - 1) / per_split;
    const dim3 grid((unsigned)splits, (unsigned)outer);
    const size_t lds = (size_t)(n_src * elem_size);
    const int64_t* ix = static_cast<const int64_t*>(index);
    switch (elem_size) {
      case 1: hipLaunchKernelGGL((gather_rows_lds_kernel<uint8_t>), grid, dim3(kIxBlock), lds, st, (const uint8_t*)src, ix, (uint8_t*)out, n_src, n_idx, (int64_t)0, per_split, err_flag); break;
      case 2: hipLaunchKernelGGL((gather_rows_lds_kernel<uint16_t>), grid, dim3(kIxBlock), lds, st, (const uint16_t*)src, ix, (uint16_t*)out, n_src, n_idx, (int64_t)0, per_split, err_flag); break;
      case 4: hipLaunchKernelGGL((gather_rows_lds_kernel<uint32_t>), grid, dim3(kIxBlock), lds, st, (const uint32_t*)src, ix, (uint32_t*)out, n_src, n_idx, (int64_t)0, per_split, err_flag); break;
      default: hipLaunchKernelGGL((gather_rows_lds_kernel<uint64_t>), grid, dim3(kIxBlock), lds, st, (const uint64_t*)src, ix, (uint64_t*)out, n_src, n_idx, (int64_t)0, per_split, err_flag); break;
    }
    return check_launch("mi355_index_select(lds)");
  }
  const int64_t row_bytes = inner * elem_size;
  const uintptr_t align = reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(out) | (uintptr_t)row_bytes;
  if (align % 16 == 0) return run_index_select<U128>(src, index, idx_dtype, out, outer, n_src, n_idx, row_bytes / 16, err_flag, st);
  if (align % 8 == 0) return run_index_select<uint64_t>(src, index, idx_dtype, out, outer, n_src, n_idx, row_bytes / 8, err_flag, st);
  if (align % 4 == 0) return run_index_select<uint32_t>(src, index, idx_dtype, out, outer, n_src, n_idx, row_bytes / 4, err_flag, st);
  if (align % 2 == 0) return run_index_select<uint16_t>(src, index, idx_dtype, out, outer, n_src, n_idx, row_bytes / 2, err_flag, st);
  return run_index_select<uint8_t>(src, index, idx_dtype, out, outer, n_src, n_idx, row_bytes, err_flag, st);
}

extern "C" int mi355_gather(const mi355_tensor* src, int dim, const mi355_tensor* index, const mi355_tensor* out,
                            int32_t* err_flag, void* stream) {
  int rc;
  if ((rc = check_tensor(src, "mi355_gather", "src"))) return rc;
  if ((rc = check_tensor(index, "mi355_gather", "index"))) return rc;
  if ((rc = check_tensor(out, "mi355_gather", "out"))) return rc;
  MI355_REQUIRE(index->dtype == MI355_I64, "mi355_gather: index must be i64");
  MI355_REQUIRE(src->ndim == index->ndim && src->ndim >= 1, "mi355_gather: src and index must have equal ndim >= 1");
  MI355_REQUIRE(dim >= 0 && dim < src->ndim, "mi355_gather: dim %d out of range", dim);
  MI355_REQUIRE(same_shape(index, out) && out->dtype == src->dtype, "mi355_gather: out must have index's shape and src's dtype");
  int64_t expect = 1;
  for (int k = out->ndim - 1; k >= 0; --k) {
    MI355_REQUIRE(out->sizes[k] == 1 || out->strides[k] == expect, "mi355_gather: out must be dense");
    expect *= out->sizes[k];
    if (k != dim) MI355_REQUIRE(index->sizes[k] <= src->sizes[k], "mi355_gather: index.size(%d) exceeds src.size(%d)", k, k);
  }
  if (numel(out) == 0) return MI355_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (dtype_size(src->dtype)) {
    case 1: return run_gather<uint8_t>(src, dim, index, out, err_flag, st);
    case 2: return run_gather<uint16_t>(src, dim, index, out, err_flag, st);
    case 4: return run_gather<uint32_t>(src, dim, index, out, err_flag, st);
    case 8: return run_gather<uint64_t>(src, dim, index, out, err_flag, st);
    default: return set_error(MI355_ERR_UNSUPPORTED, "mi355_gather: unsupported dtype");
  }
}
