// mm / addmm:  out[M,N] = beta * c + alpha * (a[M,K] @ b[K,N]),  fp32 accumulate.
//
//   mfma     bf16 / f16, a K-contiguous, b either K-contiguous ("NT", e.g. weight.t()) or
//            N-contiguous ("NN", row-major), 16-byte aligned rows.  256x256x64 block tile,
//            eight wave64 (2x4, two per SIMD), each wave 128x64 = 8x4 v_mfma_f32_16x16x32
//            tiles with 128 fp32 accumulators; A and B panels double-buffered in 128 KB of
//            LDS, swizzled so that the 128-bit global->LDS writes and the fragment reads
//            are bank-conflict free.  A row-major B stays N-contiguous in LDS and is
//            transposed by the LDS read itself (ds_read_b64_tr_b16).  The next k-tile is
//            in flight from HBM/L2 to registers during the MFMA phase; block -> tile map
//            groups tiles per XCD so that one L2 serves neighbouring tiles.
//   generic  any strides, bf16 / f16 / f32: 64x64 LDS tile, FMA inner loop.  Correctness
//            path for shapes the MFMA kernel does not take.
#include "common.h"

namespace mi355 {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct alignas(sizeof(T) * 4) VecN4 {
  T v[4];
};

template <typename T> struct Mfma;
template <> struct Mfma<bf16_t> {
  using frag = bf16x8;
  static __device__ __forceinline__ f32x4 run(frag a, frag b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mfma<f16_t> {
  using frag = f16x8;
  static __device__ __forceinline__ f32x4 run(frag a, frag b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int kGemmThreads = 512;                  // 8 waves: 2 (m) x 4 (n), each 128 x 64
constexpr int kRowBytes = BK * 2;                  // K-contiguous panel row: 64 k = 128 B = 8 chunks
constexpr int kPanelBytes = BM * kRowBytes;        // 32 KB per operand per stage (either layout)
constexpr int kStageBytes = 2 * kPanelBytes;       // A + B
constexpr int kGemmLds = 2 * kStageBytes;          // double buffered: 128 KB

// K-contiguous panel ([row][k], A and the "NT" B): byte offset of 16-byte chunk c (0..7) of
// row r.  The chunk index is XORed with (r + r/8) mod 8, which makes both any 8 consecutive
// rows (32-bank LDS) and any 16 consecutive rows (64-bank LDS) hit distinct banks when the 16
// lanes of an MFMA fragment read the same chunk of 16 rows; the 128-bit writes of a row's 8
// chunks stay a full 128-byte line.
__device__ __forceinline__ int swz_k(int r, int c) {
  return r * kRowBytes + ((c ^ ((r + (r >> 3)) & 7)) << 4);
}
// N-contiguous panel ([k][n], the row-major "NN" B, 512 B per k): byte offset of 16-byte unit u
// (0..31) of row k.  32-byte chunks are XORed with (k%4) | ((k/8)%2)*4 so that the transposing
// 64-bit reads (4 k-rows x 32 B per 16 lanes, rows k..k+3 and k+8..k+11 per 32 lanes) spread
// over all banks.
__device__ __forceinline__ int swz_n(int k, int u) {
  const int x = (k & 3) | (((k >> 3) & 1) << 2);
  return k * (BN * 2) + ((((u >> 1) ^ x)) << 5) + ((u & 1) << 4);
}

struct GemmArgs {
  const void* a;
  const void* b;
  const void* c;
  void* out;
  int64_t lda, ldb;  // element stride between rows of a ([M][K]) and between the K-contiguous
                     // rows of b ([N][K], NT) or the N-contiguous rows of b ([K][N], NN)
  int64_t c_rs, c_cs;
  int32_t M, N, K;
  float alpha, beta;
  int32_t tiles_m, tiles_n;
};

// Tile id for this block: blocks land on XCD (blockIdx % 8); give each XCD a contiguous
// band of tile ids, then walk the band in groups of 8 tile-rows so A and B panels repeat
// in that XCD's L2.
__device__ __forceinline__ void tile_coords(const GemmArgs& g, int& tm, int& tn) {
  const int nblocks = g.tiles_m * g.tiles_n;
  int pid = blockIdx.x;
  const int per_xcd = (nblocks + kNumXCD - 1) / kNumXCD;
  const int full = nblocks % kNumXCD;  // XCDs that own `per_xcd` tiles when not divisible
  const int xcd = pid % kNumXCD, local = pid / kNumXCD;
  if (full == 0) pid = xcd * per_xcd + local;
  else pid = (xcd < full ? xcd * per_xcd : full * per_xcd + (xcd - full) * (per_xcd - 1)) + local;
  constexpr int GROUP = 8;
  const int in_group = GROUP * g.tiles_n;
  const int group = pid / in_group;
  const int first_m = group * GROUP;
  const int rows = g.tiles_m - first_m < GROUP ? g.tiles_m - first_m : GROUP;
  tm = first_m + (pid % in_group) % rows;
  tn = (pid % in_group) / rows;
}

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));

// ds_read_b64_tr_b16: within each block of 16 lanes, lane s supplies the address of 4
// consecutive 16-bit elements ("row s/4, columns 4*(s%4)..+3" of a 4 x 16 block) and lane i
// receives column i of the 4 rows.  With rows = k and columns = n this turns an N-contiguous
// LDS panel into the K-contiguous MFMA operand.
__device__ __forceinline__ s16x4 lds_read_tr(const unsigned char* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (__attribute__((address_space(3))) s16x4*)(uintptr_t)(const_cast<unsigned char*>(p)));
}

template <typename T, bool B_NN>
__global__ __launch_bounds__(kGemmThreads) void gemm_mfma_kernel(GemmArgs g) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  using frag_t = typename Mfma<T>::frag;
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int wm = wave >> 2, wn = wave & 3;  // wave tile: rows wm*128.., cols wn*64..
  int tm, tn;
  tile_coords(g, tm, tn);
  const int bm = tm * BM, bn = tn * BN;
  const T* A = static_cast<const T*>(g.a);
  const T* B = static_cast<const T*>(g.b);

  // ---- global -> register staging: 4 chunks of A and 4 of B per thread per k-tile
  u32x4 ra[4], rb[4];
  const int lc = tid & 7, lr = tid >> 3;    // K-contiguous panels: chunk lc of rows lr + 64*i
  const int nu = tid & 31, kr = tid >> 5;   // NN B: 16-byte unit nu of k rows kr + 16*i
  auto load_tile = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int gr = bm + lr + 64 * i;
      gr = gr < g.M ? gr : g.M - 1;
      const int k = k0 + lc * 8;
      ra[i] = k < g.K ? *reinterpret_cast<const u32x4*>(A + (int64_t)gr * g.lda + k) : u32x4{0, 0, 0, 0};
    }
    if constexpr (!B_NN) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        int gn = bn + lr + 64 * i;
        gn = gn < g.N ? gn : g.N - 1;
        const int k = k0 + lc * 8;
        rb[i] = k < g.K ? *reinterpret_cast<const u32x4*>(B + (int64_t)gn * g.ldb + k) : u32x4{0, 0, 0, 0};
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int k = k0 + kr + 16 * i;
        int gn = bn + nu * 8;
        gn = gn < g.N ? gn : 0;  // N % 8 == 0: a unit is all-in or all-out; out-of-range columns are never stored
        rb[i] = k < g.K ? *reinterpret_cast<const u32x4*>(B + (int64_t)k * g.ldb + gn) : u32x4{0, 0, 0, 0};
      }
    }
  };
  auto store_tile = [&](int stage) {
    unsigned char* pa = lds + stage * kStageBytes;
    unsigned char* pb = pa + kPanelBytes;
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(pa + swz_k(lr + 64 * i, lc)) = ra[i];
    if constexpr (!B_NN) {
#pragma unroll
      for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(pb + swz_k(lr + 64 * i, lc)) = rb[i];
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(pb + swz_n(kr + 16 * i, nu)) = rb[i];
    }
  };

  f32x4 acc[8][4];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int nk = (g.K + BK - 1) / BK;
  if (nk > 0) {
    load_tile(0);
    store_tile(0);
    if (nk > 1) load_tile(BK);
  }
  __syncthreads();
  const int fr = lane & 15, fc = lane >> 4;  // fragment row (m or n) and k-group of this lane
  for (int kt = 0; kt < nk; ++kt) {
    const int stage = kt & 1;
    const unsigned char* pa = lds + stage * kStageBytes;
    const unsigned char* pb = pa + kPanelBytes;
#pragma unroll
    for (int kk = 0; kk < BK / 32; ++kk) {
      frag_t fa[8], fb[4];
#pragma unroll
      for (int i = 0; i < 8; ++i)
        fa[i] = *reinterpret_cast<const frag_t*>(pa + swz_k(wm * 128 + i * 16 + fr, kk * 4 + fc));
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if constexpr (!B_NN) {
          fb[j] = *reinterpret_cast<const frag_t*>(pb + swz_k(wn * 64 + j * 16 + fr, kk * 4 + fc));
        } else {
          // k = kk*32 + fc*8 + h*4 + (lane%16)/4, columns wn*64 + j*16 + 4*(lane%4) .. +3
          const int kb = kk * 32 + fc * 8 + (fr >> 2);
          const int n0 = wn * 64 + j * 16 + ((fr & 3) << 2);  // element column; 16-byte unit = n0/8
          const s16x4 lo = lds_read_tr(pb + swz_n(kb, n0 >> 3) + ((n0 & 7) << 1));
          const s16x4 hi = lds_read_tr(pb + swz_n(kb + 4, n0 >> 3) + ((n0 & 7) << 1));
          const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
          fb[j] = __builtin_bit_cast(frag_t, both);
        }
      }
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          // operands swapped: the lane ends up with 4 consecutive n of one row m
          acc[i][j] = Mfma<T>::run(fb[j], fa[i], acc[i][j]);
    }
    if (kt + 1 < nk) {
      store_tile(stage ^ 1);                       // tile kt+1, loaded during the previous compute phase
      if (kt + 2 < nk) load_tile((kt + 2) * BK);  // in flight during the next compute phase
    }
    __syncthreads();
  }

  // ---- epilogue: lane holds C[m = fr][n = fc*4 .. +3] of each 16x16 tile
  T* D = static_cast<T*>(g.out);
  const T* C = static_cast<const T*>(g.c);
  const bool use_c = C != nullptr && g.beta != 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int m = bm + wm * 128 + i * 16 + fr;
    if (m >= g.M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = bn + wn * 64 + j * 16 + fc * 4;
      if (n >= g.N) continue;  // N % 4 == 0 on this path: 4 columns are all in or all out
      VecN4<T> r;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float v = g.alpha * acc[i][j][e];
        if (use_c) v += g.beta * static_cast<float>(C[(int64_t)m * g.c_rs + (int64_t)(n + e) * g.c_cs]);
        r.v[e] = static_cast<T>(v);
      }
      *reinterpret_cast<VecN4<T>*>(D + (int64_t)m * g.N + n) = r;
    }
  }
}

// ---------------------------------------------------------------- generic fallback
constexpr int GT = 64, GK = 16;
template <typename T>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const T* __restrict__ A, int64_t a_rs, int64_t a_cs,
                                                          const T* __restrict__ B, int64_t b_rs, int64_t b_cs,
                                                          const T* __restrict__ C, int64_t c_rs, int64_t c_cs,
                                                          T* __restrict__ D, int64_t M, int64_t N, int64_t K,
                                                          float alpha, float beta) {
  __shared__ float As[GK][GT + 1], Bs[GK][GT + 1];
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  const int64_t bm = (int64_t)blockIdx.y * GT, bn = (int64_t)blockIdx.x * GT;
  float acc[4][4] = {};
  for (int64_t k0 = 0; k0 < K; k0 += GK) {
    for (int e = threadIdx.x; e < GT * GK; e += 256) {
      const int r = e / GK, kk = e % GK;
      const int64_t m = bm + r, k = k0 + kk;
      As[kk][r] = (m < M && k < K) ? static_cast<float>(A[m * a_rs + k * a_cs]) : 0.f;
      const int kk2 = e / GT, c = e % GT;
      const int64_t n = bn + c, k2 = k0 + kk2;
      Bs[kk2][c] = (n < N && k2 < K) ? static_cast<float>(B[k2 * b_rs + n * b_cs]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GK; ++kk) {
      float av[4], bv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) bv[j] = Bs[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += av[i] * bv[j];
    }
    __syncthreads();
  }
  const bool use_c = C != nullptr && beta != 0.f;
  for (int i = 0; i < 4; ++i) {
    const int64_t m = bm + ty * 4 + i;
    if (m >= M) continue;
    for (int j = 0; j < 4; ++j) {
      const int64_t n = bn + tx * 4 + j;
      if (n >= N) continue;
      float v = alpha * acc[i][j];
      if (use_c) v += beta * static_cast<float>(C[m * c_rs + n * c_cs]);
      D[m * N + n] = static_cast<T>(v);
    }
  }
}

template <typename T>
static int run_gemm(const void* a, int64_t a_rs, int64_t a_cs, const void* b, int64_t b_rs, int64_t b_cs,
                    const void* c, int64_t c_rs, int64_t c_cs, void* out, int64_t M, int64_t N, int64_t K,
                    double alpha, double beta, hipStream_t st) {
  constexpr bool can_mfma = sizeof(T) == 2;
  if constexpr (can_mfma) {
    const bool a_ok = a_cs == 1 && a_rs % 8 == 0 && aligned16(a);
    const bool b_nt = b_rs == 1 && b_cs % 8 == 0 && aligned16(b);
    const bool b_nn = b_cs == 1 && b_rs % 8 == 0 && aligned16(b);
    const bool fits = M < (1 << 30) && N < (1 << 30) && K < (1 << 30);
    // Tiny problems are cheaper on the generic kernel than on a mostly empty 256x256 tile.
    const bool worth = M * N >= 128 * 128 && K >= 32;
    if (a_ok && (b_nt || b_nn) && K % 8 == 0 && N % 8 == 0 && fits && worth && K > 0 &&
        reinterpret_cast<uintptr_t>(out) % 8 == 0) {
      GemmArgs g{};
      g.a = a; g.b = b; g.c = c; g.out = out;
      g.lda = a_rs;
      g.ldb = b_nt ? b_cs : b_rs;
      g.c_rs = c_rs; g.c_cs = c_cs;
      g.M = (int32_t)M; g.N = (int32_t)N; g.K = (int32_t)K;
      g.alpha = (float)alpha; g.beta = (float)beta;
      g.tiles_m = (int32_t)((M + BM - 1) / BM);
      g.tiles_n = (int32_t)((N + BN - 1) / BN);
      const int64_t nblocks = (int64_t)g.tiles_m * g.tiles_n;
      MI355_REQUIRE(nblocks < (int64_t(1) << 31), "mi355_gemm: too many tiles");
      static thread_local bool attr_set[2] = {false, false};
      if (b_nt) {
        auto kern = gemm_mfma_kernel<T, false>;
        if (!attr_set[0]) {
          hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, kGemmLds);
          attr_set[0] = true;
        }
        hipLaunchKernelGGL(kern, dim3((unsigned)nblocks), dim3(kGemmThreads), kGemmLds, st, g);
      } else {
        auto kern = gemm_mfma_kernel<T, true>;
        if (!attr_set[1]) {
          hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, kGemmLds);
          attr_set[1] = true;
        }
        hipLaunchKernelGGL(kern, dim3((unsigned)nblocks), dim3(kGemmThreads), kGemmLds, st, g);
      }
      return check_launch("mi355_gemm(mfma)");
    }
  }
  const int64_t gx = (N + GT - 1) / GT, gy = (M + GT - 1) / GT;
  MI355_REQUIRE(gy < 65536 && gx < (int64_t(1) << 31), "mi355_gemm: generic path needs M < 4M rows");
  hipLaunchKernelGGL((gemm_generic_kernel<T>), dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, st,
                     static_cast<const T*>(a), a_rs, a_cs, static_cast<const T*>(b), b_rs, b_cs,
                     static_cast<const T*>(c), c_rs, c_cs, static_cast<T*>(out), M, N, K, (float)alpha, (float)beta);
  return check_launch("mi355_gemm(generic)");
}

}  // namespace mi355

using namespace mi355;

extern "C" int mi355_gemm(const void* a, int64_t a_rs, int64_t a_cs, const void* b, int64_t b_rs, int64_t b_cs,
                          const void* c, int64_t c_rs, int64_t c_cs, void* out, int64_t M, int64_t N, int64_t K,
                          double alpha, double beta, int dtype, void* stream) {
  MI355_REQUIRE(M >= 0 && N >= 0 && K >= 0, "mi355_gemm: negative extent");
  if (M == 0 || N == 0) return MI355_OK;
  MI355_REQUIRE(out != nullptr, "mi355_gemm: NULL out");
  MI355_REQUIRE(K == 0 || (a != nullptr && b != nullptr), "mi355_gemm: NULL operand");
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case MI355_BF16: return run_gemm<bf16_t>(a, a_rs, a_cs, b, b_rs, b_cs, c, c_rs, c_cs, out, M, N, K, alpha, beta, st);
    case MI355_F16: return run_gemm<f16_t>(a, a_rs, a_cs, b, b_rs, b_cs, c, c_rs, c_cs, out, M, N, K, alpha, beta, st);
    case MI355_F32: return run_gemm<float>(a, a_rs, a_cs, b, b_rs, b_cs, c, c_rs, c_cs, out, M, N, K, alpha, beta, st);
    default: return set_error(MI355_ERR_UNSUPPORTED, "mi355_gemm: unsupported dtype %s", dtype_name(dtype));
  }
}
