// fp64 mm / addmm on v_mfma_f64_16x16x4_f64 (gfx950), any strides.
//
// A workgroup of WM x WN waves owns a GT x GT tile of the output, a wave WBM x WBN blocks of 16 x 16: sixteen
// waves (4 x 4) of 2 x 2 blocks on 128 x 128 tiles, sixteen waves of one block on 64 x 64 tiles, four waves of
// one block on 32 x 32 tiles (products that would leave most CUs without a 64 x 64 tile).  K advances in steps of
// 32 through two LDS buffers, one barrier per step.  The operands of step t + 1 are fetched into registers
// while step t computes (bounds-checked, zero past the edges, consecutive threads along each operand's
// contiguous dim) and parked in the other buffer behind the MFMAs.  Each operand keeps its own orientation in
// LDS, so that the lanes that fetched consecutive addresses also write consecutive ones:
//   contiguous along k (a row-major a, a transposed b):  [row][k], rows 33 doubles apart - the sixteen rows
//       of a fragment fall on sixteen different bank pairs;
//   contiguous along m / n:  [k][row], k rows GT + 16 doubles apart - the sixteen lanes of a fragment read 128
//       contiguous bytes and the next k row starts on the other half of the banks.
//
// Register layout of the instruction (lane l): the a operand is A[l % 16][l / 16], the b operand B[l / 16][l % 16],
// and register r of the result is D[4 r + l / 16][l % 16].
//
// One instruction is 2048 flops in 64 cycles of a SIMD - the rate of the fp64 vector FMA - but it takes one LDS
// read per MFMA where the FMA tile takes one read per four FMAs, which is what held the FMA kernel at 45 % of
// the peak.  A wave alone on its SIMD issues one such instruction every ~128 cycles (measured on a
// register-only loop: 35 TFLOP/s with four waves per CU, 77 with eight), and a wave that fetches, parks or waits
// issues none, hence four waves per SIMD (two: 54 TFLOP/s at 4096^3, four: 59).
#include <type_traits>

#include "gemm_shared.h"

namespace mi355 {

typedef double f64x4 __attribute__((ext_vector_type(4)));

constexpr int kF64Step = 32;  // k per step
constexpr int f64_operand_doubles(int gt) { return kF64Step * (gt + 16) > gt * (kF64Step + 1) ? kF64Step * (gt + 16) : gt * (kF64Step + 1); }
constexpr int f64_lds_bytes(int gt) { return 2 * 2 * f64_operand_doubles(gt) * 8; }

// A_KF: a is contiguous along k (or has no unit stride); B_NF: b is contiguous along n (or has none).
template <int WBM, int WBN, int WM, int WN, bool A_KF, bool B_NF>
__global__ __launch_bounds__(64 * WM * WN) void gemm_f64_mfma_kernel(const double* __restrict__ A, int64_t a_rs, int64_t a_cs,
                                                           const double* __restrict__ B, int64_t b_rs, int64_t b_cs,
                                                           const double* __restrict__ C, int64_t c_rs, int64_t c_cs,
                                                           double* __restrict__ D, int64_t M, int64_t N, int64_t K, double alpha,
                                                           double beta) {
  constexpr int GT = 16 * WBM * WM, GK = kF64Step, THREADS = 64 * WM * WN;  // WM x WN waves of WBM x WBN blocks each
  static_assert(WBM * WM == WBN * WN, "square tiles");
  constexpr int PER = GT * GK / THREADS;  // elements of each operand a thread moves per step
  static_assert(PER * THREADS == GT * GK, "whole elements per thread");
  constexpr int OP = f64_operand_doubles(GT);
  // element (row, k) of an operand's buffer
  constexpr int A_RS = A_KF ? GK + 1 : 1, A_KS = A_KF ? 1 : GT + 16;
  constexpr int B_RS = B_NF ? 1 : GK + 1, B_KS = B_NF ? GT + 16 : 1;
  extern __shared__ __attribute__((aligned(16))) double f64_lds[];  // [buffer][a, b][OP]
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int wm = wave / WN, wn = wave % WN;
  const int l16 = lane & 15, lk = lane >> 4;
  const int64_t bm = (int64_t)blockIdx.y * GT, bn = (int64_t)blockIdx.x * GT;
  double ra[PER], rb[PER];
  auto fetch = [&](int64_t k0) {
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int e = tid + THREADS * u;
      const int r = A_KF ? e / GK : e % GT, kk = A_KF ? e % GK : e / GT;
      const int64_t m = bm + r, k = k0 + kk;
      ra[u] = (m < M && k < K) ? A[m * a_rs + k * a_cs] : 0.0;
      const int c = B_NF ? e % GT : e / GK, kk2 = B_NF ? e / GT : e % GK;
      const int64_t n = bn + c, k2 = k0 + kk2;
      rb[u] = (n < N && k2 < K) ? B[k2 * b_rs + n * b_cs] : 0.0;
    }
  };
  auto park = [&](double* buf) {
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int e = tid + THREADS * u;
      const int r = A_KF ? e / GK : e % GT, kk = A_KF ? e % GK : e / GT;
      buf[r * A_RS + kk * A_KS] = ra[u];
      const int c = B_NF ? e % GT : e / GK, kk2 = B_NF ? e / GT : e % GK;
      buf[OP + c * B_RS + kk2 * B_KS] = rb[u];
    }
  };
  f64x4 acc[WBM][WBN];
#pragma unroll
  for (int i = 0; i < WBM; ++i)
#pragma unroll
    for (int j = 0; j < WBN; ++j) acc[i][j] = f64x4{0.0, 0.0, 0.0, 0.0};
  fetch(0);
  park(f64_lds);
  __syncthreads();
  int cur = 0;
  for (int64_t k0 = 0; k0 < K; k0 += GK) {
    const bool more = k0 + GK < K;
    if (more) fetch(k0 + GK);
    const double* as = f64_lds + cur * (2 * OP) + (wm * (16 * WBM) + l16) * A_RS + lk * A_KS;
    const double* bs = f64_lds + cur * (2 * OP) + OP + (wn * (16 * WBN) + l16) * B_RS + lk * B_KS;
#pragma unroll
    for (int k4 = 0; k4 < GK / 4; ++k4) {
      double av[WBM], bv[WBN];
#pragma unroll
      for (int i = 0; i < WBM; ++i) av[i] = as[i * 16 * A_RS + k4 * 4 * A_KS];
#pragma unroll
      for (int j = 0; j < WBN; ++j) bv[j] = bs[j * 16 * B_RS + k4 * 4 * B_KS];
#pragma unroll
      for (int i = 0; i < WBM; ++i)
#pragma unroll
        for (int j = 0; j < WBN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(av[i], bv[j], acc[i][j], 0, 0, 0);
    }
    cur ^= 1;
    if (more) park(f64_lds + cur * (2 * OP));  // the buffer every wave finished reading before the last barrier
    __syncthreads();
  }
  const bool use_c = C != nullptr && beta != 0.0;
#pragma unroll
  for (int i = 0; i < WBM; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int64_t m = bm + wm * (16 * WBM) + i * 16 + 4 * r + lk;
      if (m >= M) continue;
#pragma unroll
      for (int j = 0; j < WBN; ++j) {
        const int64_t n = bn + wn * (16 * WBN) + j * 16 + l16;
        if (n >= N) continue;
        double v = alpha * acc[i][j][r];
        if (use_c) v += beta * C[m * c_rs + n * c_cs];
        D[m * N + n] = v;
      }
    }
}

template <int WBM, int WBN, int WM, int WN>
static const void* pick_f64(bool a_kf, bool b_nf) {
  if (a_kf) return b_nf ? (const void*)gemm_f64_mfma_kernel<WBM, WBN, WM, WN, true, true> : (const void*)gemm_f64_mfma_kernel<WBM, WBN, WM, WN, true, false>;
  return b_nf ? (const void*)gemm_f64_mfma_kernel<WBM, WBN, WM, WN, false, true> : (const void*)gemm_f64_mfma_kernel<WBM, WBN, WM, WN, false, false>;
}

int launch_gemm_f64(const double* a, int64_t a_rs, int64_t a_cs, const double* b, int64_t b_rs, int64_t b_cs, const double* c,
                    int64_t c_rs, int64_t c_cs, double* out, int64_t M, int64_t N, int64_t K, double alpha, double beta,
                    hipStream_t st) {
  // 128x128 tiles once they still give every CU a block, else 64x64, and 32x32 (four waves) when even those
  // leave more than half of the CUs idle
  const bool big = ((M + 127) / 128) * ((N + 127) / 128) >= kNumCU;
  const bool tiny = !big && ((M + 63) / 64) * ((N + 63) / 64) < kNumCU / 2;
  const int64_t gt = big ? 128 : tiny ? 32 : 64;
  const int64_t gx = (N + gt - 1) / gt, gy = (M + gt - 1) / gt;
  MI355_REQUIRE(gy < 65536 && gx < (int64_t(1) << 31), "mi355_gemm: the fp64 path needs M < 2M rows");
  const bool a_kf = a_cs == 1 || a_rs != 1;  // consecutive threads along k, unless a is M-contiguous
  const bool b_nf = b_cs == 1 || b_rs != 1;  // consecutive threads along n, unless b is K-contiguous
  const void* kern = big ? pick_f64<2, 2, 4, 4>(a_kf, b_nf) : tiny ? pick_f64<1, 1, 2, 2>(a_kf, b_nf) : pick_f64<1, 1, 4, 4>(a_kf, b_nf);
  const int lds_bytes = f64_lds_bytes((int)gt);
  const unsigned threads = tiny ? 256 : 1024;
  static thread_local const void* attr_done[12] = {};  // kernels whose LDS limit has been raised
  bool seen = false;
  for (const void* k : attr_done) seen = seen || k == kern;
  if (!seen) {
    hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (e != hipSuccess)
      return set_error(MI355_ERR_LAUNCH, "mi355_gemm(f64): cannot reserve %d bytes of LDS: %s", lds_bytes, hipGetErrorString(e));
    for (const void*& k : attr_done)
      if (k == nullptr) { k = kern; break; }
  }
  void* params[] = {&a, &a_rs, &a_cs, &b, &b_rs, &b_cs, &c, &c_rs, &c_cs, &out, &M, &N, &K, &alpha, &beta};
  hipError_t e = hipLaunchKernel(kern, dim3((unsigned)gx, (unsigned)gy), dim3(threads), params, lds_bytes, st);
  if (e != hipSuccess) return set_error(MI355_ERR_LAUNCH, "mi355_gemm(f64 mfma): launch failed: %s", hipGetErrorString(e));
  return check_launch("mi355_gemm(f64 mfma)");
}

}  // namespace mi355
