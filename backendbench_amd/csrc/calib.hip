// Calibration kernel: the matrix-core instruction stream of the four-wave GEMM kernel with no
// memory traffic at all.  One wave per SIMD holds the register tile of gemm_mfma_w4_kernel (two
// sets of 2 x 4 A fragments and 2 x 4 B fragments, 256 fp32 accumulators) and issues the same 32
// v_mfma_f32_32x32x16 per 32-k step in the same order, alternating between the two fragment
// sets, for `steps` steps.  The fragments are loaded once from the caller's buffers, so the
// operand DATA is the caller's choice: the sustained rate of this loop on a given data
// distribution is what the chip's power / clock envelope leaves to any GEMM on that data, before
// a byte is moved.  mi355_calib_mfma only serves measurement (bench.py --only-op calib.mfma).
#include "common.h"

namespace mi355 {

typedef __bf16 cbf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 cf16x8 __attribute__((ext_vector_type(8)));
typedef float cf32x16 __attribute__((ext_vector_type(16)));
typedef float cf32x4 __attribute__((ext_vector_type(4)));

template <typename F> struct CalibMfma;
template <> struct CalibMfma<cbf16x8> {
  static __device__ __forceinline__ cf32x16 run32(cbf16x8 a, cbf16x8 b, cf32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ cf32x4 run16(cbf16x8 a, cbf16x8 b, cf32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
};
template <> struct CalibMfma<cf16x8> {
  static __device__ __forceinline__ cf32x16 run32(cf16x8 a, cf16x8 b, cf32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ cf32x4 run16(cf16x8 a, cf16x8 b, cf32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
};

// ORDER 0: the GEMM kernel's order (B fragment first operand, held over four MFMAs; A fragment
//          second, changing every MFMA).
// ORDER 1: operands swapped between the two ports.
// ORDER 2: second operand held over four MFMAs, first changing.
// ORDER 3: the four MFMAs of a pair of steps that feed one accumulator block issued back to back
//          (k innermost): every MFMA takes its addend from the one before it.
// ORDER 4: the same in chains of two (the two 16-k halves of one step).
template <typename F, int ORDER>
__global__ __launch_bounds__(256) void calib_mfma32_kernel(const F* __restrict__ a, const F* __restrict__ b, float* __restrict__ out, int steps) {
  const int64_t lane_slot = (int64_t)blockIdx.x * 256 + threadIdx.x;
  F xa[2][2][4], xb[2][2][4];
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        xa[s][ks][i] = a[lane_slot * 16 + (s * 2 + ks) * 4 + i];
        xb[s][ks][i] = b[lane_slot * 16 + (s * 2 + ks) * 4 + i];
      }
  cf32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  for (int t = 0; t < steps; t += 2) {
    if constexpr (ORDER == 3) {
#pragma unroll
      for (int p = 0; p < 4; ++p)
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) acc[q][p] = CalibMfma<F>::run32(xb[s][ks][p], xa[s][ks][q], acc[q][p]);
      continue;
    }
    if constexpr (ORDER == 4) {
#pragma unroll
      for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int p = 0; p < 4; ++p)
#pragma unroll
          for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) acc[q][p] = CalibMfma<F>::run32(xb[s][ks][p], xa[s][ks][q], acc[q][p]);
      continue;
    }
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int p = 0; p < 4; ++p)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            if constexpr (ORDER == 0) acc[q][p] = CalibMfma<F>::run32(xb[s][ks][p], xa[s][ks][q], acc[q][p]);
            else if constexpr (ORDER == 1) acc[q][p] = CalibMfma<F>::run32(xa[s][ks][q], xb[s][ks][p], acc[q][p]);
            else acc[p][q] = CalibMfma<F>::run32(xb[s][ks][q], xa[s][ks][p], acc[p][q]);
          }
  }
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) sum += acc[i][j][e];
  out[lane_slot] = sum;
}

// The same register tile on v_mfma_f32_16x16x32: 8 x 8 blocks of 16 x 16 (64 accumulators of four
// registers), eight A and eight B fragments per 32-k step, 64 MFMAs of half the work each.
template <typename F, bool CHAIN = false>
__global__ __launch_bounds__(256) void calib_mfma16_kernel(const F* __restrict__ a, const F* __restrict__ b, float* __restrict__ out, int steps) {
  const int64_t lane_slot = (int64_t)blockIdx.x * 256 + threadIdx.x;
  F xa[2][8], xb[2][8];
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      xa[s][i] = a[lane_slot * 16 + s * 8 + i];
      xb[s][i] = b[lane_slot * 16 + s * 8 + i];
    }
  cf32x4 acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[i][j][e] = 0.f;
  for (int t = 0; t < steps; t += 2) {
    if constexpr (CHAIN) {  // the two MFMAs of a pair of steps on one accumulator block back to back
#pragma unroll
      for (int p = 0; p < 8; ++p)
#pragma unroll
        for (int q = 0; q < 8; ++q)
#pragma unroll
          for (int s = 0; s < 2; ++s) acc[q][p] = CalibMfma<F>::run16(xb[s][p], xa[s][q], acc[q][p]);
      continue;
    }
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int p = 0; p < 8; ++p)
#pragma unroll
        for (int q = 0; q < 8; ++q) acc[q][p] = CalibMfma<F>::run16(xb[s][p], xa[s][q], acc[q][p]);
  }
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) sum += acc[i][j][e];
  out[lane_slot] = sum;
}

// 16x16x32 with chains of L MFMAs per accumulator block (L = 1, 2, 4): four k-sets of 4 + 4 fragments
// (two for L < 4), reused by all four 4 x 4 quadrants of the 8 x 8 block grid; the quadrants are
// walked one after the other (what a kernel that keeps one quadrant's fragments live would issue).
template <typename F, int L>
__global__ __launch_bounds__(256) void calib_mfma16q_kernel(const F* __restrict__ a, const F* __restrict__ b, float* __restrict__ out, int steps) {
  constexpr int NS = L == 4 ? 4 : 2;
  const int64_t lane_slot = (int64_t)blockIdx.x * 256 + threadIdx.x;
  F xa[NS][4], xb[NS][4];
#pragma unroll
  for (int s = 0; s < NS; ++s)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      xa[s][i] = a[lane_slot * 16 + s * 4 + i];
      xb[s][i] = b[lane_slot * 16 + s * 4 + i];
    }
  cf32x4 acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[i][j][e] = 0.f;
  for (int t = 0; t < steps; t += NS) {
#pragma unroll
    for (int g = 0; g < NS; g += L)
#pragma unroll
      for (int quad = 0; quad < 4; ++quad)
#pragma unroll
        for (int p = 0; p < 4; ++p)
#pragma unroll
          for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int s = g; s < g + L; ++s)
              acc[(quad >> 1) * 4 + q][(quad & 1) * 4 + p] =
                  CalibMfma<F>::run16(xb[s][p], xa[s][q], acc[(quad >> 1) * 4 + q][(quad & 1) * 4 + p]);
    __builtin_amdgcn_sched_barrier(0);
  }
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) sum += acc[i][j][e];
  out[lane_slot] = sum;
}

// The same quadrant walk with the MFMAs as asm statements, so that their order is exactly the written one:
// MODE 0: the two MFMAs on an accumulator block back to back; 1: an s_nop between the two; 2: two blocks
// interleaved (a0 b0 a1 b1: the addend comes from the MFMA before the last); 3: all first halves of a
// quadrant, then all second halves (the addend is 16 MFMAs old); 4: as 1 with three s_nop.
template <typename F, int MODE>
__global__ __launch_bounds__(256) void calib_mfma16a_kernel(const F* __restrict__ a, const F* __restrict__ b, float* __restrict__ out, int steps) {
  typedef uint32_t cu32x4 __attribute__((ext_vector_type(4)));
  const int64_t lane_slot = (int64_t)blockIdx.x * 256 + threadIdx.x;
  cu32x4 xa[2][4], xb[2][4];
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      xa[s][i] = __builtin_bit_cast(cu32x4, a[lane_slot * 16 + s * 4 + i]);
      xb[s][i] = __builtin_bit_cast(cu32x4, b[lane_slot * 16 + s * 4 + i]);
    }
  cf32x4 acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) {
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[i][j][e] = 0.f;
      asm volatile("" : "+a"(acc[i][j]));
    }
  constexpr bool BF = sizeof(a[0][0]) == 2 && !__is_same(F, cf16x8);
#define MI355_CALIB_M(C, B_, A_)                                                                                    \
  if constexpr (BF) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(C) : "v"(B_), "v"(A_));        \
  else asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(C) : "v"(B_), "v"(A_));
  for (int t = 0; t < steps; t += 2) {
#pragma unroll
    for (int quad = 0; quad < 4; ++quad) {
      const int i0 = (quad >> 1) * 4, j0 = (quad & 1) * 4;
      if constexpr (MODE == 3) {
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
          for (int c = 0; c < 16; ++c) { MI355_CALIB_M(acc[i0 + (c & 3)][j0 + (c >> 2)], xb[s][c >> 2], xa[s][c & 3]) }
      } else if constexpr (MODE == 2) {
#pragma unroll
        for (int c = 0; c < 16; c += 2) {
          MI355_CALIB_M(acc[i0 + (c & 3)][j0 + (c >> 2)], xb[0][c >> 2], xa[0][c & 3])
          MI355_CALIB_M(acc[i0 + ((c + 1) & 3)][j0 + (c >> 2)], xb[0][c >> 2], xa[0][(c + 1) & 3])
          MI355_CALIB_M(acc[i0 + (c & 3)][j0 + (c >> 2)], xb[1][c >> 2], xa[1][c & 3])
          MI355_CALIB_M(acc[i0 + ((c + 1) & 3)][j0 + (c >> 2)], xb[1][c >> 2], xa[1][(c + 1) & 3])
        }
      } else {
#pragma unroll
        for (int c = 0; c < 16; ++c) {
          MI355_CALIB_M(acc[i0 + (c & 3)][j0 + (c >> 2)], xb[0][c >> 2], xa[0][c & 3])
          if constexpr (MODE == 1) asm volatile("s_nop 0");
          if constexpr (MODE == 4) asm volatile("s_nop 0\n\ts_nop 0\n\ts_nop 0");
          MI355_CALIB_M(acc[i0 + (c & 3)][j0 + (c >> 2)], xb[1][c >> 2], xa[1][c & 3])
        }
      }
    }
  }
#undef MI355_CALIB_M
  asm volatile("s_nop 15\n\ts_nop 15");
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) sum += acc[i][j][e];
  out[lane_slot] = sum;
}

// fp64: WAVES waves per workgroup, each issuing `steps` rounds of eight independent v_mfma_f64_16x16x4_f64
// (2048 flop each) on one operand value per lane.
typedef double calib_f64x4 __attribute__((ext_vector_type(4)));
template <int WAVES>
__global__ __launch_bounds__(64 * WAVES) void calib_mfma_f64_kernel(const double* __restrict__ a, const double* __restrict__ b,
                                                                  float* __restrict__ out, int steps) {
  calib_f64x4 acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = calib_f64x4{0.0, 0.0, 0.0, 0.0};
  const double av = a[threadIdx.x % 256], bv = b[threadIdx.x % 256];
  for (int s = 0; s < steps; ++s) {
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_f64_16x16x4f64(av, bv, acc[i], 0, 0, 0);
  }
  double t = 0.0;
#pragma unroll
  for (int i = 0; i < 8; ++i) t += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
  if (threadIdx.x < 256) out[blockIdx.x * 256 + threadIdx.x] = static_cast<float>(t);
}

}  // namespace mi355

using namespace mi355;

// blocks x 256 threads, each wave issuing `steps` (even) 32-k steps of a 128 x 128 register tile:
// 2 * 128 * 128 * 32 flop per wave and step.  a, b: 16 fragments of 16 bytes per thread
// (blocks * 256 * 256 bytes each); out: blocks * 256 floats.  variant 0..2: 32x32x16 in the three
// operand orders, 3: 16x16x32, 4 / 5: 32x32x16 with the MFMAs on one accumulator block chained in
// fours / twos, 6: 16x16x32 chained in twos, 7 / 8 / 9: 16x16x32 walked quadrant by quadrant in chains
// of 1 / 2 / 4 (steps % 4 == 0), 10 .. 14: the quadrant walk in chains of two as asm statements in exactly
// the written order: back to back / an s_nop between the two / two blocks interleaved / all first halves
// then all second halves / three s_nop between the two.
extern "C" int mi355_calib_mfma(const void* a, const void* b, void* out, int dtype, int blocks, int steps, int variant,
                                void* stream) {
  MI355_REQUIRE(a != nullptr && b != nullptr && out != nullptr, "mi355_calib_mfma: NULL buffer");
  MI355_REQUIRE(blocks > 0 && steps > 0 && steps % 4 == 0, "mi355_calib_mfma: blocks > 0 and a number of steps divisible by four");
  if (dtype == MI355_F64) {  // variant = waves per workgroup; a, b: 256 doubles each
    const double* pa = static_cast<const double*>(a);
    const double* pb = static_cast<const double*>(b);
    float* of = static_cast<float*>(out);
    hipStream_t sf = static_cast<hipStream_t>(stream);
    switch (variant) {
      case 1: hipLaunchKernelGGL((calib_mfma_f64_kernel<1>), dim3(blocks), dim3(64), 0, sf, pa, pb, of, steps); break;
      case 4: hipLaunchKernelGGL((calib_mfma_f64_kernel<4>), dim3(blocks), dim3(256), 0, sf, pa, pb, of, steps); break;
      case 8: hipLaunchKernelGGL((calib_mfma_f64_kernel<8>), dim3(blocks), dim3(512), 0, sf, pa, pb, of, steps); break;
      case 16: hipLaunchKernelGGL((calib_mfma_f64_kernel<16>), dim3(blocks), dim3(1024), 0, sf, pa, pb, of, steps); break;
      default: return set_error(MI355_ERR_INVALID, "mi355_calib_mfma: f64 takes 1, 4, 8 or 16 waves per workgroup as variant");
    }
    return check_launch("mi355_calib_mfma(f64)");
  }
  MI355_REQUIRE(dtype == MI355_BF16 || dtype == MI355_F16, "mi355_calib_mfma: bf16, f16 or f64");
  MI355_REQUIRE(variant >= 0 && variant <= 14, "mi355_calib_mfma: variant 0..14");
  hipStream_t st = static_cast<hipStream_t>(stream);
  float* o = static_cast<float*>(out);
#define MI355_CALIB(F_)                                                                                                        \
  {                                                                                                                            \
    const F_* pa = static_cast<const F_*>(a);                                                                                  \
    const F_* pb = static_cast<const F_*>(b);                                                                                  \
    switch (variant) {                                                                                                         \
      case 0: hipLaunchKernelGGL((calib_mfma32_kernel<F_, 0>), dim3(blocks), dim3(256), 0, st, pa, pb, o, steps); break;       \
      case 1: hipLaunchKernelGGL((calib_mfma32_kernel<F_, 1>), dim3(blocks), dim3(256), 0, st, pa, pb, o, steps); break;       \
      case 2: hipLaunchKernelGGL((calib_mfma32_kernel<F_, 2>), dim3(blocks), dim3(256), 0, st, pa, pb, o, steps); break;       \
      case 3: hipLaunchKernelGGL((calib_mfma16_kernel<F_>), dim3(blocks), dim3(256), 0, st, pa, pb, o, steps); break;          \
      case 4: hipLaunchKernelGGL((calib_mfma32_kernel<F_, 3>), dim3(blocks), dim3(256), 0, st, pa, pb, o, steps); break;       \
      case 5: hipLaunchKernelGGL((calib_mfma32_kernel<F_, 4>), dim3(blocks), dim3(256), 0, st, pa, pb, o, steps); break;       \
      case 6: hipLaunchKernelGGL((calib_mfma16_kernel<F_, true>), dim3(blocks), dim3(256), 0, st, pa, pb, o, steps); break;    \
      case 7: hipLaunchKernelGGL((calib_mfma16q_kernel<F_, 1>), dim3(blocks), dim3(256), 0, st, pa, pb, o, steps); break;      \
      case 8: hipLaunchKernelGGL((calib_mfma16q_kernel<F_, 2>), dim3(blocks), dim3(256), 0, st, pa, pb, o, steps); break;      \
      case 9: hipLaunchKernelGGL((calib_mfma16q_kernel<F_, 4>), dim3(blocks), dim3(256), 0, st, pa, pb, o, steps); break;      \
      case 10: hipLaunchKernelGGL((calib_mfma16a_kernel<F_, 0>), dim3(blocks), dim3(256), 0, st, pa, pb, o, steps); break;     \
      case 11: hipLaunchKernelGGL((calib_mfma16a_kernel<F_, 1>), dim3(blocks), dim3(256), 0, st, pa, pb, o, steps); break;     \
      case 12: hipLaunchKernelGGL((calib_mfma16a_kernel<F_, 2>), dim3(blocks), dim3(256), 0, st, pa, pb, o, steps); break;     \
      case 13: hipLaunchKernelGGL((calib_mfma16a_kernel<F_, 3>), dim3(blocks), dim3(256), 0, st, pa, pb, o, steps); break;     \
      default: hipLaunchKernelGGL((calib_mfma16a_kernel<F_, 4>), dim3(blocks), dim3(256), 0, st, pa, pb, o, steps); break;     \
    }                                                                                                                          \
  }
  if (dtype == MI355_BF16) MI355_CALIB(cbf16x8) else MI355_CALIB(cf16x8)
#undef MI355_CALIB
  return check_launch("mi355_calib_mfma");
}
