// mm / addmm on v_mfma_f32_16x16x32: 256x256 tiles, four waves of 128x128 (8 x 8 blocks of 16x16, 256
// fp32 accumulators per lane), bf16 / f16, K % 128 == 0, K >= 256, a K-contiguous, b K-contiguous or row-major.
//
// Why a second form of the four-wave kernel.  On real operand data the GEMM is bound by the power
// envelope, not by issue slots: the clock falls when a kernel does more per cycle.  The MFMA stream
// alone (mi355_calib_mfma) sustains 1.77 PFLOP/s with v_mfma_f32_32x32x16 and 1.96 - 1.99 with
// v_mfma_f32_16x16x32 when the two MFMAs that feed one accumulator block from a 64-k stage are issued
// back to back (the second takes its addend from the first inside the matrix core).  This kernel is
// built around that order.
//
// A 64-k stage of a wave's tile is walked in four quadrants of 4 x 4 blocks, 32 MFMAs each (16 blocks
// x 2 chained 32-k halves).  A quadrant needs one "set" of A fragments (4 row blocks x 2 halves, 32
// VGPRs) and one set of B fragments; neighbouring quadrants share one of the two, so each quadrant
// loads exactly one new set from LDS while it computes, and four sets (128 VGPRs) are live:
//     even stage S:  (B0,A0) (B0,A1) (B1,A1) (B1,A0)      odd stage:  (B0,A1) (B0,A0) (B1,A0) (B1,A1)
//     loads:           A1(S)   B1(S)  B0(S+1) A1(S+1)                   A0(S)   B1(S)  B0(S+1) A0(S+1)
// LDS therefore holds the operands as "pairs": one A sub-panel (the 64 + 64 rows that the two wave rows
// load as one set, 64 k: 16 KB) plus one B sub-panel, in the order they are read: pair 2S = {A_h(S),
// B0(S)}, pair 2S+1 = {A_(1-h)(S), B1(S)}, h = S % 2.  A ring of five 32 KB pairs; during half-stage t
// (two quadrants, 64 MFMAs) every wave reads pair t+1, requests pair t+5 into the slot pair t left
// (eight global_load_lds_dwordx4 per lane) and then waits until only the 24 requests of pairs t+3..t+5
// are in flight, so every pair has three half-stages (about 2 us) to arrive.
#include <type_traits>

#include "gemm_shared.h"

// Timing-only ablations for measurement builds (python -m backendbench_amd._build --ablate N, bench.py
// --only-op C3.mm_down --ablate N): results are wrong, the product library is built with 0.  Bits: 1 no fill
// requests in the K loop, 2 no barriers, 4 no LDS fragment reads, 8 no wait for the fills, 16 no global
// stores in the epilogue, 32 no epilogue; split K: 64 producers store no plane, 128 the summing workgroup neither
// waits nor reads planes, 1024 wall-clock stamps of
// every workgroup's phases behind the flags (eight 64-bit words per block: entry, K loop done, plane stored /
// flags seen, end, role, XCC id).
#ifndef MI355_X16_ABLATE
#define MI355_X16_ABLATE 0
#endif

namespace mi355 {

template <typename T> struct Mfma16;
template <> struct Mfma16<bf16_t> {
  using frag = bf16x8;
  static __device__ __forceinline__ f32x4 run(frag a, frag b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
};
template <> struct Mfma16<f16_t> {
  using frag = f16x8;
  static __device__ __forceinline__ f32x4 run(frag a, frag b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
};

constexpr int kXSub = 128 * 64 * 2;  // one operand's half of a 64-k stage
constexpr int kXPair = 2 * kXSub;
constexpr int kXSlots = 5;
static_assert(kXSlots * kXPair == kX16Lds, "ring size");

// K-contiguous sub-panel: 128 rows of 128 B; 16-byte chunk c of row r sits at chunk c ^ ((r / 2) % 8), so
// that the 16 rows x one chunk of a fragment read fall into 16 distinct 16-byte columns of the 256-byte
// bank window.
__device__ __forceinline__ int xswz_k(int r, int c) { return r * 128 + ((c ^ ((r >> 1) & 7)) << 4); }
// Row-major B sub-panel: 64 k-rows of 256 B (128 columns); the 32-byte segment (16 columns) index is
// XORed with (k % 4) | ((k / 8) % 2) * 4: the 4 + 4 k-rows that 32 lanes of a transposing read touch
// land in eight distinct segments.
__device__ __forceinline__ int xswz_seg(int k) { return (k & 3) | (((k >> 3) & 1) << 2); }

// Split-K inside one launch (gemm_mfma_x16_splitk_kernel): `role` 1 .. nprod are the producers of a tile -
// each leaves its raw fp32 accumulators in its plane (register order, x16_plane_store), then raises its flag; role 0 sums
// the planes into its own accumulators and runs the epilogue.  Producers never wait and sit in front of the
// summing workgroups in block order, so whatever shares the chip with this launch cannot make it wait for a
// workgroup that has not been dispatched.
struct X16Split {
  f32x4* planes;              // this tile's planes (role 0) or this producer's plane (role > 0)
  unsigned long long* flags;  // likewise
  unsigned long long epoch;
  int role, nprod;
  int spin_limit;  // polls of one flag before the summing workgroup gives up
};
// Set by a summing workgroup whose bounded wait ran out (it then writes NaNs into its tile): the launch
// still reports success, so this word is how the host learns of it (mi355_gemm_status).  Sticky until read.
static __device__ unsigned int x16_gave_up_word;

// Plane accesses are agent-scope accesses (the sc1 bit on the instruction), not plain ones between agent-scope
// fences: a fence writes back / invalidates the whole L2 of the XCD, under the feet of the workgroups that
// are still in their K loops (measured: 89 us instead of 64 for the product it was meant to speed up).
// They are buffer instructions of 16 bytes per lane (bit 4 of the cache policy operand is sc1), ordered against the flag by
// the producer's wait for its stores and the summing workgroup's barrier behind the poll.  Block (i, j) of wave
// w: 1 KB at byte (w * 64 + 8 i + j) * 1024 of the plane, lane l's four values at 16 l (register order).
constexpr int kX16Sc1 = 1 << 4;
__device__ __forceinline__ __amdgpu_buffer_rsrc_t x16_plane_rsrc(f32x4* planes, int nplanes) {
  return __builtin_amdgcn_make_buffer_rsrc(planes, 0, nplanes * (BM * BN * 4), 0x00020000);  // raw bytes, bounds-checked
}
__device__ __forceinline__ void x16_plane_store(__amdgpu_buffer_rsrc_t planes, int block, int lane, const f32x4& v) {
  if constexpr ((MI355_X16_ABLATE & 64) != 0) return;
  __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), planes, lane * 16, block * 1024, kX16Sc1);
}
// The summing workgroup (role 0, once the flags are up) adds the producers' values to its own on the way out, in
// the epilogue: what the NPROD producers hold for accumulator block (i, j) of this wave, summed.  The epilogue
// asks for x16_part_rows<NPROD>() rows of a half's blocks at a time - as many as 128 VGPRs hold - and all their
// loads are issued before the first value is used: the planes come over at the latency of one batch after the
// other (1.4 us each, measured), so few large batches are what makes the exchange cheap (two rows at a time took
// 11 us for one plane).  NPROD is a constant: with a run-time count every plane's load is waited for before the
// next one is issued.  The accumulators stay in the AGPRs until their block's turn (pinned there at the use),
// which is what leaves the VGPRs free for the values in flight.
template <int NPROD>
constexpr int x16_part_rows() { return NPROD <= 1 ? 8 : NPROD == 2 ? 4 : 2; }
struct X16Planes {
  __amdgpu_buffer_rsrc_t rsrc;
  float poison;  // -0 (x + -0 == x), or NaN when a producer never arrived
};
template <int NPROD>
__device__ __forceinline__ f32x4 x16_split_partial(const X16Planes& pl, int wave, int lane, int i, int j) {
  const int block = (wave * 64 + i * 8 + j) * 1024;
  f32x4 v[NPROD > 0 ? NPROD : 1];
#pragma unroll
  for (int q = 0; q < NPROD; ++q)
    v[q] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(pl.rsrc, lane * 16, block + q * (BM * BN * 4), kX16Sc1));
#pragma unroll
  for (int q = 1; q < NPROD; ++q) v[0] += v[q];
  v[0][0] += pl.poison;
  return v[0];
}

// Epilogue: the wave's 128 x 32 NPQ result, 16 NPQ columns at a time, through a 16 KB slab of the idle ring
// (rows of 128 B, 16-byte slot s of row r at s ^ ((r / 2) % 8)) and out in whole 128-byte rows.
// Register e of acc[i][j] in lane l is C[m0 + 16 i + l % 16][n0 + 16 j + 4 (l / 16) + e] (operands swapped).
template <typename T, int NPQ, int RH = 1, int NPROD = 0>
__device__ __forceinline__ void store_tile_result16(const GemmArgs& g, f32x4 (&acc)[8][2 * NPQ], unsigned char* lds,
                                                    int wave, int lane, int m0, int n0, const X16Planes* pl = nullptr) {
  static_assert(RH == 1 || RH == 2, "the slab holds all 128 rows of the wave's tile or 64 at a time");
  constexpr int IB = 8 / RH;  // row blocks per pass
  const int lr = lane & 15, lg = lane >> 4;
  const T* C = static_cast<const T*>(g.c);
  const bool use_c = C != nullptr && g.beta != 0.f;
  const bool row_bias = use_c && (RH == 1 ? g.bias_vec != 0 : g.c_vec && g.c_rs == 0);  // (whole tiles in the persistent form: N % 4 == 0)
  unsigned char* slab = lds + wave * (128 * 128 / RH);
  T* D = static_cast<T*>(g.out);
  const bool inside = NPQ == 4 && m0 + 128 <= g.M && n0 + 128 <= g.N;  // no row or column of this wave's tile is cut
  // MODE 0: alpha * acc; 1: + beta * a bias row (loaded once per 64 columns); 2: + beta * c.  The mode is
  // chosen once per call, outside the loops over the accumulator blocks.
  // The bias row of a half's 16 NPQ columns.  One workgroup per tile (RH == 1): both halves are loaded before
  // anything is staged, one exposed load latency per tile instead of two.  The persistent form (RH == 2)
  // keeps the next tile's first fragments in registers across its epilogue and has no room for that.
  auto load_bias = [&](int y, float (&bias)[NPQ][4]) __attribute__((always_inline)) {
#pragma unroll
    for (int p = 0; p < NPQ; ++p) {
      const int n = n0 + y * (16 * NPQ) + p * 16 + lg * 4;
      const VecN4<T> t = *reinterpret_cast<const VecN4<T>*>(C + (n + 4 <= g.N ? n : 0));
#pragma unroll
      for (int e = 0; e < 4; ++e) bias[p][e] = g.beta * static_cast<float>(t.v[e]);
      if constexpr (RH == 1) {  // (the persistent form walks whole tiles)
        if (n < g.N && n + 4 > g.N) {  // the last columns of an N that is no multiple of 4
#pragma unroll
          for (int e = 0; e < 4; ++e) bias[p][e] = g.beta * static_cast<float>(C[n + e < g.N ? n + e : g.N - 1]);
        }
      }
    }
  };
  float bias2[RH == 1 ? 2 : 1][NPQ][4];
  if constexpr (RH == 1) {
    if (row_bias) {
      load_bias(0, bias2[0]);
      load_bias(1, bias2[1]);
    }
  }
  auto half = [&](auto MODE_, int y, int rh) __attribute__((always_inline)) {
    constexpr int MODE = decltype(MODE_)::value;
    const int nh = n0 + y * (16 * NPQ);
    float (&bias)[NPQ][4] = bias2[RH == 1 ? y : 0];
    if constexpr (MODE == 1 && RH != 1) load_bias(y, bias);
    unsigned char* wr = slab + lr * 128 + (lg & 1) * 8;
    const int sx = (lr >> 1) & 7;  // = (row / 2) % 8 for every row 16 i + lr
    // split K: what the producers hold for PR rows of this half's blocks at a time
    constexpr bool SPLITK = NPROD > 0;  // the summing workgroup of a K split over NPROD + 1 workgroups
    constexpr int PR = SPLITK ? x16_part_rows<NPROD>() : 1;
    f32x4 part[PR][SPLITK ? NPQ : 1];
#pragma unroll
    for (int ii = 0; ii < IB; ++ii) {
      const int i = rh * IB + ii;
      if constexpr (SPLITK) {
        if (ii % PR == 0) {
#pragma unroll
          for (int u = 0; u < PR; ++u)
#pragma unroll
            for (int p = 0; p < NPQ; ++p) part[u][p] = x16_split_partial<NPROD>(*pl, wave, lane, i + u, (y ? NPQ : 0) + p);
        }
      }
      const int m = m0 + i * 16 + lr;
      const int mc = m < g.M ? m : g.M - 1;
#pragma unroll
      for (int p = 0; p < NPQ; ++p) {
        const int nl = p * 16 + lg * 4;
        const int n = nh + nl;
        if constexpr (SPLITK) asm volatile("" : "+a"(acc[i][(y ? NPQ : 0) + p]));
        f32x4 v = acc[i][(y ? NPQ : 0) + p];
        if constexpr (SPLITK) v += part[ii % PR][p];
        VecN4<T> r;
        if constexpr (MODE == 0) {
#pragma unroll
          for (int e = 0; e < 4; ++e) r.v[e] = static_cast<T>(g.alpha * v[e]);
        } else if constexpr (MODE == 1) {
#pragma unroll
          for (int e = 0; e < 4; ++e) r.v[e] = static_cast<T>(g.alpha * v[e] + bias[p][e]);
        } else {
          float cv[4];  // columns past N are computed on valid addresses and never stored
          if (g.c_vec) {
            const int nv = n + 4 <= g.N ? n : 0;
            const VecN4<T> t = *reinterpret_cast<const VecN4<T>*>(C + (int64_t)mc * g.c_rs + nv);
#pragma unroll
            for (int e = 0; e < 4; ++e) cv[e] = static_cast<float>(t.v[e]);
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int ne = n + e < g.N ? n + e : g.N - 1;
              cv[e] = static_cast<float>(C[(int64_t)mc * g.c_rs + (int64_t)ne * g.c_cs]);
            }
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) r.v[e] = static_cast<T>(g.alpha * v[e] + g.beta * cv[e]);
        }
        *reinterpret_cast<VecN4<T>*>(wr + ii * (16 * 128) + (((p * 2 + (lg >> 1)) ^ sx) << 4)) = r;
      }
    }
    // same wave wrote and reads: LDS operations of a wave complete in order
    if (g.out_vec) {
      const int s = lane & 7, r0 = lane >> 3;  // 16-byte chunk s of rows r0 + 8 t
      const unsigned char* rdp = slab + r0 * 128;
      T* dst = D + (int64_t)(m0 + rh * (16 * IB) + r0) * g.N + nh + s * 8;
      if (inside) {
#pragma unroll
        for (int t = 0; t < 2 * IB; ++t) {
          const int row = r0 + 8 * t;  // (row / 2) % 8 = (r0 / 2 + 4 t) % 8
          const u32x4 v = *reinterpret_cast<const u32x4*>(rdp + t * 1024 + ((s ^ (((r0 >> 1) + 4 * t) & 7)) << 4));
          if ((MI355_X16_ABLATE & 16) && v[0] != 0x12345678u) continue;
          *reinterpret_cast<u32x4*>(dst + (int64_t)(8 * t) * g.N) = v;
          (void)row;
        }
      } else {
#pragma unroll
        for (int t = 0; t < 2 * IB; ++t) {
          const int row = r0 + 8 * t;
          const u32x4 v = *reinterpret_cast<const u32x4*>(rdp + t * 1024 + ((s ^ ((row >> 1) & 7)) << 4));
          if (m0 + rh * (16 * IB) + row >= g.M || nh + s * 8 >= g.N || s >= 2 * NPQ) continue;
          *reinterpret_cast<u32x4*>(dst + (int64_t)(8 * t) * g.N) = v;
        }
      }
    } else if constexpr (RH == 1) {  // (the persistent form is only launched on vector stores)
      // output rows at any 2-byte offset (N % 8 != 0): the lanes walk the 16-byte grid of the destination
      const int mh = m0 + rh * (16 * IB);
      const int rows = g.M - mh < 16 * IB ? g.M - mh : 16 * IB;
      const int cols = g.N - nh < 16 * NPQ ? g.N - nh : 16 * NPQ;
      store_slab_rows_shifted<T, 16 * IB>(slab, D, g.N, mh, rows, nh, cols, lane);
    }
  };
  auto all = [&](auto MODE_) __attribute__((always_inline)) {
#pragma unroll
    for (int rh = 0; rh < RH; ++rh) {
      half(MODE_, 0, rh);
      half(MODE_, 1, rh);
    }
  };
  if (!use_c) all(std::integral_constant<int, 0>{});
  else if (row_bias) all(std::integral_constant<int, 1>{});
  else all(std::integral_constant<int, 2>{});
}

// Epilogue of the one-workgroup-per-tile kernel for output rows that do not start on 128-byte lines
// (N % 64 != 0: a 50264- or 50257-wide vocabulary).  With one slab per wave every store instruction writes
// 128-byte pieces that straddle two lines of the destination, each line is completed by another wave's
// stores later, and the 4 MB of L2 behind the 32 CUs of an XCD write many of them back half-filled in
// between (WRITE_SIZE reads 1.34 x the output bytes, [8192,768]x[768,50264] takes 812 us against 620 us at
// N = 50240).  Here the four waves park the whole 256 x 256 tile in the (idle) ring as rows of 512 bytes
// (16-byte slot s of row r at s ^ (r % 32)) and every store instruction then writes two whole tile rows:
// three complete lines and the two pieces a row shares with the neighbouring tiles.  Rows at any 2-byte
// offset (N % 8 != 0) go out along the destination's 16-byte grid (store_slab_rows_shifted).
template <typename T, int NPROD = 0>
__device__ __forceinline__ void store_tile_rows16(const GemmArgs& g, f32x4 (&acc)[8][8], unsigned char* lds, int wave,
                                                  int lane, int bm, int bn, const X16Planes* pl = nullptr) {
  const int wm = wave >> 1, wn = wave & 1;
  const int lr = lane & 15, lg = lane >> 4;
  const T* C = static_cast<const T*>(g.c);
  const bool use_c = C != nullptr && g.beta != 0.f;
  const bool row_bias = use_c && g.bias_vec;
  auto stage = [&](auto MODE_) __attribute__((always_inline)) {
    constexpr int MODE = decltype(MODE_)::value;
    float bias2[2][4][4];  // the bias row of the wave's 128 columns, loaded before anything is staged
    if constexpr (MODE == 1) {
#pragma unroll
      for (int y = 0; y < 2; ++y)
#pragma unroll
        for (int p = 0; p < 4; ++p) {
          const int n = bn + wn * 128 + y * 64 + p * 16 + lg * 4;
          const VecN4<T> t = *reinterpret_cast<const VecN4<T>*>(C + (n + 4 <= g.N ? n : 0));
#pragma unroll
          for (int e = 0; e < 4; ++e) bias2[y][p][e] = g.beta * static_cast<float>(t.v[e]);
          if (n < g.N && n + 4 > g.N) {  // the last columns of an N that is no multiple of 4
#pragma unroll
            for (int e = 0; e < 4; ++e) bias2[y][p][e] = g.beta * static_cast<float>(C[n + e < g.N ? n + e : g.N - 1]);
          }
        }
    }
#pragma unroll
    for (int y = 0; y < 2; ++y) {
      const int nh = bn + wn * 128 + y * 64;
      const float (&bias)[4][4] = bias2[y];
      constexpr bool SPLITK = NPROD > 0;
      constexpr int PR = SPLITK ? x16_part_rows<NPROD>() : 1;
      f32x4 part[PR][SPLITK ? 4 : 1];  // split K: what the producers hold for PR rows of this half's blocks at a time
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if constexpr (SPLITK) {
          if (i % PR == 0) {
#pragma unroll
            for (int u = 0; u < PR; ++u)
#pragma unroll
              for (int p = 0; p < 4; ++p) part[u][p] = x16_split_partial<NPROD>(*pl, wave, lane, i + u, y * 4 + p);
          }
        }
        const int row = wm * 128 + i * 16 + lr;
        const int m = bm + row;
        const int mc = m < g.M ? m : g.M - 1;
        unsigned char* wr = lds + row * 512 + (lg & 1) * 8;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
          const int n = nh + p * 16 + lg * 4;
          if constexpr (SPLITK) asm volatile("" : "+a"(acc[i][y * 4 + p]));
          f32x4 v = acc[i][y * 4 + p];
          if constexpr (SPLITK) v += part[i % PR][p];
          VecN4<T> r;
          if constexpr (MODE == 0) {
#pragma unroll
            for (int e = 0; e < 4; ++e) r.v[e] = static_cast<T>(g.alpha * v[e]);
          } else if constexpr (MODE == 1) {
#pragma unroll
            for (int e = 0; e < 4; ++e) r.v[e] = static_cast<T>(g.alpha * v[e] + bias[p][e]);
          } else {
            float cv[4];  // columns past N are computed on valid addresses and never stored
            if (g.c_vec) {
              const int nv = n + 4 <= g.N ? n : 0;
              const VecN4<T> t = *reinterpret_cast<const VecN4<T>*>(C + (int64_t)mc * g.c_rs + nv);
#pragma unroll
              for (int e = 0; e < 4; ++e) cv[e] = static_cast<float>(t.v[e]);
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                const int ne = n + e < g.N ? n + e : g.N - 1;
                cv[e] = static_cast<float>(C[(int64_t)mc * g.c_rs + (int64_t)ne * g.c_cs]);
              }
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) r.v[e] = static_cast<T>(g.alpha * v[e] + g.beta * cv[e]);
          }
          const int slot = wn * 16 + (y * 4 + p) * 2 + (lg >> 1);
          *reinterpret_cast<VecN4<T>*>(wr + ((slot ^ (row & 31)) << 4)) = r;
        }
      }
    }
  };
  if (!use_c) stage(std::integral_constant<int, 0>{});
  else if (row_bias) stage(std::integral_constant<int, 1>{});
  else stage(std::integral_constant<int, 2>{});
  __syncthreads();
  // wave w stores rows 64 w .. 64 w + 63 of the tile, two per instruction
  T* D = static_cast<T*>(g.out);
  const int r0 = wave * 64;
  const int rows = g.M - (bm + r0) < 64 ? g.M - (bm + r0) : 64;
  const int cols = g.N - bn < 256 ? g.N - bn : 256;
  if (g.out_vec) {
    const int s = lane & 31;
#pragma unroll 8
    for (int t = 0; t < 32; ++t) {
      const int row = r0 + 2 * t + (lane >> 5);
      const u32x4 v = *reinterpret_cast<const u32x4*>(lds + row * 512 + ((s ^ (row & 31)) << 4));
      if (2 * t + (lane >> 5) < rows && 8 * s < cols) *reinterpret_cast<u32x4*>(D + (int64_t)(bm + row) * g.N + bn + 8 * s) = v;
    }
  } else {
    store_slab_rows_shifted<T, 64, 32>(lds + r0 * 512, D, g.N, bm + r0, rows, bn, cols, lane);
  }
}

// Fill requests.  x16_set_m0 sets the LDS base of the requests behind it; request i of a group of four
// lands 1024 i bytes further (the instruction offset, which also moves the global address: the lane
// offsets take it back out).
__device__ __forceinline__ void x16_set_m0(uint32_t lds_byte_offset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0" ::"s"(lds_byte_offset) : "memory");
}
template <int I>
__device__ __forceinline__ void x16_fill(uint32_t lane_byte_offset, const void* base) {
  asm volatile("global_load_lds_dwordx4 %0, %1 offset:%2" ::"v"(lane_byte_offset), "s"(base), "n"(1024 * I) : "memory");
}
constexpr int kXBias = 3072;  // the bases point this many bytes low, so that lane offset - 1024 i stays non-negative

// NPQ = 4: a 256 x 256 tile.  NPQ = 3: a 256 x 192 tile on the same LDS layout and fill requests - a wave
// owns 96 columns, 48 per half, its quadrants are 4 x 3 blocks (24 MFMAs), and the 16 columns per
// half-wave that the B sub-panels hold beyond that are fetched (the next columns, clamped at the matrix
// edge) and not used.  Such tiles let a last, partly filled round of tiles be cut to fit the chip.
//
// PERSIST: the workgroup walks the tiles blockIdx.x, blockIdx.x + gridDim.x, ... (bm, bn are ignored) and
// its fill requests run on as one stream across them: the last five half-stages of a tile request the
// first five pairs of the next one, its last half-stage reads the next tile's first fragments, and the
// next K loop starts the moment the epilogue has issued its stores - no prologue latency, no gap between
// workgroups, and the stores drain while the next tile computes.  The epilogue borrows the one ring slot
// that is free at that point (the pair just read), 64 rows of the wave's tile at a time.  Every tile is
// whole (no clamped rows, so the lane offsets are the same for every tile): when M or N is no multiple of 256
// the last row / column of tiles overlaps its neighbour.  Vector stores only.
template <typename T, bool B_NN, int NPQ, bool PERSIST = false, bool SPLITK = false>
__device__ __forceinline__ void x16_tile(const GemmArgs& g, unsigned char* lds, int bm, int bn, const X16Split& sk = X16Split{}) {
  static_assert(NPQ == 3 || NPQ == 4, "wave tile is 128 x 32 NPQ");
  static_assert(!PERSIST || NPQ == 4, "the persistent form walks 256 x 256 tiles");
  using frag_t = typename Mfma16<T>::frag;
  constexpr int WCOLS = 32 * NPQ, HCOLS = 16 * NPQ;  // columns per wave and per half
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave >> 1, wn = wave & 1;
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;
  [[maybe_unused]] uint64_t st_entry = 0, st_loop = 0, st_met = 0;
  if constexpr (SPLITK && (MI355_X16_ABLATE & 1024) != 0) st_entry = __builtin_amdgcn_s_memrealtime();
#ifdef MI355_GEMM_TRACE
  // Diagnostic build only (-DMI355_GEMM_TRACE, libmi355_gemm_trace.so): shader-clock stamps (s_memtime,
  // read behind the next barrier's wait, so no wait is added).  Lane 0 of every wave leaves 16 uint64 in
  // the caller's workspace at ((block * 4 + wave) * 16), the layout of the stamps in gemm.hip:
  //   [0..5]  sums over the half-stages that end in a wait and a barrier (all but the last two), for the
  //           even and the odd ones: ticks issuing the half-stage's MFMAs / reads / requests, ticks in
  //           s_waitcnt for the requests, ticks from there to behind the barrier;
  //   [6] ticks in the K loop   [7] pairs of half-stages summed
  //   [10] stamp at loop entry   [11] HW_ID   [12] stamp at tile entry   [13], [14] at the end of the
  //   K loop   [15] when the tile's stores have completed.
  const uint64_t tr_entry = __builtin_readcyclecounter();
  uint64_t tr_sum[6] = {0, 0, 0, 0, 0, 0};
  uint64_t tr_start[2] = {0, 0}, tr_p2_prev = 0, tr_pairs = 0;
#endif

  // Fill addresses: a uniform base per operand (moved along k) plus one 32-bit byte offset per lane,
  // request and half (the host checks that they fit: leading dimensions below 4 M elements).  A wave
  // fills the four consecutive 1 KB regions 4 wave .. 4 wave + 3 of a sub-panel: eight rows each of a
  // K-contiguous sub-panel (lane = row % 8 * 8 + chunk position), four k-rows of a row-major one.
  int pid = blockIdx.x, ptm = 0, ptn = 0;
  if constexpr (PERSIST) {
    tile_coords(g.tiles_m, g.tiles_n, pid, ptm, ptn);
    bm = 0;  // the lane offsets below are relative to the tile (nothing is clamped: whole tiles only)
    bn = 0;
  }
  // where a tile's operands start, kXBias bytes low (a row-major b: its first k-row at the tile's first column
  // when PERSIST, else at column 0 with the columns in the lane offsets)
  auto a_start = [&](int tm) { return reinterpret_cast<const unsigned char*>(static_cast<const T*>(g.a) + (int64_t)tm * g.lda) - kXBias; };
  auto b_start = [&](int tn) {
    const T* B = static_cast<const T*>(g.b);
    return reinterpret_cast<const unsigned char*>(B_NN ? (PERSIST ? B + tn : B) : B + (int64_t)tn * g.ldb) - kXBias;
  };
  // PERSIST: a last row or column of tiles that would stick out of the matrix is moved back so that it ends
  // at the edge (M, N >= 256): every tile stays whole, and the rows / columns it shares with its neighbour are
  // computed - from the same k sequence - and stored twice with the same values.
  auto row0 = [&](int tm) { const int m = tm * BM; return m + BM <= g.M ? m : g.M - BM; };
  auto col0 = [&](int tn) { const int n = tn * BN; return n + BN <= g.N ? n : g.N - BN; };
  const unsigned char* a_base = a_start(PERSIST ? row0(ptm) : bm);  // of the tile being computed
  const unsigned char* b_base = b_start(PERSIST ? col0(ptn) : bn);
  const int64_t a_step = 128;                                   // bytes per 64-k stage
  const int64_t b_step = B_NN ? (int64_t)128 * g.ldb : 128;
  uint32_t a_off[2][4], b_off[2][4];
#pragma unroll
  for (int x = 0; x < 2; ++x)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = 8 * (4 * wave + i) + (lane >> 3);
      const int c = (lane & 7) ^ ((r >> 1) & 7);
      int lr = (r >> 6) * 128 + x * 64 + (r & 63);  // rows of wave row r / 64, half x
      lr = bm + lr < g.M ? lr : g.M - 1 - bm;         // rows past M re-read the last row
      a_off[x][i] = ((uint32_t)lr * (uint32_t)g.lda + (uint32_t)c * 8u) * 2u + (uint32_t)(kXBias - 1024 * i);
      if constexpr (B_NN) {
        const int k = 4 * (4 * wave + i) + (lane >> 4), pos = lane & 15;
        const int cc = ((((pos >> 1) ^ xswz_seg(k)) << 1) | (pos & 1)) * 8;  // first of the 8 columns this lane fetches
        int gn = bn + (cc >> 6) * WCOLS + x * HCOLS + (cc & 63);
        gn = gn < g.N ? gn : 0;
        b_off[x][i] = ((uint32_t)k * (uint32_t)g.ldb + (uint32_t)gn) * 2u + (uint32_t)(kXBias - 1024 * i);
      } else {
        int ln = (r >> 6) * WCOLS + x * HCOLS + (r & 63);
        ln = bn + ln < g.N ? ln : g.N - 1 - bn;
        b_off[x][i] = ((uint32_t)ln * (uint32_t)g.ldb + (uint32_t)c * 8u) * 2u + (uint32_t)(kXBias - 1024 * i);
      }
    }
  auto fill_i = [&](auto I_, const uint32_t (&vo)[4], const unsigned char* base) __attribute__((always_inline)) {
    constexpr int I = decltype(I_)::value;
    x16_fill<I>(vo[I], base);
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;

  const int l16 = lane & 15, lg = lane >> 4;
  // Fragment (blk, s) of a set: 16 rows x 32 k, lane = (k group lg, row l16).
  auto read_k = [&](const unsigned char* sub, int w, int blk, int s) __attribute__((always_inline)) {
    return *reinterpret_cast<const frag_t*>(sub + xswz_k(w * 64 + blk * 16 + l16, s * 4 + lg));
  };
  auto read_n = [&](const unsigned char* sub, int blk, int s) __attribute__((always_inline)) {
    const int k = s * 32 + lg * 8 + (l16 >> 2);
    const int n = wn * 64 + blk * 16 + ((lane & 3) << 2);
    const unsigned char* p = sub + k * 256 + (((n >> 4) ^ xswz_seg(k)) << 5) + ((n & 15) << 1);
    const s16x4 lo = lds_read_tr(p);
    const s16x4 hi = lds_read_tr(p + 4 * 256);
    return __builtin_bit_cast(frag_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };

  frag_t ra[2][2][4], rb[2][2][NPQ];  // [half][32-k half of the stage][block]
  f32x4 acc[8][2 * NPQ];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 2 * NPQ; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[i][j][e] = 0.f;
  // the zeros are written here, far ahead of the first MFMA that reads them (the compiler would
  // otherwise sink the moves to just in front of the loop, and it does not see an MFMA in the asm)
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 2 * NPQ; ++j) asm volatile("" : "+a"(acc[i][j]));

  // The two MFMAs of a couple as one asm statement: the accumulator block is tied to its AGPRs (with the
  // builtin the register allocator rotates the 256 accumulators through copies and spills), nothing
  // comes between the two (the second takes its addend straight from the first), and the "memory"
  // clobber keeps the LDS reads and fill requests of a quadrant where they are written, between the
  // couples.  Back-to-back MFMAs on one accumulator block need no wait states; nothing else reads the
  // accumulators before the epilogue.
  auto mfma2 = [&](f32x4& c, const frag_t& b0, const frag_t& a0, const frag_t& b1, const frag_t& a1) __attribute__((always_inline)) {
    if constexpr ((MI355_X16_ABLATE & 2048) != 0) {  // no MFMAs: the operands are still waited for
      asm volatile("" : "+a"(c) : "v"(__builtin_bit_cast(u32x4, b0)), "v"(__builtin_bit_cast(u32x4, a0)), "v"(__builtin_bit_cast(u32x4, b1)), "v"(__builtin_bit_cast(u32x4, a1)) : "memory");
    } else
    if constexpr (std::is_same<T, bf16_t>::value)
      asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0\n\tv_mfma_f32_16x16x32_bf16 %0, %3, %4, %0"
                   : "+a"(c)
                   : "v"(__builtin_bit_cast(u32x4, b0)), "v"(__builtin_bit_cast(u32x4, a0)), "v"(__builtin_bit_cast(u32x4, b1)),
                     "v"(__builtin_bit_cast(u32x4, a1))
                   : "memory");
    else
      asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0\n\tv_mfma_f32_16x16x32_f16 %0, %3, %4, %0"
                   : "+a"(c)
                   : "v"(__builtin_bit_cast(u32x4, b0)), "v"(__builtin_bit_cast(u32x4, a0)), "v"(__builtin_bit_cast(u32x4, b1)),
                     "v"(__builtin_bit_cast(u32x4, a1))
                   : "memory");
  };

  // One quadrant: 32 MFMAs on blocks (4 X + q, 4 Y + p), the two halves of the stage chained; the
  // operand whose set is the newer one runs in the outer loop, so its fragments are needed one by one.
  // LOAD: 0 nothing, 1 the A set into ra[LSET], 2 the B set into rb[LSET], read from the pair at `pair`
  // in the order in which a later quadrant consumes them.  Memory instructions only go behind the
  // second MFMA of a chained couple: the fragment reads behind the first couples, one each, and (FILL)
  // the four requests of one sub-panel, base m0v, behind every second one of the last seven couples.
  auto quadrant = [&](auto X_, auto Y_, auto AOUTER_, auto LOAD_, auto LSET_, auto FILL_, const unsigned char* pair, uint32_t m0v,
                      const uint32_t (&vo)[4], const unsigned char* fbase) __attribute__((always_inline)) {
    constexpr int X = decltype(X_)::value, Y = decltype(Y_)::value, LOAD = decltype(LOAD_)::value, LSET = decltype(LSET_)::value;
    constexpr bool AOUTER = decltype(AOUTER_)::value, FILL = decltype(FILL_)::value && !(MI355_X16_ABLATE & 1);
    constexpr int NC = 4 * NPQ;  // couples
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int q = AOUTER ? c / NPQ : c % 4, p = AOUTER ? c % NPQ : c / 4;
      mfma2(acc[4 * X + q][NPQ * Y + p], rb[Y][0][p], ra[X][0][q], rb[Y][1][p], ra[X][1][q]);
      if (c < (LOAD == 2 ? 2 * NPQ : 8)) {
        const int r = c;  // fragment r of the set: block r / 2, half r % 2
        if constexpr ((MI355_X16_ABLATE & 4) != 0) {
        } else if constexpr (LOAD == 1) {
          ra[LSET][r & 1][r >> 1] = read_k(pair, wm, r >> 1, r & 1);
        } else if constexpr (LOAD == 2) {
          if constexpr (B_NN) rb[LSET][r & 1][r >> 1] = read_n(pair + kXSub, r >> 1, r & 1);
          else rb[LSET][r & 1][r >> 1] = read_k(pair + kXSub, wn, r >> 1, r & 1);
        }
      }
      if constexpr (FILL) {
        if (c == NC - 7) { x16_set_m0(m0v); fill_i(I0{}, vo, fbase); }
        if (c == NC - 5) fill_i(I1{}, vo, fbase);
        if (c == NC - 3) fill_i(I2{}, vo, fbase);
        if (c == NC - 1) fill_i(I3{}, vo, fbase);
      }
    }
  };

  auto bump = [](uint32_t v) { return v + (uint32_t)kXPair == (uint32_t)(kXSlots * kXPair) ? 0u : v + (uint32_t)kXPair; };

  // Half-stage t = 4 u + HH (HH static: the register sets alternate with a period of two stages).
  // Computes two quadrants of stage t / 2, reads pair t + 1 (READ) and requests pair t + 5 (FILL; fa, fb:
  // where its stage starts in a and b) into the slot at `fl`, then waits until at most WAIT requests
  // are in flight (pair t + 2 is in) and meets the other waves (SYNC).  No branches between the MFMA
  // statements: the compiler would be free to copy the accumulators there, and it does not know the
  // wait states such a copy needs.
  uint32_t rd = kXPair, fl = 0;
  auto half_stage = [&](auto HH_, auto FILL_, auto READ_, auto WAIT_, auto SYNC_, const unsigned char* fa, const unsigned char* fb)
                        __attribute__((always_inline)) {
    constexpr int HH = decltype(HH_)::value, WAIT = decltype(WAIT_)::value;
    constexpr bool READ = decltype(READ_)::value;
    constexpr int H = (HH >> 1) & 1;                      // parity of the stage being computed
    constexpr int XR = ((HH + 1) & 1) ? 1 - (((HH + 1) >> 1) & 1) : (((HH + 1) >> 1) & 1);  // A half held by pair t + 1
    constexpr int XF = ((HH + 5) & 1) ? 1 - (((HH + 5) >> 1) & 1) : (((HH + 5) >> 1) & 1);  // and by pair t + 5
    constexpr int YF = (HH + 5) & 1;
    using XRc = std::integral_constant<int, XR>;
    using LA = std::integral_constant<int, READ ? 1 : 0>;
    using LB = std::integral_constant<int, READ ? 2 : 0>;
    const unsigned char* pair = lds + rd;
    const uint32_t m0a = lds_base + fl + (uint32_t)wave * 4096u, m0b = m0a + (uint32_t)kXSub;
    if constexpr ((HH & 1) == 0) {
      // first half of the stage: (B0, A_H) then (B0, A_(1-H)); pair t + 1 = {A_(1-H)(S), B1(S)}
      quadrant(std::integral_constant<int, H>{}, I0{}, std::true_type{}, LA{}, XRc{}, FILL_, pair, m0a, a_off[XF], fa);
      quadrant(std::integral_constant<int, 1 - H>{}, I0{}, std::true_type{}, LB{}, I1{}, FILL_, pair, m0b, b_off[YF], fb);
    } else {
      // second half: (B1, A_(1-H)) then (B1, A_H); pair t + 1 = {A_h'(S+1), B0(S+1)}, h' = 1 - H
      quadrant(std::integral_constant<int, 1 - H>{}, I1{}, std::false_type{}, LB{}, I0{}, FILL_, pair, m0b, b_off[YF], fb);
      quadrant(std::integral_constant<int, H>{}, I1{}, std::false_type{}, LA{}, XRc{}, FILL_, pair, m0a, a_off[XF], fa);
    }
#ifdef MI355_GEMM_TRACE
    if constexpr (decltype(SYNC_)::value && WAIT >= 0) {
      // wait, barrier and three stamps in one statement: the two stamps in front of the barrier have arrived
      // behind its lgkmcnt(0); the one behind it is read a half-stage later (tr_start alternates between
      // two scalars, so it is never copied before it has arrived)
      constexpr int par = HH & 1;
      uint64_t p1, p2;
#define MI355_TR_END(N)                                                                                                 \
  asm volatile("s_memtime %0\n\ts_waitcnt vmcnt(" #N ")\n\ts_memtime %1\n\ts_waitcnt lgkmcnt(0)\n\ts_barrier\n\ts_memtime %2" \
               : "=s"(p1), "=s"(p2), "=s"(tr_start[1 - par]) : "s"(tr_start[par]) : "memory");
      if constexpr (WAIT == 56) MI355_TR_END(56)
      if constexpr (WAIT == 24) MI355_TR_END(24)
      if constexpr (WAIT == 16) MI355_TR_END(16)
      if constexpr (WAIT == 8) MI355_TR_END(8)
      if constexpr (WAIT == 0) MI355_TR_END(0)
#undef MI355_TR_END
      tr_sum[par * 3 + 0] += p1 - tr_start[par];
      tr_sum[par * 3 + 1] += p2 - p1;
      if (tr_p2_prev != 0) tr_sum[(1 - par) * 3 + 2] += tr_start[par] - tr_p2_prev;
      tr_p2_prev = p2;
      tr_pairs += par;
    } else {
      if constexpr (decltype(SYNC_)::value) __syncthreads();
    }
#else
    if constexpr (WAIT == 56) asm volatile("s_waitcnt vmcnt(56)" ::: "memory");
    if constexpr (WAIT == 24 && !(MI355_X16_ABLATE & 8)) asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
    if constexpr (WAIT == 16) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
    if constexpr (WAIT == 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    if constexpr (WAIT == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if constexpr (decltype(SYNC_)::value && !(MI355_X16_ABLATE & 2)) __syncthreads();
#endif
    rd = bump(rd);
    fl = bump(fl);
  };
  using W56 = std::integral_constant<int, 56>;
  using W24 = std::integral_constant<int, 24>;
  using W16 = std::integral_constant<int, 16>;
  using W8 = std::integral_constant<int, 8>;
  using W0 = std::integral_constant<int, 0>;
  using WN = std::integral_constant<int, -1>;
  using Yes = std::true_type;
  using No = std::false_type;

  // Prologue: pairs 0..4 (K >= 256: they all exist); pairs 0 and 1 must be in before anything is read.
#pragma unroll
  for (int gi = 0; gi < kXSlots; ++gi) {
    const int s = gi >> 1, second = gi & 1, h = s & 1;
    const int x = second ? 1 - h : h;
    const uint32_t m0a = lds_base + (uint32_t)gi * kXPair + (uint32_t)wave * 4096u;
    x16_set_m0(m0a);
    fill_i(I0{}, a_off[x], a_base + s * a_step);
    fill_i(I1{}, a_off[x], a_base + s * a_step);
    fill_i(I2{}, a_off[x], a_base + s * a_step);
    fill_i(I3{}, a_off[x], a_base + s * a_step);
    x16_set_m0(m0a + (uint32_t)kXSub);
    fill_i(I0{}, b_off[second], b_base + s * b_step);
    fill_i(I1{}, b_off[second], b_base + s * b_step);
    fill_i(I2{}, b_off[second], b_base + s * b_step);
    fill_i(I3{}, b_off[second], b_base + s * b_step);
  }
  if constexpr (PERSIST) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // all five: the first tile's waits assume what later tiles find
  else asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
  __syncthreads();
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    ra[0][0][q] = read_k(lds, wm, q, 0);
    ra[0][1][q] = read_k(lds, wm, q, 1);
    if (q >= NPQ) continue;
    if constexpr (B_NN) {
      rb[0][0][q] = read_n(lds + kXSub, q, 0);
      rb[0][1][q] = read_n(lds + kXSub, q, 1);
    } else {
      rb[0][0][q] = read_k(lds + kXSub, wn, q, 0);
      rb[0][1][q] = read_k(lds + kXSub, wn, q, 1);
    }
  }
  __syncthreads();  // every wave holds pair 0: its slot may be refilled

  // Half-stages t .. t + 3 request pairs t + 5 .. t + 8 = stages t / 2 + 2, + 3, + 3, + 4.
  const int np = g.K / 32;  // pairs = half-stages; a multiple of 4 (K % 128 == 0), at least 8
  if constexpr (PERSIST) {
    const int total = g.tiles_m * g.tiles_n;
    for (;;) {
      // the tile behind this one (the last tile requests its own first pairs once more: nobody reads them)
      const int npid = pid + (int)gridDim.x;
      const bool has_next = npid < total;
      int ntm = ptm, ntn = ptn;
      if (has_next) tile_coords(g.tiles_m, g.tiles_n, npid, ntm, ntn);
      const unsigned char* na = a_start(row0(ntm));
      const unsigned char* nb = b_start(col0(ntn));
      const unsigned char* fa = a_base + 2 * a_step;
      const unsigned char* fb = b_base + 2 * b_step;
      // First four half-stages (np >= 12): pairs 2 .. 4 were requested before the previous tile's 32
      // stores per lane, pair 5 behind them - only the wait for pair 5 has to see the stores out.
      half_stage(I0{}, Yes{}, Yes{}, W56{}, Yes{}, fa, fb);
      half_stage(I1{}, Yes{}, Yes{}, W56{}, Yes{}, fa + a_step, fb + b_step);
      half_stage(I2{}, Yes{}, Yes{}, W56{}, Yes{}, fa + a_step, fb + b_step);
      half_stage(I3{}, Yes{}, Yes{}, W24{}, Yes{}, fa + 2 * a_step, fb + 2 * b_step);
      fa += 2 * a_step;
      fb += 2 * b_step;
      for (int t = 4; t + 8 < np; t += 4) {
        half_stage(I0{}, Yes{}, Yes{}, W24{}, Yes{}, fa, fb);
        half_stage(I1{}, Yes{}, Yes{}, W24{}, Yes{}, fa + a_step, fb + b_step);
        half_stage(I2{}, Yes{}, Yes{}, W24{}, Yes{}, fa + a_step, fb + b_step);
        half_stage(I3{}, Yes{}, Yes{}, W24{}, Yes{}, fa + 2 * a_step, fb + 2 * b_step);
        fa += 2 * a_step;
        fb += 2 * b_step;
      }
      // last eight: this tile's pairs np - 3 .. np - 1, then pairs 0 .. 4 of the next tile (stages 0, 0, 1, 1, 2)
      half_stage(I0{}, Yes{}, Yes{}, W24{}, Yes{}, fa, fb);
      half_stage(I1{}, Yes{}, Yes{}, W24{}, Yes{}, fa + a_step, fb + b_step);
      half_stage(I2{}, Yes{}, Yes{}, W24{}, Yes{}, fa + a_step, fb + b_step);
      half_stage(I3{}, Yes{}, Yes{}, W24{}, Yes{}, na, nb);
      half_stage(I0{}, Yes{}, Yes{}, W24{}, Yes{}, na, nb);
      half_stage(I1{}, Yes{}, Yes{}, W24{}, Yes{}, na + a_step, nb + b_step);
      half_stage(I2{}, Yes{}, Yes{}, W24{}, Yes{}, na + a_step, nb + b_step);
      half_stage(I3{}, Yes{}, Yes{}, W24{}, Yes{}, na + 2 * a_step, nb + 2 * b_step);  // reads the next tile's pair 0
      // the last MFMA's result is read by VALU moves next; the slot of the pair just read (`fl`) is free
      // until the next half-stage requests into it
      asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
      store_tile_result16<T, NPQ, 2>(g, acc, lds + fl, wave, lane, row0(ptm) + wm * 128, col0(ptn) + wn * 128);
      __syncthreads();  // every wave is done with its slab before anyone requests into the slot
      if (!has_next) break;
      pid = npid; ptm = ntm; ptn = ntn;
      a_base = na; b_base = nb;
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 2 * NPQ; ++j) {
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[i][j][e] = 0.f;
          asm volatile("" : "+a"(acc[i][j]));
        }
      asm volatile("s_nop 7" ::: "memory");  // the zeros are in before the first MFMA reads them
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the surplus requests of the last tile
    return;
  }
  const unsigned char* fa = a_base + 2 * a_step;
  const unsigned char* fb = b_base + 2 * b_step;
#ifdef MI355_GEMM_TRACE
  const uint64_t tr_begin = __builtin_readcyclecounter();
  tr_start[0] = tr_begin;
#endif
  int t = 0;
  for (; t + 8 < np; t += 4) {
    half_stage(I0{}, Yes{}, Yes{}, W24{}, Yes{}, fa, fb);
    half_stage(I1{}, Yes{}, Yes{}, W24{}, Yes{}, fa + a_step, fb + b_step);
    half_stage(I2{}, Yes{}, Yes{}, W24{}, Yes{}, fa + a_step, fb + b_step);
    half_stage(I3{}, Yes{}, Yes{}, W24{}, Yes{}, fa + 2 * a_step, fb + 2 * b_step);
    fa += 2 * a_step;
    fb += 2 * b_step;
  }
  // The last two pairs of stages: the requests run out (pairs np - 3 .. np - 1 are the last), then the reads.
  half_stage(I0{}, Yes{}, Yes{}, W24{}, Yes{}, fa, fb);
  half_stage(I1{}, Yes{}, Yes{}, W24{}, Yes{}, fa + a_step, fb + b_step);
  half_stage(I2{}, Yes{}, Yes{}, W24{}, Yes{}, fa + a_step, fb + b_step);
  half_stage(I3{}, No{}, Yes{}, W16{}, Yes{}, fa, fb);
  half_stage(I0{}, No{}, Yes{}, W8{}, Yes{}, fa, fb);
  half_stage(I1{}, No{}, Yes{}, W0{}, Yes{}, fa, fb);
  half_stage(I2{}, No{}, Yes{}, WN{}, Yes{}, fa, fb);
  half_stage(I3{}, No{}, No{}, WN{}, No{}, fa, fb);
  // the last MFMA's result is read by VALU moves next; every wave is past its last LDS read (the barrier
  // that ended the half-stage before the last) and no request is in flight, so the ring is free
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#ifdef MI355_GEMM_TRACE
  const uint64_t tr_end = __builtin_readcyclecounter();
#endif
  if constexpr (SPLITK && (MI355_X16_ABLATE & 1024) != 0) st_loop = __builtin_amdgcn_s_memrealtime();
  [[maybe_unused]] auto stamp_out = [&]() {
    if constexpr ((MI355_X16_ABLATE & 1024) != 0) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      if (tid == 0) {
        unsigned long long* o = g.sk_flags + (int64_t)(g.sk_splits - 1) * g.tiles_m * g.tiles_n + 64 + (int64_t)blockIdx.x * 8;
        o[0] = st_entry; o[1] = st_loop; o[2] = st_met; o[3] = __builtin_amdgcn_s_memrealtime(); o[4] = sk.role;
        o[5] = __builtin_amdgcn_s_getreg((20 << 0) | (0 << 6) | (3 << 11));  // HW_REG_XCC_ID
      }
    }
  };
  if constexpr (SPLITK) {
    // Two paths read the accumulators from here on.  Pin them to their AGPRs at this point: without it the
    // compiler copies them out early - between the last MFMA statements, whose wait states it does not know -
    // to have them at hand for both paths.
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 2 * NPQ; ++j) asm volatile("" : "+a"(acc[i][j]));
    if (sk.role > 0) {
      const __amdgpu_buffer_rsrc_t plane = x16_plane_rsrc(sk.planes, 1);
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) x16_plane_store(plane, wave * 64 + i * 8 + j, lane, acc[i][j]);
      // this wave's stores have completed before the barrier (a workgroup-scope fence leaves the counter
      // alone here, an agent-scope one writes back the whole L2)
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      if (tid == 0) __hip_atomic_store(sk.flags, sk.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if constexpr ((MI355_X16_ABLATE & 1024) != 0) st_met = __builtin_amdgcn_s_memrealtime();
      stamp_out();
      return;
    }
    if constexpr ((MI355_X16_ABLATE & 128) != 0) {
      store_tile_result16<T, NPQ>(g, acc, lds, wave, lane, bm + wm * 128, bn + wn * WCOLS);
      return;
    }
    volatile uint32_t* gave_up = reinterpret_cast<volatile uint32_t*>(lds);  // the ring is idle
    if (tid == 0) {
      uint32_t bad = 0;
      for (int q = 0; q < sk.nprod; ++q) {
        int polls = 0;
        while (__hip_atomic_load(sk.flags + q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != sk.epoch) {
          if (++polls > sk.spin_limit) { bad = 1; break; }
          __builtin_amdgcn_s_sleep(8);
        }
      }
      *gave_up = bad;
      if (bad) __hip_atomic_store(&x16_gave_up_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");  // the plane loads stay behind the polls
    __syncthreads();
    if constexpr ((MI355_X16_ABLATE & 1024) != 0) st_met = __builtin_amdgcn_s_memrealtime();
    X16Planes pl;
    pl.rsrc = x16_plane_rsrc(sk.planes, sk.nprod);
    pl.poison = *gave_up != 0 ? __builtin_nanf("") : -0.f;
    __syncthreads();  // everyone has read *gave_up: the epilogue reuses the ring
    auto finish = [&](auto NPROD_) __attribute__((always_inline)) {
      constexpr int NPROD = decltype(NPROD_)::value;
      if constexpr (NPQ == 4) {
        if (g.out_rows) return store_tile_rows16<T, NPROD>(g, acc, lds, wave, lane, bm, bn, &pl);
      }
      store_tile_result16<T, NPQ, 1, NPROD>(g, acc, lds, wave, lane, bm + wm * 128, bn + wn * WCOLS, &pl);
    };
    if (sk.nprod == 1) finish(std::integral_constant<int, 1>{});
    else if (sk.nprod == 2) finish(std::integral_constant<int, 2>{});
    else finish(std::integral_constant<int, 3>{});  // (the host plans at most four workgroups per tile)
    __syncthreads();  // every wave has read the planes
    if (tid == 0)
      for (int q = 0; q < sk.nprod; ++q) __hip_atomic_store(sk.flags + q, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    stamp_out();
    return;
  }
  if (!(MI355_X16_ABLATE & 32) || g.alpha == 12345.f) {
    if constexpr (NPQ == 4) {
      if (g.out_rows) store_tile_rows16<T>(g, acc, lds, wave, lane, bm, bn);
      else store_tile_result16<T, NPQ>(g, acc, lds, wave, lane, bm + wm * 128, bn + wn * WCOLS);
    } else {
      store_tile_result16<T, NPQ>(g, acc, lds, wave, lane, bm + wm * 128, bn + wn * WCOLS);
    }
  }
#ifdef MI355_GEMM_TRACE
  {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const uint64_t tr_stored = __builtin_readcyclecounter();
    if (lane == 0 && g.ws != nullptr) {
      uint64_t* o = reinterpret_cast<uint64_t*>(g.ws) + ((int64_t)blockIdx.x * 4 + wave) * 16;
      for (int q = 0; q < 6; ++q) o[q] = tr_sum[q];
      o[6] = tr_end - tr_begin; o[7] = tr_pairs; o[8] = 0; o[9] = 0; o[10] = tr_begin;
      o[11] = __builtin_amdgcn_s_getreg((4 << 0) | (0 << 6) | (31 << 11));  // HW_REG_HW_ID (XCC / SE / CU of this wave)
      o[12] = tr_entry; o[13] = tr_end; o[14] = tr_end; o[15] = tr_stored;
    }
  }
#endif
}

template <typename T, bool B_NN>
__global__ __launch_bounds__(256) void gemm_mfma_x16_kernel(GemmArgs g) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  if ((int)blockIdx.x >= g.tiles_m * g.tiles_n) return warm_operands<T, false, B_NN>(g, 0, g.K);
  int tm, tn;
  tile_coords(g, tm, tn);
  x16_tile<T, B_NN, 4>(g, lds, __builtin_amdgcn_readfirstlane(tm * BM), __builtin_amdgcn_readfirstlane(tn * BN));
}

// Fewer tiles than half the CUs and a long K: sk_splits workgroups per tile, each with its share of K.
// Blocks [r * sk_tiles8, (r + 1) * sk_tiles8) have one role: r < sk_splits - 1 the producers r + 1, the
// last group the summing workgroups (blocks are dispatched in order: a summing workgroup only ever waits
// for workgroups in front of it).  Block t of a group works on tile t; sk_tiles8 is a multiple of 8, so the
// workgroups of one tile share an XCD and its L2 (blocks go to the XCDs round robin), and blocks past the
// tile count have nothing to do.  K is shared out in units of 128, the summing workgroup gets the largest
// share (x16_split_summing_units): what it does with the planes only starts when the last producer has stored
// its plane, 3 us after its K loop, so the summing workgroup's own K loop should end about then.
template <typename T, bool B_NN>
__global__ __launch_bounds__(256) void gemm_mfma_x16_splitk_kernel(GemmArgs g) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int S = g.sk_splits, tiles = g.tiles_m * g.tiles_n;
  const int grp = __builtin_amdgcn_readfirstlane((int)blockIdx.x / g.sk_tiles8);
  const int t = __builtin_amdgcn_readfirstlane((int)blockIdx.x % g.sk_tiles8);
  if (t >= tiles) return;
  const int role = grp == S - 1 ? 0 : grp + 1;
  int tm, tn;
  tile_coords(g.tiles_m, g.tiles_n, t, tm, tn);
  const int units = g.K / kX16SplitUnit;
  const int cu = x16_split_summing_units(units, S);
  const int pu = units - cu, pbase = pu / (S - 1), prem = pu % (S - 1);
  int k0 = 0, ku = cu;
  if (role > 0) {
    const int q = role - 1;
    k0 = cu + q * pbase + (q < prem ? q : prem);
    ku = pbase + (q < prem ? 1 : 0);
  }
  GemmArgs gs = g;
  const T* A = static_cast<const T*>(g.a);
  const T* B = static_cast<const T*>(g.b);
  gs.a = A + (int64_t)k0 * kX16SplitUnit;
  gs.b = B_NN ? B + (int64_t)k0 * kX16SplitUnit * g.ldb : B + (int64_t)k0 * kX16SplitUnit;
  gs.K = ku * kX16SplitUnit;
  X16Split sk;
  const int64_t first = (int64_t)t * (S - 1) + (role > 0 ? role - 1 : 0);  // plane / flag index
  sk.planes = reinterpret_cast<f32x4*>(g.ws) + first * 16384;
  sk.flags = g.sk_flags + first;
  sk.epoch = g.sk_epoch;
  sk.spin_limit = g.sk_spin_limit;
  sk.role = role;
  sk.nprod = S - 1;
  x16_tile<T, B_NN, 4, false, true>(gs, lds, __builtin_amdgcn_readfirstlane(tm * BM), __builtin_amdgcn_readfirstlane(tn * BN), sk);
}

// Two tile widths in one launch: blocks [0, tiles_m * tiles_n) are 256 x 256 tiles of the columns
// [0, 256 tiles_n); the blocks behind them are 256 x 192 tiles of the columns from there on (tiles_m *
// tail_n of them).  Workgroups are dispatched in block order, so the narrow tiles form the last round.
template <typename T, bool B_NN>
__global__ __launch_bounds__(256) void gemm_mfma_x16_mixed_kernel(GemmArgs g) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int wide = g.tiles_m * g.tiles_n;
  int tm, tn;
  if ((int)blockIdx.x < wide) {
    tile_coords(g.tiles_m, g.tiles_n, blockIdx.x, tm, tn);
    x16_tile<T, B_NN, 4>(g, lds, __builtin_amdgcn_readfirstlane(tm * BM), __builtin_amdgcn_readfirstlane(tn * BN));
  } else {
    tile_coords(g.tiles_m, g.tail_n, blockIdx.x - wide, tm, tn);
    x16_tile<T, B_NN, 3>(g, lds, __builtin_amdgcn_readfirstlane(tm * BM), __builtin_amdgcn_readfirstlane(g.tiles_n * BN + tn * 192));
  }
}

// One workgroup per CU walks the tiles (x16_tile<..., PERSIST>): gridDim.x workgroups, tiles_m * tiles_n tiles.
template <typename T, bool B_NN>
__global__ __launch_bounds__(256) void gemm_mfma_x16_persistent_kernel(GemmArgs g) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  x16_tile<T, B_NN, 4, true>(g, lds, 0, 0);
}

const void* gemm_x16_persistent_kernel(bool is_bf16, bool b_nn) {
  if (is_bf16) return b_nn ? (const void*)gemm_mfma_x16_persistent_kernel<bf16_t, true> : (const void*)gemm_mfma_x16_persistent_kernel<bf16_t, false>;
  return b_nn ? (const void*)gemm_mfma_x16_persistent_kernel<f16_t, true> : (const void*)gemm_mfma_x16_persistent_kernel<f16_t, false>;
}

const void* gemm_x16_kernel(bool is_bf16, bool b_nn) {
  if (is_bf16) return b_nn ? (const void*)gemm_mfma_x16_kernel<bf16_t, true> : (const void*)gemm_mfma_x16_kernel<bf16_t, false>;
  return b_nn ? (const void*)gemm_mfma_x16_kernel<f16_t, true> : (const void*)gemm_mfma_x16_kernel<f16_t, false>;
}

const void* gemm_x16_splitk_kernel(bool is_bf16, bool b_nn) {
  if (is_bf16) return b_nn ? (const void*)gemm_mfma_x16_splitk_kernel<bf16_t, true> : (const void*)gemm_mfma_x16_splitk_kernel<bf16_t, false>;
  return b_nn ? (const void*)gemm_mfma_x16_splitk_kernel<f16_t, true> : (const void*)gemm_mfma_x16_splitk_kernel<f16_t, false>;
}

const void* gemm_x16_mixed_kernel(bool is_bf16, bool b_nn) {
  if (is_bf16) return b_nn ? (const void*)gemm_mfma_x16_mixed_kernel<bf16_t, true> : (const void*)gemm_mfma_x16_mixed_kernel<bf16_t, false>;
  return b_nn ? (const void*)gemm_mfma_x16_mixed_kernel<f16_t, true> : (const void*)gemm_mfma_x16_mixed_kernel<f16_t, false>;
}

}  // namespace mi355

extern "C" int mi355_gemm_status(void) {
  unsigned int word = 0, word2 = 0;
  hipError_t e = hipMemcpyFromSymbol(&word, HIP_SYMBOL(mi355::x16_gave_up_word), sizeof(word));
  if (e != hipSuccess) return mi355::set_error(MI355_ERR_LAUNCH, "mi355_gemm_status: reading the status word failed: %s", hipGetErrorString(e));
  if (word != 0) {
    const unsigned int zero = 0;
    e = hipMemcpyToSymbol(HIP_SYMBOL(mi355::x16_gave_up_word), &zero, sizeof(zero));
    if (e != hipSuccess) return mi355::set_error(MI355_ERR_LAUNCH, "mi355_gemm_status: clearing the status word failed: %s", hipGetErrorString(e));
  }
  const int e2 = mi355::read_insplit_status(&word2);  // the 128x128- and 64x64-tile kernels' word (gemm.hip)
  if (e2 != 0) return mi355::set_error(MI355_ERR_LAUNCH, "mi355_gemm_status: reading the status word failed: %s", hipGetErrorString((hipError_t)e2));
  if (word == 0 && word2 == 0) return MI355_OK;
  return mi355::set_error(MI355_ERR_LAUNCH,
                          "mi355_gemm: a split-K launch gave up waiting for a partial product (its output tile holds NaNs)");
}
