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

// Epilogue: the wave's 128 x 128 result, 64 columns at a time, through a 16 KB slab of the idle ring
// (rows of 128 B, 16-byte slot s of row r at s ^ ((r / 2) % 8)) and out in whole 128-byte rows.
// Register e of acc[i][j] in lane l is C[m0 + 16 i + l % 16][n0 + 16 j + 4 (l / 16) + e] (operands swapped).
template <typename T>
__device__ __forceinline__ void store_tile_result16(const GemmArgs& g, const f32x4 (&acc)[8][8], unsigned char* lds,
                                                    int wave, int lane, int m0, int n0) {
  const int lr = lane & 15, lg = lane >> 4;
  const T* C = static_cast<const T*>(g.c);
  const bool use_c = C != nullptr && g.beta != 0.f;
  const bool row_bias = use_c && g.c_vec && g.c_rs == 0;
  unsigned char* slab = lds + wave * (128 * 128);
  T* D = static_cast<T*>(g.out);
#pragma unroll
  for (int y = 0; y < 2; ++y) {
    const int nh = n0 + y * 64;
    float bias[4][4];
    if (row_bias) {
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const int n = nh + p * 16 + lg * 4;
        const VecN4<T> t = *reinterpret_cast<const VecN4<T>*>(C + (n + 4 <= g.N ? n : 0));
#pragma unroll
        for (int e = 0; e < 4; ++e) bias[p][e] = g.beta * static_cast<float>(t.v[e]);
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = i * 16 + lr;
      const int m = m0 + row;
      const int mc = m < g.M ? m : g.M - 1;
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const int nl = p * 16 + lg * 4;
        const int n = nh + nl;
        const f32x4 v = acc[i][y * 4 + p];
        VecN4<T> r;
        if (row_bias) {
#pragma unroll
          for (int e = 0; e < 4; ++e) r.v[e] = static_cast<T>(g.alpha * v[e] + bias[p][e]);
        } else {
          float cv[4] = {0.f, 0.f, 0.f, 0.f};  // columns past N are computed on valid addresses and never stored
          if (use_c) {
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
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float s = g.alpha * v[e];
            r.v[e] = static_cast<T>(use_c ? s + g.beta * cv[e] : s);
          }
        }
        const int slot = (nl >> 3) ^ ((row >> 1) & 7);
        *reinterpret_cast<VecN4<T>*>(slab + row * 128 + slot * 16 + (lg & 1) * 8) = r;
      }
    }
    // same wave wrote and reads: LDS operations of a wave complete in order
    if (g.out_vec) {
#pragma unroll
      for (int t = 0; t < 16; ++t) {
        const int chunk = t * kWave + lane;  // 1024 chunks of 16 bytes, 8 per row
        const int row = chunk >> 3, s = chunk & 7;
        const u32x4 v = *reinterpret_cast<const u32x4*>(slab + row * 128 + ((s ^ ((row >> 1) & 7)) << 4));
        const int m = m0 + row, n = nh + s * 8;
        if (m >= g.M || n >= g.N) continue;
        *reinterpret_cast<u32x4*>(D + (int64_t)m * g.N + n) = v;
      }
    } else {
      // output rows at any 2-byte offset (N % 8 != 0): one row per store instruction, lane l writes column l
      const int n = nh + lane;
      const int rows = g.M - m0 < 128 ? g.M - m0 : 128;
#pragma unroll 8
      for (int row = 0; row < rows; ++row) {
        const T v = *reinterpret_cast<const T*>(slab + row * 128 + (((lane >> 3) ^ ((row >> 1) & 7)) << 4) + ((lane & 7) << 1));
        if (n < g.N) D[(int64_t)(m0 + row) * g.N + n] = v;
      }
    }
  }
}

template <typename T, bool B_NN>
__global__ __launch_bounds__(256) void gemm_mfma_x16_kernel(GemmArgs g) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  using frag_t = typename Mfma16<T>::frag;
  int tm, tn;
  tile_coords(g, tm, tn);
  const int bm = tm * BM, bn = tn * BN;
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave >> 1, wn = wave & 1;
  const T* A = static_cast<const T*>(g.a);
  const T* B = static_cast<const T*>(g.b);
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;

  // Fill addresses: a uniform base per operand (moved along k by the requests) plus one 32-bit byte
  // offset per lane, request and half (the host checks that they fit: leading dimensions below 4 M
  // elements).  Request i of a sub-panel is its 1 KB region wave + 4 i: eight rows of a K-contiguous
  // sub-panel (lane = row % 8 * 8 + chunk position) or four k-rows of a row-major one.
  const T* a_base = A + (int64_t)bm * g.lda;
  const T* b_base = B_NN ? B : B + (int64_t)bn * g.ldb;
  uint32_t a_off[2][4], b_off[2][4];
#pragma unroll
  for (int x = 0; x < 2; ++x)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = 8 * (wave + 4 * i) + (lane >> 3);
      const int c = (lane & 7) ^ ((r >> 1) & 7);
      int lr = (r >> 6) * 128 + x * 64 + (r & 63);  // rows of wave row r / 64, half x
      lr = bm + lr < g.M ? lr : g.M - 1 - bm;         // rows past M re-read the last row
      a_off[x][i] = ((uint32_t)lr * (uint32_t)g.lda + (uint32_t)c * 8u) * 2u;
      if constexpr (B_NN) {
        const int k = 4 * (wave + 4 * i) + (lane >> 4), pos = lane & 15;
        const int cc = ((((pos >> 1) ^ xswz_seg(k)) << 1) | (pos & 1)) * 8;  // first of the 8 columns this lane fetches
        int gn = bn + (cc >> 6) * 128 + x * 64 + (cc & 63);
        gn = gn < g.N ? gn : 0;
        b_off[x][i] = ((uint32_t)k * (uint32_t)g.ldb + (uint32_t)gn) * 2u;
      } else {
        int ln = (r >> 6) * 128 + x * 64 + (r & 63);
        ln = bn + ln < g.N ? ln : g.N - 1 - bn;
        b_off[x][i] = ((uint32_t)ln * (uint32_t)g.ldb + (uint32_t)c * 8u) * 2u;
      }
    }
  // Request q (0..3: A, 4..7: B) of the pair that holds halves (x, y) of stage s, into the slot at slot_off.
  auto request = [&](int q, int x, int y, int s, uint32_t slot_off) __attribute__((always_inline)) {
    if (q < 4) {
      lds_dma16s(lds_base + slot_off + (uint32_t)(wave + 4 * q) * 1024u, x ? a_off[1][q] : a_off[0][q], a_base + (int64_t)s * 64);
    } else {
      const int i = q - 4;
      lds_dma16s(lds_base + slot_off + (uint32_t)kXSub + (uint32_t)(wave + 4 * i) * 1024u, y ? b_off[1][i] : b_off[0][i],
                 b_base + (B_NN ? (int64_t)s * 64 * g.ldb : (int64_t)s * 64));
    }
  };

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

  frag_t ra[2][2][4], rb[2][2][4];  // [half][32-k half of the stage][block]
  f32x4 acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[i][j][e] = 0.f;
  // the zeros are written here, far ahead of the first MFMA that reads them (the compiler would
  // otherwise sink the moves to just in front of the loop, and it does not see an MFMA in the asm)
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) asm volatile("" : "+a"(acc[i][j]));

  // The MFMA as an asm statement: the accumulator block is tied to its AGPRs (with the builtin the
  // register allocator rotates the 256 accumulators through copies and spills), and the "memory"
  // clobber keeps the LDS reads and fill requests of a quadrant where they are written, between the
  // MFMAs.  Back-to-back MFMAs on one accumulator block need no wait states; nothing else reads the
  // accumulators before the epilogue.
  auto mfma = [&](f32x4& c, const frag_t& b, const frag_t& a) __attribute__((always_inline)) {
    if constexpr (std::is_same<T, bf16_t>::value)
      asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(__builtin_bit_cast(u32x4, b)), "v"(__builtin_bit_cast(u32x4, a)) : "memory");
    else
      asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(__builtin_bit_cast(u32x4, b)), "v"(__builtin_bit_cast(u32x4, a)) : "memory");
  };

  // One quadrant: 32 MFMAs on blocks (4 X + q, 4 Y + p), the two halves of the stage chained; the
  // operand whose set is the newer one runs in the outer loop, so its fragments are needed one by one.
  // LOAD: 0 nothing, 1 the A set into ra[LSET], 2 the B set into rb[LSET], read from the pair at `pair`
  // in the order in which a later quadrant consumes them: one fragment behind every third MFMA of the
  // first 24, and a fill request (first request FQ) behind every second fragment.
  auto quadrant = [&](auto X_, auto Y_, auto AOUTER_, auto LOAD_, auto LSET_, const unsigned char* pair, bool fill, auto FQ_,
                      int fx, int fy, int fs, uint32_t fslot) __attribute__((always_inline)) {
    constexpr int X = decltype(X_)::value, Y = decltype(Y_)::value, LOAD = decltype(LOAD_)::value, LSET = decltype(LSET_)::value;
    constexpr int fq = decltype(FQ_)::value;
    constexpr bool AOUTER = decltype(AOUTER_)::value;
#pragma unroll
    for (int m = 0; m < 32; ++m) {
      const int o = m >> 3, n = (m >> 1) & 3, s = m & 1;
      const int q = AOUTER ? o : n, p = AOUTER ? n : o;
      mfma(acc[4 * X + q][4 * Y + p], rb[Y][s][p], ra[X][s][q]);
      if (m < 24 && m % 3 == 2) {
        const int r = m / 3;  // fragment r of the set: block r / 2, half r % 2
        if constexpr (LOAD == 1) {
          ra[LSET][r & 1][r >> 1] = read_k(pair, wm, r >> 1, r & 1);
        } else if constexpr (LOAD == 2) {
          if constexpr (B_NN) rb[LSET][r & 1][r >> 1] = read_n(pair + kXSub, r >> 1, r & 1);
          else rb[LSET][r & 1][r >> 1] = read_k(pair + kXSub, wn, r >> 1, r & 1);
        }
        if ((r & 1) && fill) request(fq + (r >> 1), fx, fy, fs, fslot);
      }
    }
  };

  auto bump = [](uint32_t v) { return v + (uint32_t)kXPair == (uint32_t)(kXSlots * kXPair) ? 0u : v + (uint32_t)kXPair; };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I4 = std::integral_constant<int, 4>;

  // Half-stage t = 4 u + HH (HH static: the register sets alternate with a period of two stages).
  // Computes two quadrants of stage t / 2, reads pair t + 1 and requests pair t + 5 into the slot at
  // `fl`.  The steps have no conditional parts: past the end of K the reads fetch a stale slot into
  // registers nobody uses again and the requests fetch the last stage once more into slots nobody reads
  // (four pairs per tile), so the accumulators never cross a branch between two MFMA statements - the
  // compiler would be free to copy them there, and it does not know the wait states such a copy needs.
  const int ns = g.K / 64;
  uint32_t rd = kXPair, fl = 0;
  auto half_stage = [&](auto HH_, int t) __attribute__((always_inline)) {
    constexpr int HH = decltype(HH_)::value;
    constexpr int H = (HH >> 1) & 1;                      // parity of the stage being computed
    constexpr int XR = ((HH + 1) & 1) ? 1 - (((HH + 1) >> 1) & 1) : (((HH + 1) >> 1) & 1);  // A half held by pair t + 1
    constexpr int XF = ((HH + 5) & 1) ? 1 - (((HH + 5) >> 1) & 1) : (((HH + 5) >> 1) & 1);  // and by pair t + 5
    constexpr int YF = (HH + 5) & 1;
    using XRc = std::integral_constant<int, XR>;
    const int fs = (t + 5) >> 1 < ns ? (t + 5) >> 1 : ns - 1;
    const unsigned char* pair = lds + rd;
    if constexpr ((HH & 1) == 0) {
      // first half of the stage: (B0, A_H) then (B0, A_(1-H)); pair t + 1 = {A_(1-H)(S), B1(S)}
      quadrant(std::integral_constant<int, H>{}, I0{}, std::true_type{}, I1{}, XRc{}, pair, true, I0{}, XF, YF, fs, fl);
      quadrant(std::integral_constant<int, 1 - H>{}, I0{}, std::true_type{}, I2{}, I1{}, pair, true, I4{}, XF, YF, fs, fl);
    } else {
      // second half: (B1, A_(1-H)) then (B1, A_H); pair t + 1 = {A_h'(S+1), B0(S+1)}, h' = 1 - H
      quadrant(std::integral_constant<int, 1 - H>{}, I1{}, std::false_type{}, I2{}, I0{}, pair, true, I4{}, XF, YF, fs, fl);
      quadrant(std::integral_constant<int, H>{}, I1{}, std::false_type{}, I1{}, XRc{}, pair, true, I0{}, XF, YF, fs, fl);
    }
    asm volatile("s_waitcnt vmcnt(24)" ::: "memory");  // pair t + 2 is in: only the requests of pairs t + 3 .. t + 5 fly
    __syncthreads();
    rd = bump(rd);
    fl = bump(fl);
  };

  // Prologue: pairs 0..4 (K >= 256: they all exist); pairs 0 and 1 must be in before anything is read.
#pragma unroll
  for (int gi = 0; gi < kXSlots; ++gi) {
    const int s = gi >> 1, second = gi & 1, h = s & 1;
#pragma unroll
    for (int q = 0; q < 8; ++q) request(q, second ? 1 - h : h, second, s, (uint32_t)gi * kXPair);
  }
  asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
  __syncthreads();
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    ra[0][0][q] = read_k(lds, wm, q, 0);
    ra[0][1][q] = read_k(lds, wm, q, 1);
    if constexpr (B_NN) {
      rb[0][0][q] = read_n(lds + kXSub, q, 0);
      rb[0][1][q] = read_n(lds + kXSub, q, 1);
    } else {
      rb[0][0][q] = read_k(lds + kXSub, wn, q, 0);
      rb[0][1][q] = read_k(lds + kXSub, wn, q, 1);
    }
  }
  __syncthreads();  // every wave holds pair 0: its slot may be refilled

  const int np = 2 * ns;  // ns is even (K % 128 == 0): whole pairs of stages
  for (int t = 0; t < np; t += 4) {
    half_stage(I0{}, t);
    half_stage(I1{}, t + 1);
    half_stage(I2{}, t + 2);
    half_stage(std::integral_constant<int, 3>{}, t + 3);
  }
  // the surplus requests still land in the ring, which the epilogue reuses; the last MFMA's result is
  // read by VALU moves next
  asm volatile("s_waitcnt vmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  __syncthreads();
  store_tile_result16<T>(g, acc, lds, wave, lane, bm + wm * 128, bn + wn * 128);
}

const void* gemm_x16_kernel(bool is_bf16, bool b_nn) {
  if (is_bf16) return b_nn ? (const void*)gemm_mfma_x16_kernel<bf16_t, true> : (const void*)gemm_mfma_x16_kernel<bf16_t, false>;
  return b_nn ? (const void*)gemm_mfma_x16_kernel<f16_t, true> : (const void*)gemm_mfma_x16_kernel<f16_t, false>;
}

}  // namespace mi355
