// mm / addmm:  out[M,N] = beta * c + alpha * (a[M,K] @ b[K,N]),  fp32 accumulate.
//
//   mfma     bf16 / f16, a K-contiguous (or M-contiguous, a transposed view, when K % 64 == 0), b either
//            K-contiguous ("NT", e.g. weight.t()) or N-contiguous ("NN", row-major), 16-byte aligned rows.  256x256 block tile, 32-k steps,
//            v_mfma_f32_32x32x16, LDS panels swizzled so that the fills and the fragment reads
//            are bank-conflict free.  A row-major B stays N-contiguous in LDS and is transposed
//            by the LDS read itself (ds_read_b64_tr_b16).  Block -> tile map groups tiles per
//            XCD so that one L2 serves neighbouring tiles.  By K:
//              gemm_mfma_x16_kernel    (gemm_x16.hip) K % 128 == 0, K >= 512, a K-contiguous: four
//                                      waves of 128x128 on v_mfma_f32_16x16x32, the form the power
//                                      envelope favours;
//              gemm_mfma_w4_kernel     K % 64 == 0, K >= 2048: four waves of 128x128, fragments
//                                      read a step ahead, fills issued one at a time;
//              gemm_mfma_dma64_kernel  K % 64 == 0: eight waves of 128x64 (two per SIMD), A
//                                      fetched in whole 128-byte lines;
//              gemm_mfma_dma_kernel    K % 32 == 0: as above with a ring of 32-k stages; all three
//                                      fill LDS directly (global_load_lds_dwordx4);
//              gemm_mfma_kernel        K tail: global -> registers -> LDS with zero fill.
//            Problems with few tiles run on 128x128 tiles (two workgroups per CU), split along
//            K over the chip when the caller provides a workspace.
//   mfma f32 v_mfma_f32_32x32x2_f32, 128x128 tiles.
//   generic  any strides, the dtypes but f64: 64x64 LDS tile, FMA inner loop.
//            Correctness path for shapes the MFMA kernels do not take.
//   f64      gemm_f64.hip: v_mfma_f64_16x16x4_f64, any strides.
#include <stdlib.h>
#include <string.h>
#include <type_traits>

#include "common.h"
#include <atomic>
#include "gemm_shared.h"

namespace mi355 {


// v_mfma_f32_32x32x16: measured at ~96 % of the 2.5 PFLOP/s bf16 peak on MI355X when issued
// back to back on all-zero operands.  (The 16x16x32 form issues at the same rate and draws less power
// on real operand data; the kernels of this file predate that measurement, gemm_x16.hip uses it.)
// Operand layout: lane l holds 8 consecutive k (k = (l/32)*8 + e) of row/column l%32; the
// 32x32 result puts column l%32 and rows 8*(r/4) + (l/32)*4 + r%4 in register r of lane l.
template <typename T> struct Mfma;
template <> struct Mfma<bf16_t> {
  using frag = bf16x8;
  static __device__ __forceinline__ f32x16 run(frag a, frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mfma<f16_t> {
  using frag = f16x8;
  static __device__ __forceinline__ f32x16 run(frag a, frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

// N-contiguous panel ([k][n], the row-major "NN" B, 512 B per k): byte offset of 16-byte unit u
// (0..31) of row k.  64-byte segments are rotated by k%4 (XOR on the segment index) so that a
// transposing 64-bit read by 32 lanes — 4 consecutive k-rows x 64 B, see lds_read_tr — covers
// four distinct 64-byte segments of the 256-byte bank window.
__device__ __forceinline__ int swz_n(int k, int u) {
  return k * (BN * 2) + ((((u >> 2) ^ (k & 3))) << 6) + ((u & 3) << 4);
}


// fp32 partial tile of one split: register r of acc[i][j] in lane l is
// C[m0 + 32 i + l%32][n0 + 32 j + 8 (r/4) + 4 (l/32) + r%4]; N % 4 == 0 on the MFMA paths.
template <int MI, int NJ = 2>
__device__ __forceinline__ void store_partial_tile(const GemmArgs& g, const f32x16 (&acc)[MI][NJ], int lane, int m0,
                                                   int n0) {
  const int fr = lane & 31, fg = lane >> 5;
  float* W = g.ws + (int64_t)blockIdx.y * g.M * g.ws_ld;
#pragma unroll
  for (int i = 0; i < MI; ++i) {
    const int m = m0 + i * 32 + fr;
    if (m >= g.M) continue;
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + j * 32 + q * 8 + fg * 4;
        if (n >= g.N) continue;
        f32x4 r;
#pragma unroll
        for (int e = 0; e < 4; ++e) r[e] = acc[i][j][q * 4 + e];
        *reinterpret_cast<f32x4*>(W + (int64_t)m * g.ws_ld + n) = r;  // columns past N land in the row's padding
      }
  }
}

// ---- split K inside one launch (the 128x128- and 64x64-tile kernels, SPLIT == 2)
// blockIdx.y is the part of K, as in the two-launch form.  Parts 0 .. gridDim.y - 2 are producers: each
// leaves its raw fp32 accumulators in its plane of the workspace (register order: 16-byte piece q of block b
// of wave w at byte ((w NB + b) 4 + q) 1024 + 16 lane - one `buffer_store_dwordx4 ... sc1` per piece), waits for
// the stores and raises its 64-bit flag.  The last part sums: it polls the flags (bounded), adds the planes
// to its own accumulators, sets the flags back to 0 and runs the ordinary epilogue.  Blocks are dispatched
// in order, x fastest, so a summing workgroup only ever waits for workgroups in front of it, and producers
// never wait: nothing that shares the chip with the launch can make it wait for a workgroup that has not
// been dispatched.  Agent-scope accesses (the sc1 bit), not fences: see gemm_x16.hip.  The flag value is the
// launch's own (GemmArgs::sk_epoch), so stale workspace contents and graph replays are both safe.
// A plane is NB x 16 KB (64 KB for a 128x128 tile): reading one costs the summing workgroup 1 - 2 us, where
// a summing launch costs 3 us plus every plane written and read through HBM.
constexpr int kSc1 = 1 << 4;  // bit 4 of a buffer instruction's cache policy operand
static __device__ unsigned int insplit_gave_up_word;  // sticky, read and cleared by mi355_gemm_status

template <int NB>
__device__ __forceinline__ __amdgpu_buffer_rsrc_t insplit_rsrc(const GemmArgs& g, int64_t first_plane, int nplanes) {
  return __builtin_amdgcn_make_buffer_rsrc(g.ws + first_plane * (NB * 4096), 0, nplanes * (NB * 16384), 0x00020000);
}

template <int MI, int NJ>
__device__ __forceinline__ void insplit_leave(const GemmArgs& g, const f32x16 (&acc)[MI][NJ], int tid, int wave, int lane) {
  constexpr int NB = MI * NJ;
  const int nprod = (int)gridDim.y - 1;
  const int64_t plane = (int64_t)blockIdx.x * nprod + blockIdx.y;
  const __amdgpu_buffer_rsrc_t rsrc = insplit_rsrc<NB>(g, plane, 1);
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        f32x4 r;
#pragma unroll
        for (int e = 0; e < 4; ++e) r[e] = acc[i][j][q * 4 + e];
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, r), rsrc, lane * 16, ((wave * NB + i * NJ + j) * 4 + q) * 1024, kSc1);
      }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's plane is out before the barrier
  __syncthreads();
  if (tid == 0) __hip_atomic_store(g.sk_flags + plane, g.sk_epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int MI, int NJ>
__device__ __forceinline__ void insplit_sum(const GemmArgs& g, f32x16 (&acc)[MI][NJ], unsigned char* lds, int tid, int wave, int lane) {
  constexpr int NB = MI * NJ;
  const int nprod = (int)gridDim.y - 1;
  const int64_t first = (int64_t)blockIdx.x * nprod;
  __syncthreads();  // every wave is past its last LDS read: the ring is idle
  volatile uint32_t* gave_up = reinterpret_cast<volatile uint32_t*>(lds);
  if (tid == 0) {
    uint32_t bad = 0;
    for (int p = 0; p < nprod; ++p) {
      int polls = 0;
      while (__hip_atomic_load(g.sk_flags + first + p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != g.sk_epoch) {
        if (++polls > g.sk_spin_limit) { bad = 1; break; }
        __builtin_amdgcn_s_sleep(8);
      }
    }
    *gave_up = bad;
    if (bad) __hip_atomic_store(&insplit_gave_up_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");  // the plane loads stay behind the polls
  __syncthreads();
  const float poison = *gave_up != 0 ? __builtin_nanf("") : -0.f;  // -0: x + -0 == x
  const __amdgpu_buffer_rsrc_t rsrc = insplit_rsrc<NB>(g, first, nprod);
  // The planes of several producers are in flight at once (four for a one-block wave tile, two for four blocks:
  // 64 / 128 registers): a plane comes from another CU's stores through the L2, about a microsecond each when
  // they are read one after the other.  A batch's last planes may lie past the count: they re-read the last
  // plane and are not added.  The order of the additions is the order of the parts, as before.
  constexpr int PB = NB == 1 ? 4 : NB <= 4 ? 2 : 1;
  for (int p0 = 0; p0 < nprod; p0 += PB) {
    f32x4 part[PB][NB][4];
#pragma unroll
    for (int u = 0; u < PB; ++u) {
      const int p = p0 + u < nprod ? p0 + u : nprod - 1;
#pragma unroll
      for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int q = 0; q < 4; ++q)
          part[u][b][q] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, lane * 16, p * (NB * 16384) + ((wave * NB + b) * 4 + q) * 1024, kSc1));
    }
#pragma unroll
    for (int u = 0; u < PB; ++u) {
      if (p0 + u >= nprod) break;
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[i][j][q * 4 + e] += part[u][i * NJ + j][q][e];
    }
  }
  acc[0][0][0] += poison;  // NaN marks the tile of a producer that never arrived
  __syncthreads();  // every wave has used what it read of the planes, and has read *gave_up: the epilogue reuses the ring
  if (tid == 0)
    for (int p = 0; p < nprod; ++p) __hip_atomic_store(g.sk_flags + first + p, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The in-launch split's status word for mi355_gemm_status: reads it into *word and clears it when set.
int read_insplit_status(unsigned int* word) {
  hipError_t e = hipMemcpyFromSymbol(word, HIP_SYMBOL(insplit_gave_up_word), sizeof(*word));
  if (e == hipSuccess && *word != 0) {
    const unsigned int zero = 0;
    e = hipMemcpyToSymbol(HIP_SYMBOL(insplit_gave_up_word), &zero, sizeof(zero));
  }
  return e == hipSuccess ? 0 : (int)e;
}

// out = alpha * sum over splits of ws + beta * c, four consecutive n per thread.  A group of
// four columns that starts inside a row may end in its padding (N % 4 != 0): those output rows
// are misaligned and are stored element by element.
template <typename T>
__device__ __forceinline__ void finish_store(const GemmArgs& g, const f32x4& sum, int64_t m, int64_t n) {
  const T* C = static_cast<const T*>(g.c);
  const bool use_c = C != nullptr && g.beta != 0.f;
  T* D = static_cast<T*>(g.out) + m * g.N + n;
  VecN4<T> r;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    float v = g.alpha * sum[e];
    if (use_c && n + e < g.N) v += g.beta * static_cast<float>(C[m * g.c_rs + (n + e) * g.c_cs]);
    r.v[e] = static_cast<T>(v);
  }
  if (g.ws_ld == g.N) {
    *reinterpret_cast<VecN4<T>*>(D) = r;
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (n + e < g.N) D[e] = r.v[e];
  }
}

template <typename T>
__global__ __launch_bounds__(256) void gemm_splitk_finish_kernel(GemmArgs g, int nsplit) {
  const int64_t plane = (int64_t)g.M * g.ws_ld, quads = plane / 4;
  const int qpr = g.ws_ld / 4;  // quads per row
  for (int64_t qd = (int64_t)blockIdx.x * 256 + threadIdx.x; qd < quads; qd += (int64_t)gridDim.x * 256) {
    const int64_t e0 = qd * 4;
    f32x4 sum = *reinterpret_cast<const f32x4*>(g.ws + e0);
    for (int sp = 1; sp < nsplit; ++sp) sum += *reinterpret_cast<const f32x4*>(g.ws + sp * plane + e0);
    const int64_t m = qd / qpr;
    finish_store<T>(g, sum, m, (qd - m * qpr) * 4);
  }
}

// The same for outputs too small to fill the chip with one thread per four columns: four
// neighbouring lanes share a group of four columns, each sums every fourth partial plane, and
// two DPP steps combine them.
template <typename T>
__global__ __launch_bounds__(256) void gemm_splitk_finish4_kernel(GemmArgs g, int nsplit) {
  const int64_t plane = (int64_t)g.M * g.ws_ld, quads = plane / 4;
  const int qpr = g.ws_ld / 4;
  const int part = threadIdx.x & 3;
  const int64_t stride = (int64_t)gridDim.x * 64;
  const int64_t rounds = (quads + stride - 1) / stride;  // every lane of a wave stays in the loop: the combine below is wave-wide
  for (int64_t r = 0; r < rounds; ++r) {
    const int64_t qd = r * stride + (int64_t)blockIdx.x * 64 + (threadIdx.x >> 2);
    const bool live = qd < quads;
    const int64_t e0 = live ? qd * 4 : 0;
    f32x4 sum = {0.f, 0.f, 0.f, 0.f};
    if (live)
      for (int sp = part; sp < nsplit; sp += 4) sum += *reinterpret_cast<const f32x4*>(g.ws + sp * plane + e0);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float v = sum[e];
      v += dpp<0xB1>(v);  // lanes 0<->1, 2<->3
      v += dpp<0x4E>(v);  // pairs
      sum[e] = v;
    }
    if (!live || part != 0) continue;
    const int64_t m = qd / qpr;
    finish_store<T>(g, sum, m, (qd - m * qpr) * 4);
  }
}



// ---------------------------------------------------------------- epilogue
// A wave's (32 MI)x64 result: register r of acc[i][j] in lane l is C[m0 + 32 i + l%32][n0 + 32 j +
// 8 (r/4) + 4 (l/32) + r%4] (operands were swapped, so a lane owns runs of 4 consecutive n).
// Writing those 8-byte runs straight to global memory leaves every 128-byte line to be
// assembled from 16 stores in L2, and the epilogue then costs more than a tenth of the whole
// GEMM.  Instead the wave applies alpha / beta * c in fp32, parks the rounded tile in its own
// 16 KB slice of the (now idle) LDS ring, and reads it back row-major: every global store
// instruction then writes 8 complete 128-byte rows.  Must be called by all waves after the
// last barrier of the main loop (the ring is no longer read).
// A wave with more than two 32-column blocks (NJ > 2) calls this once per pair of blocks, J0 = 0, 2, ...;
// NB = 1 stores the single block J0 (the last one of an odd count): the left 64 bytes of every slab row.
template <typename T, int MI, int J0 = 0, int NB = 2, int NJ>
__device__ __forceinline__ void store_tile_result(const GemmArgs& g, const f32x16 (&acc)[MI][NJ], unsigned char* lds,
                                                  int wave, int lane, int m0, int n0) {
  const int fr = lane & 31, fg = lane >> 5;
  const T* C = static_cast<const T*>(g.c);
  const bool use_c = C != nullptr && g.beta != 0.f;
  unsigned char* slab = lds + wave * (MI * 32 * 128);  // MI * 32 rows x 128 bytes
  // A bias row (c broadcast along m: the Linear-layer addmm) is the same for every row of the
  // tile: its 8 groups of four columns are loaded once, scaled by beta, and reused for all rows.
  const bool row_bias = use_c && g.bias_vec;
  float bias[NB][4][4];
  if (row_bias) {
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + j * 32 + q * 8 + fg * 4;
        const VecN4<T> t = *reinterpret_cast<const VecN4<T>*>(C + (n + 4 <= g.N ? n : 0));
#pragma unroll
        for (int e = 0; e < 4; ++e) bias[j][q][e] = g.beta * static_cast<float>(t.v[e]);
        if (n < g.N && n + 4 > g.N) {  // the last columns of an N that is no multiple of 4
#pragma unroll
          for (int e = 0; e < 4; ++e) bias[j][q][e] = g.beta * static_cast<float>(C[n + e < g.N ? n + e : g.N - 1]);
        }
      }
  }
  // 16-byte slot s of row r lives at slot s ^ ((r/2) % 8): two-way conflicts at most on both sides
  auto stage = [&](auto ROW_BIAS) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < MI; ++i) {
      const int row = i * 32 + fr;
      const int m = m0 + row;
      const int mc = m < g.M ? m : g.M - 1;
#pragma unroll
      for (int j = 0; j < NB; ++j) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int nl = j * 32 + q * 8 + fg * 4;
          const int n = n0 + nl;
          VecN4<T> r;
          if constexpr (decltype(ROW_BIAS)::value) {
#pragma unroll
            for (int e = 0; e < 4; ++e) r.v[e] = static_cast<T>(g.alpha * acc[i][J0 + j][q * 4 + e] + bias[j][q][e]);
          } else {
            // Columns past N are computed on valid addresses and never stored.
            float cv[4] = {0.f, 0.f, 0.f, 0.f};
            if (use_c) {
              if (g.c_vec) {  // N % 4 == 0: a group of four columns is wholly inside or wholly outside
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
              const float v = g.alpha * acc[i][J0 + j][q * 4 + e];
              r.v[e] = static_cast<T>(use_c ? v + g.beta * cv[e] : v);
            }
          }
          const int slot = (j * 4 + q) ^ ((row >> 1) & 7);
          *reinterpret_cast<VecN4<T>*>(slab + row * 128 + slot * 16 + fg * 8) = r;
        }
      }
    }
  };
  if (row_bias) stage(std::true_type{});
  else stage(std::false_type{});
  // same wave wrote and reads: LDS operations of a wave complete in order
  T* D = static_cast<T*>(g.out);
  if (g.out_vec) {
#pragma unroll
    for (int t = 0; t < MI * 4; ++t) {
      const int chunk = t * kWave + lane;  // MI * 256 chunks of 16 bytes, 8 per row
      const int row = chunk >> 3, s = chunk & 7;
      const u32x4 v = *reinterpret_cast<const u32x4*>(slab + row * 128 + ((s ^ ((row >> 1) & 7)) << 4));
      const int m = m0 + row, n = n0 + s * 8;
      if (m >= g.M || n >= g.N || s >= NB * 4) continue;
      *reinterpret_cast<u32x4*>(D + (int64_t)m * g.N + n) = v;
    }
  } else {
    // N not a multiple of 8 (e.g. a 50257-wide vocabulary): the rows of out start at any 2-byte
    // offset; the lanes walk the 16-byte grid of the destination (store_slab_rows_shifted).
    const int rows = g.M - m0 < MI * 32 ? g.M - m0 : MI * 32;
    const int cols = g.N - n0 < NB * 32 ? g.N - n0 : NB * 32;
    store_slab_rows_shifted<T, MI * 32>(slab, D, g.N, m0, rows, n0, cols, lane);
  }
}

// ---------------------------------------------------------------- MFMA kernel
// 256x256 block tile, BK = 32, a ring of four 32 KB LDS stages (A 256x32 + B 32x256 each).
// In iteration `it` a wave (a) writes tile it+2 from registers into the ring, (b) starts the
// global loads of tile it+3, (c) multiplies tile `it`, and already reads the first fragments
// of tile it+1 — visible since the previous barrier — before it reaches the barrier, so the
// MFMA pipe has work the moment the barrier opens.  The slot being overwritten held tile
// it-2, which every wave finished before the previous barrier.
constexpr int BK3 = 32;
constexpr int kStages3 = 4;
constexpr int kPanel3 = BM * BK3 * 2;        // 16 KB per operand per stage
constexpr int kStage3 = 2 * kPanel3;         // 32 KB
constexpr int kGemmLds = kStages3 * kStage3;  // 128 KB

// K-contiguous panel with 64-byte rows (4 chunks): four consecutive rows fill the four 64-byte
// segments of the 256-byte bank window and the XOR with (r/4)%4 moves each group of four rows
// to another 16-byte position.  The 16 lanes of one ds_read_b128 pass hold rows {0-3, 12-15,
// 20-27} or {4-11, 16-19, 28-31} of a fragment (see swz_k64): in both sets (r/4)%4 takes every
// value once, so a pass touches 16 distinct positions (SQ_LDS_BANK_CONFLICT reads 0).
__device__ __forceinline__ int swz_k32(int r, int c) { return r * 64 + ((c ^ ((r >> 2) & 3)) << 4); }

// KTAIL: K is not a multiple of BK3, so chunks past K are zero-filled (branch-free: the address
// is clamped and the loaded value replaced); the common case compiles without the checks.
template <typename T, bool B_NN, bool KTAIL>
__global__ __launch_bounds__(512) void gemm_mfma_kernel(GemmArgs g) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  using frag_t = typename Mfma<T>::frag;
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int wm = wave >> 2, wn = wave & 3;  // wave tile: rows wm*128.., cols wn*64..
  int tm, tn;
  tile_coords(g, tm, tn);
  const int bm = tm * BM, bn = tn * BN;
  const T* A = static_cast<const T*>(g.a);
  const T* B = static_cast<const T*>(g.b);

  u32x4 ra[2], rb[2];
  const int lc = tid & 3, lr = tid >> 2;   // K-contiguous panels: chunk lc of rows lr + 128*i
  const int nu = tid & 31, kr = tid >> 5;  // NN B: 16-byte unit nu of k rows kr + 16*i
  const u32x4 zero4 = {0, 0, 0, 0};
  const T* a_ptr[2];
  const T* b_ptr[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    int gr = bm + lr + 128 * i;
    gr = gr < g.M ? gr : g.M - 1;
    a_ptr[i] = A + (int64_t)gr * g.lda + lc * 8;
    if constexpr (!B_NN) {
      int gn = bn + lr + 128 * i;
      gn = gn < g.N ? gn : g.N - 1;
      b_ptr[i] = B + (int64_t)gn * g.ldb + lc * 8;
    } else {
      int gn = bn + nu * 8;
      gn = gn < g.N ? gn : 0;
      b_ptr[i] = B + (int64_t)(kr + 16 * i) * g.ldb + gn;
    }
  }
  auto load_tile = [&](int t) {
    const int k0 = t * BK3;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const bool in_a = !KTAIL || k0 + lc * 8 < g.K;
      const u32x4 va = *reinterpret_cast<const u32x4*>(a_ptr[i] + (in_a ? k0 : 0));
      ra[i] = in_a ? va : zero4;
      if constexpr (!B_NN) {
        const u32x4 vb = *reinterpret_cast<const u32x4*>(b_ptr[i] + (in_a ? k0 : 0));
        rb[i] = in_a ? vb : zero4;
      } else {
        const bool in_b = !KTAIL || k0 + kr + 16 * i < g.K;
        const u32x4 vb = *reinterpret_cast<const u32x4*>(b_ptr[i] + (int64_t)(in_b ? k0 : 0) * g.ldb);
        rb[i] = in_b ? vb : zero4;
      }
    }
  };
  auto store_tile = [&](int t) {
    unsigned char* pa = lds + (t % kStages3) * kStage3;
    unsigned char* pb = pa + kPanel3;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      *reinterpret_cast<u32x4*>(pa + swz_k32(lr + 128 * i, lc)) = ra[i];
      if constexpr (!B_NN) *reinterpret_cast<u32x4*>(pb + swz_k32(lr + 128 * i, lc)) = rb[i];
      else *reinterpret_cast<u32x4*>(pb + swz_n(kr + 16 * i, nu)) = rb[i];
    }
  };

  const int fr = lane & 31, fg = lane >> 5;
  const int tr_k = fg * 8 + ((lane & 15) >> 2);
  const int tr_n = (((lane >> 4) & 1) << 4) + ((lane & 3) << 2);
  auto read_frags = [&](int t, int ks, frag_t (&fa)[4], frag_t (&fb)[2]) {
    const unsigned char* pa = lds + (t % kStages3) * kStage3;
    const unsigned char* pb = pa + kPanel3;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      fa[i] = *reinterpret_cast<const frag_t*>(pa + swz_k32(wm * 128 + i * 32 + fr, ks * 2 + fg));
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      if constexpr (!B_NN) {
        fb[j] = *reinterpret_cast<const frag_t*>(pb + swz_k32(wn * 64 + j * 32 + fr, ks * 2 + fg));
      } else {
        const int k = ks * 16 + tr_k;
        const int n = wn * 64 + j * 32 + tr_n;
        const s16x4 lo = lds_read_tr(pb + swz_n(k, n >> 3) + ((n & 7) << 1));
        const s16x4 hi = lds_read_tr(pb + swz_n(k + 4, n >> 3) + ((n & 7) << 1));
        fb[j] = __builtin_bit_cast(frag_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      }
    }
  };

  f32x16 acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  auto mma = [&](frag_t (&fa)[4], frag_t (&fb)[2]) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[i][j] = Mfma<T>::run(fb[j], fa[i], acc[i][j]);
  };

  const int nk = (g.K + BK3 - 1) / BK3;
  if (nk > 0) { load_tile(0); store_tile(0); }
  if (nk > 1) { load_tile(1); store_tile(1); }
  if (nk > 2) load_tile(2);
  __syncthreads();
  frag_t fa0[4], fb0[2], fa1[4], fb1[2];
  if (nk > 0) read_frags(0, 0, fa0, fb0);
  for (int it = 0; it < nk; ++it) {
    if (it + 2 < nk) store_tile(it + 2);
    if (it + 3 < nk) load_tile(it + 3);
    read_frags(it, 1, fa1, fb1);
    mma(fa0, fb0);
    if (it + 1 < nk) read_frags(it + 1, 0, fa0, fb0);
    mma(fa1, fb1);
    __syncthreads();
  }

  store_tile_result<T, 4>(g, acc, lds, wave, lane, bm + wm * 128, bn + wn * 64);
}

// ---------------------------------------------------------------- MFMA kernel, direct-to-LDS fills
// Same tiling, ring and fragment reads as gemm_mfma_kernel, but the panels are filled with
// global_load_lds_dwordx4: each wave-level load moves 64 x 16 bytes from global memory straight
// into 1 KB of LDS (lane l lands at M0 + 16 l), without passing through VGPRs and without
// ds_write instructions.  Because the LDS position of a lane is fixed, the swizzle is applied
// on the global side: a lane fetches the chunk that belongs at its LDS position.
// Tile it+3 is requested at the start of iteration `it` into the slot tile it-1 just left, and
// must have landed by the end of iteration it+1 (s_waitcnt vmcnt(4): only the four loads of
// the newest tile may still be in flight), so every tile has two iterations to arrive.  The
// loads are issued from inline asm, so the compiler's own wait-count bookkeeping does not see
// them and adds no waits of its own.  Needs K % 32 == 0 (no zero fill on this path).

template <typename T, bool B_NN>
__global__ __launch_bounds__(512) void gemm_mfma_dma_kernel(GemmArgs g) {
  constexpr int S = kStages3;   // ring depth
  constexpr bool PF = true;     // fragments of the next tile are read before the barrier
  constexpr bool SCHED = true;  // pin the MFMA / DS-read interleave
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  using frag_t = typename Mfma<T>::frag;
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave >> 2, wn = wave & 3;
  int tm, tn;
  tile_coords(g, tm, tn);
  const int bm = tm * BM, bn = tn * BN;
  const T* A = static_cast<const T*>(g.a);
  const T* B = static_cast<const T*>(g.b);
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;  // LDS-relative address of the ring

  // Per-lane source pointers of this wave's four 1 KB regions per tile (two per panel): region
  // q = wave + 8 i of a panel is LDS bytes [q*1024, q*1024 + 1024).
  const T* a_src[2];
  const T* b_src[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int q = wave + 8 * i;
    {  // K-contiguous A panel: region q = rows 16q .. 16q+15, 4 chunks per row
      const int r = 16 * q + (lane >> 2), slot = lane & 3;
      const int c = slot ^ ((r >> 2) & 3);
      int gr = bm + r;
      gr = gr < g.M ? gr : g.M - 1;
      a_src[i] = A + (int64_t)gr * g.lda + c * 8;
    }
    if constexpr (!B_NN) {
      const int r = 16 * q + (lane >> 2), slot = lane & 3;
      const int c = slot ^ ((r >> 2) & 3);
      int gn = bn + r;
      gn = gn < g.N ? gn : g.N - 1;
      b_src[i] = B + (int64_t)gn * g.ldb + c * 8;
    } else {  // N-contiguous B panel: region q = k rows 2q, 2q+1, 32 units per row
      const int k = 2 * q + (lane >> 5), pos = lane & 31;
      const int u = (((pos >> 2) ^ (k & 3)) << 2) | (pos & 3);
      int gn = bn + u * 8;
      gn = gn < g.N ? gn : 0;
      b_src[i] = B + (int64_t)k * g.ldb + gn;
    }
  }
  auto request_tile = [&](int t) {
    const uint32_t stage = lds_base + (uint32_t)(t % S) * kStage3;
    const int64_t k0 = (int64_t)t * BK3;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const uint32_t region = (uint32_t)(wave + 8 * i) * 1024u;
      lds_dma16(stage + region, a_src[i] + k0);
      if constexpr (!B_NN) lds_dma16(stage + kPanel3 + region, b_src[i] + k0);
      else lds_dma16(stage + kPanel3 + region, b_src[i] + k0 * g.ldb);
    }
  };

  const int fr = lane & 31, fg = lane >> 5;
  const int tr_k = fg * 8 + ((lane & 15) >> 2);
  const int tr_n = (((lane >> 4) & 1) << 4) + ((lane & 3) << 2);
  auto read_frags = [&](int t, int ks, frag_t (&fa)[4], frag_t (&fb)[2]) {
    const unsigned char* pa = lds + (t % S) * kStage3;
    const unsigned char* pb = pa + kPanel3;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      fa[i] = *reinterpret_cast<const frag_t*>(pa + swz_k32(wm * 128 + i * 32 + fr, ks * 2 + fg));
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      if constexpr (!B_NN) {
        fb[j] = *reinterpret_cast<const frag_t*>(pb + swz_k32(wn * 64 + j * 32 + fr, ks * 2 + fg));
      } else {
        const int k = ks * 16 + tr_k;
        const int n = wn * 64 + j * 32 + tr_n;
        const s16x4 lo = lds_read_tr(pb + swz_n(k, n >> 3) + ((n & 7) << 1));
        const s16x4 hi = lds_read_tr(pb + swz_n(k + 4, n >> 3) + ((n & 7) << 1));
        fb[j] = __builtin_bit_cast(frag_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      }
    }
  };

  f32x16 acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  auto mma = [&](frag_t (&fa)[4], frag_t (&fb)[2]) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[i][j] = Mfma<T>::run(fb[j], fa[i], acc[i][j]);
  };

  // Ring of S stages; PF = fragments of the next tile are read before the barrier.  At the wait
  // point of iteration `it`, tile it+1+PF must have landed; the S-2-PF newer tiles may fly on.
  constexpr int FLY = S - 2 - (PF ? 1 : 0);
  const int nk = g.K / BK3;
  for (int t = 0; t < S - 1 && t < nk; ++t) request_tile(t);
  if (nk >= S - 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(4 * FLY) : "memory");
  else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  frag_t fa0[4], fb0[2], fa1[4], fb1[2];
  read_frags(0, 0, fa0, fb0);
  int it = 0;
  // Steady state: no conditions inside, so the body is one scheduling region.  The MFMAs of a
  // 16-k step are interleaved with the LDS reads of the following step (SCHED: one MFMA, then
  // one or two DS reads), so the matrix pipe and the LDS pipe of a wave work at the same time.
  for (; it + S - 1 < nk; ++it) {
    request_tile(it + S - 1);
    read_frags(it, 1, fa1, fb1);
    mma(fa0, fb0);
    if constexpr (PF) read_frags(it + 1, 0, fa0, fb0);
    mma(fa1, fb1);
    if constexpr (SCHED) {
#define MI355_MFMA_THEN_READS                              \
  __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);       \
  __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);       \
  __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);       \
  __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      MI355_MFMA_THEN_READS MI355_MFMA_THEN_READS MI355_MFMA_THEN_READS MI355_MFMA_THEN_READS
      MI355_MFMA_THEN_READS MI355_MFMA_THEN_READS MI355_MFMA_THEN_READS MI355_MFMA_THEN_READS
#undef MI355_MFMA_THEN_READS
    }
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(4 * FLY) : "memory");
    __syncthreads();
    if constexpr (!PF) read_frags(it + 1, 0, fa0, fb0);
  }
  for (; it < nk; ++it) {  // drain: nothing left to request
    read_frags(it, 1, fa1, fb1);
    mma(fa0, fb0);
    if (PF && it + 1 < nk) read_frags(it + 1, 0, fa0, fb0);
    mma(fa1, fb1);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (!PF && it + 1 < nk) read_frags(it + 1, 0, fa0, fb0);
  }

  store_tile_result<T, 4>(g, acc, lds, wave, lane, bm + wm * 128, bn + wn * 64);
}

// ---------------------------------------------------------------- MFMA kernel, full-line A fills
// K % 64 == 0, either B layout.  As gemm_mfma_dma_kernel, except that the A panel is
// fetched 64 k (one whole 128-byte line per row) at a time: with 32-k steps every line of A is
// requested twice, 64 bytes each, which halves the useful width of each L2 request and was
// measured to hold the A stream to ~13.5 TB/s chip-wide against ~21.5 TB/s for whole lines.
// LDS: three A slots of 256 x 64 (32 KB, rows of 128 B, swz_k64) and four B slots of 32 x 256
// (16 KB, swz_n) = 160 KB.  A step is still 32 k.  At the start of an even step t the A slot
// that steps t-2, t-1 used is refilled with k-range of steps t+4, t+5 (four loads per lane);
// every step t refills the B slot of step t-1 with step t+3 (two loads per lane).  The first
// fragments of step t+1 are read before the barrier that ends step t, so at that barrier the
// panels of step t+2 must have landed: only the loads issued in step t itself may still fly
// (s_waitcnt vmcnt(6) after an even step, vmcnt(2) after an odd one).
constexpr int kASlot64 = BM * 64 * 2;                 // 32 KB
constexpr int kBRing64 = 3 * kASlot64;                // B slots start here
constexpr int kGemmLds64 = kBRing64 + 4 * kPanel3;    // 160 KB
// K-contiguous panel with 128-byte rows (8 chunks).  A ds_read_b128 is served in four passes of
// 16 lanes, and the passes are not runs of consecutive lanes: measured on gfx950 they are lanes
// {0-3, 12-15, 20-27}, {4-11, 16-19, 28-31} and the same sets + 32.  A fragment read puts rows
// r0 + lane%32 in the lanes, so the rows of one pass are {0-3, 12-15, 20-27} or the rest; the
// XOR term (bits 1, 3, 4 of the row) takes all eight values over the even rows of either set
// and over the odd rows, which with the row parity selecting the 128-byte half gives the 16
// lanes of a pass 16 distinct 16-byte positions of the 256-byte bank window.
__device__ __forceinline__ int swz_k64(int r, int c) {
  return r * 128 + ((c ^ (((r >> 1) & 1) | ((r >> 2) & 6))) << 4);
}

template <typename T, bool B_NN>
__global__ __launch_bounds__(512) void gemm_mfma_dma64_kernel(GemmArgs g) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  using frag_t = typename Mfma<T>::frag;
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave >> 2, wn = wave & 3;
  int tm, tn;
  tile_coords(g, tm, tn);
  const int bm = tm * BM, bn = tn * BN;
  const T* A = static_cast<const T*>(g.a);
  const T* B = static_cast<const T*>(g.b);
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;

  // A: region q = wave + 8 i (i < 4) of a slot is rows 8q .. 8q+7, eight 16-byte chunks per row.
  // B: region q = wave + 8 i (i < 2) of a slot is k rows 2q, 2q+1, 32 units per row.
  const T* a_src[4];
  const T* b_src[2];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = 8 * (wave + 8 * i) + (lane >> 3), slot = lane & 7;
    const int c = slot ^ (((r >> 1) & 1) | ((r >> 2) & 6));
    int gr = bm + r;
    gr = gr < g.M ? gr : g.M - 1;
    a_src[i] = A + (int64_t)gr * g.lda + c * 8;
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    if constexpr (B_NN) {
      const int k = 2 * (wave + 8 * i) + (lane >> 5), pos = lane & 31;
      const int u = (((pos >> 2) ^ (k & 3)) << 2) | (pos & 3);
      int gn = bn + u * 8;
      gn = gn < g.N ? gn : 0;
      b_src[i] = B + (int64_t)k * g.ldb + gn;
    } else {  // K-contiguous B ([N][K]): 64-byte rows per step, as the A panel of gemm_mfma_dma_kernel
      const int r = 16 * (wave + 8 * i) + (lane >> 2), slot = lane & 3;
      const int c = slot ^ ((r >> 2) & 3);
      int gn = bn + r;
      gn = gn < g.N ? gn : g.N - 1;
      b_src[i] = B + (int64_t)gn * g.ldb + c * 8;
    }
  }
  // a_slot: byte offset of the A slot to fill; t: first of the two steps it will hold.
  auto request_a = [&](int t, uint32_t a_slot) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      lds_dma16(lds_base + a_slot + (uint32_t)(wave + 8 * i) * 1024u, a_src[i] + (int64_t)t * BK3);
  };
  auto request_b = [&](int t) {
    const uint32_t stage = lds_base + kBRing64 + (uint32_t)(t & 3) * kPanel3;
#pragma unroll
    for (int i = 0; i < 2; ++i)
      lds_dma16(stage + (uint32_t)(wave + 8 * i) * 1024u, b_src[i] + (B_NN ? (int64_t)t * BK3 * g.ldb : (int64_t)t * BK3));
  };

  const int fr = lane & 31, fg = lane >> 5;
  const int tr_k = fg * 8 + ((lane & 15) >> 2);
  const int tr_n = (((lane >> 4) & 1) << 4) + ((lane & 3) << 2);
  // Fragments of 16-k sub-step ks (0, 1) of step t, whose A data is half `half` of `a_slot`.
  auto read_frags = [&](int t, uint32_t a_slot, int half, int ks, frag_t (&fa)[4], frag_t (&fb)[2]) {
    const unsigned char* pa = lds + a_slot;
    const unsigned char* pb = lds + kBRing64 + (t & 3) * kPanel3;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      fa[i] = *reinterpret_cast<const frag_t*>(pa + swz_k64(wm * 128 + i * 32 + fr, half * 4 + ks * 2 + fg));
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      if constexpr (B_NN) {
        const int k = ks * 16 + tr_k;
        const int n = wn * 64 + j * 32 + tr_n;
        const s16x4 lo = lds_read_tr(pb + swz_n(k, n >> 3) + ((n & 7) << 1));
        const s16x4 hi = lds_read_tr(pb + swz_n(k + 4, n >> 3) + ((n & 7) << 1));
        fb[j] = __builtin_bit_cast(frag_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      } else {
        fb[j] = *reinterpret_cast<const frag_t*>(pb + swz_k32(wn * 64 + j * 32 + fr, ks * 2 + fg));
      }
    }
  };

  f32x16 acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  auto mma = [&](frag_t (&fa)[4], frag_t (&fb)[2]) {
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i][j] = Mfma<T>::run(fb[j], fa[i], acc[i][j]);
  };
  auto next_slot = [](uint32_t s) { return s + kASlot64 == (uint32_t)kBRing64 ? 0u : s + kASlot64; };

#define MI355_MFMA_THEN_READS                              \
  __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);       \
  __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);       \
  __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);       \
  __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
#define MI355_STEP_SCHEDULE                                                                   \
  MI355_MFMA_THEN_READS MI355_MFMA_THEN_READS MI355_MFMA_THEN_READS MI355_MFMA_THEN_READS     \
  MI355_MFMA_THEN_READS MI355_MFMA_THEN_READS MI355_MFMA_THEN_READS MI355_MFMA_THEN_READS

  const int nk = g.K / BK3;  // even: K % 64 == 0
  request_a(0, 0);
  if (nk > 2) request_a(2, kASlot64);
  request_b(0);
  if (nk > 1) request_b(1);
  if (nk > 2) request_b(2);
  if (nk > 2) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
  else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  frag_t fa0[4], fb0[2], fa1[4], fb1[2];
  uint32_t cur = 0;  // A slot of steps t, t+1
  read_frags(0, cur, 0, 0, fa0, fb0);
  int t = 0;
  // Steady state, two steps per trip and no conditions inside: each half is one scheduling
  // region in which the MFMAs of a 16-k sub-step are interleaved with the LDS reads of the
  // following one.
  for (; t + 5 < nk; t += 2) {
    const uint32_t nxt = next_slot(cur);
    // even step t
    request_a(t + 4, next_slot(nxt));
    request_b(t + 3);
    read_frags(t, cur, 0, 1, fa1, fb1);
    mma(fa0, fb0);
    read_frags(t + 1, cur, 1, 0, fa0, fb0);
    mma(fa1, fb1);
    MI355_STEP_SCHEDULE
    asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
    __syncthreads();
    // odd step t+1
    request_b(t + 4);
    read_frags(t + 1, cur, 1, 1, fa1, fb1);
    mma(fa0, fb0);
    read_frags(t + 2, nxt, 0, 0, fa0, fb0);
    mma(fa1, fb1);
    MI355_STEP_SCHEDULE
    asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
    __syncthreads();
    cur = nxt;
  }
#undef MI355_STEP_SCHEDULE
#undef MI355_MFMA_THEN_READS
  for (; t < nk; ++t) {  // drain: every A slot is already requested, B may lack up to two steps
    const int half = t & 1;
    if (t + 3 < nk) request_b(t + 3);
    read_frags(t, cur, half, 1, fa1, fb1);
    mma(fa0, fb0);
    const uint32_t nxt = half ? next_slot(cur) : cur;
    if (t + 1 < nk) read_frags(t + 1, nxt, half ^ 1, 0, fa0, fb0);
    mma(fa1, fb1);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    cur = nxt;
  }

  store_tile_result<T, 4>(g, acc, lds, wave, lane, bm + wm * 128, bn + wn * 64);
}

constexpr int SBM = 128, SBN = 128;
// N-contiguous B panel of the 128-wide tile: 256 B per k row, 64-byte segments rotated by k % 4.
__device__ __forceinline__ int swz_n128(int k, int u) {
  return k * (SBN * 2) + ((((u >> 2) ^ (k & 3))) << 6) + ((u & 3) << 4);
}

// ---------------------------------------------------------------- MFMA kernel, four waves of 128x128
// Same LDS layout, fills and step structure as gemm_mfma_dma64_kernel, with the 256x256 tile
// split over four waves (2x2, one per SIMD) instead of eight: each wave owns 128x128 = 4x4 MFMA
// blocks (256 fp32 accumulators) and reads 4 + 4 fragments for 16 MFMAs per 16-k sub-step, where
// the eight-wave form reads 4 + 2 for 8 — one third fewer LDS fragment bytes per flop.  Every
// lane issues twice the fills (A: region q = wave + 4 i, i < 8; B: q = wave + 4 i, i < 4).
// NJ = 2 is the same kernel on a 256x128 tile (wave tiles of 128x64, half the B panel) for
// problems that do not fill the chip with 256x256 tiles.
// A_T: the left operand is M-contiguous (a transposed view, e.g. x.t() @ dy): its panel stays k-major
// in LDS like a row-major B and is transposed by the LDS read.
// NJA < NJ (3 of 4): the tile is 32 NJA x 2 columns wide (256 x 192) on the LDS layout and fills of the
// NJ form; the panel columns past the tile are fetched (clamped at the matrix edge) and not used.
// Such tiles cost about three quarters of a 256 x 256 one and let a last, partly filled round
// of tiles be cut to fit the chip (see gemm_mfma_w4_mixed_kernel).
template <typename T, bool B_NN, int NJ, bool A_T, int NJA = NJ>
__device__ __forceinline__ void w4_tile(const GemmArgs& g, unsigned char* lds, const int bm, const int bn) {
  static_assert(NJ == 2 || NJ == 4, "wave tile is 128 x 32 NJ");
  static_assert(NJA == NJ || (NJ == 4 && NJA == 3), "narrow form: three of four column blocks");
  using frag_t = typename Mfma<T>::frag;
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave >> 1, wn = wave & 1;
  const T* A = static_cast<const T*>(g.a);
  const T* B = static_cast<const T*>(g.b);
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;
#ifdef MI355_GEMM_TRACE
  const uint64_t tr_entry = __builtin_readcyclecounter();
#endif

  // Fill addresses: a uniform base per operand (moved along k by the requests) plus one 32-bit byte
  // offset per lane and request (the host checks that they fit: leading dimensions below 4 M elements).
  const T* a_base = A_T ? A : A + (int64_t)bm * g.lda;   // K-contiguous A: offsets are relative to the tile's first row
  const T* b_base = B_NN ? B : B + (int64_t)bn * g.ldb;  // K-contiguous B: relative to the tile's first column
  // B_PAIR (a K-contiguous B on the 256x128 tile, whose LDS has the room): B is fetched like A, 64 k - one whole
  // 128-byte line per column - at a time into three pair slots of 128 x 64 (16 KB, swz_k64) instead of four step
  // slots of 128 x 32.  With 32-k requests every line of B is asked for twice, 64 bytes each time, the second while
  // the first may still be on its way from HBM.
  constexpr bool B_PAIR = !B_NN && NJ == 2;
  constexpr int NB_OFF = B_PAIR ? 4 : NJ;
  uint32_t a_off[8];
  uint32_t b_off[NB_OFF];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    if constexpr (A_T) {  // M-contiguous A: the pair slot holds 64 k-rows of 512 B (swz_n), region = two k-rows
      const int k = 2 * (wave + 4 * i) + (lane >> 5), pos = lane & 31;
      const int u = (((pos >> 2) ^ (k & 3)) << 2) | (pos & 3);
      int gm = bm + u * 8;
      gm = gm < g.M ? gm : 0;
      a_off[i] = ((uint32_t)k * (uint32_t)g.lda + (uint32_t)gm) * 2u;
    } else {
      const int r = 8 * (wave + 4 * i) + (lane >> 3), slot = lane & 7;
      const int c = slot ^ (((r >> 1) & 1) | ((r >> 2) & 6));
      const int lr = bm + r < g.M ? r : g.M - 1 - bm;  // rows past M re-read the last row
      a_off[i] = ((uint32_t)lr * (uint32_t)g.lda + (uint32_t)c * 8u) * 2u;
    }
  }
#pragma unroll
  for (int i = 0; i < NB_OFF; ++i) {
    if constexpr (B_PAIR) {  // 128-byte rows of 64 k (swz_k64): region = eight columns
      const int r = 8 * (wave + 4 * i) + (lane >> 3), slot = lane & 7;
      const int c = slot ^ (((r >> 1) & 1) | ((r >> 2) & 6));
      const int ln = bn + r < g.N ? r : g.N - 1 - bn;
      b_off[i] = ((uint32_t)ln * (uint32_t)g.ldb + (uint32_t)c * 8u) * 2u;
    } else if constexpr (B_NN && NJ == 4) {  // 512-byte k-rows (swz_n): region = two k-rows
      const int k = 2 * (wave + 4 * i) + (lane >> 5), pos = lane & 31;
      const int u = (((pos >> 2) ^ (k & 3)) << 2) | (pos & 3);
      int gn = bn + u * 8;
      gn = gn < g.N ? gn : 0;
      b_off[i] = ((uint32_t)k * (uint32_t)g.ldb + (uint32_t)gn) * 2u;
    } else if constexpr (B_NN) {  // 256-byte k-rows (swz_n128): region = four k-rows
      const int k = 4 * (wave + 4 * i) + (lane >> 4), pos = lane & 15;
      const int u = (((pos >> 2) ^ (k & 3)) << 2) | (pos & 3);
      int gn = bn + u * 8;
      gn = gn < g.N ? gn : 0;
      b_off[i] = ((uint32_t)k * (uint32_t)g.ldb + (uint32_t)gn) * 2u;
    } else {
      const int r = 16 * (wave + 4 * i) + (lane >> 2), slot = lane & 3;
      const int c = slot ^ ((r >> 2) & 3);
      const int ln = bn + r < g.N ? r : g.N - 1 - bn;
      b_off[i] = ((uint32_t)ln * (uint32_t)g.ldb + (uint32_t)c * 8u) * 2u;
    }
  }
  // Fill requests: A request i (0..7) of the slot at byte offset a_slot, holding steps t, t+1;
  // B request i (0..NJ-1) of step t.
  auto request_a = [&](int i, int t, uint32_t a_slot) {
    lds_dma16s(lds_base + a_slot + (uint32_t)(wave + 4 * i) * 1024u, a_off[i],
               a_base + (A_T ? (int64_t)t * BK3 * g.lda : (int64_t)t * BK3));
  };
  auto request_b = [&](int i, int t) {
    lds_dma16s(lds_base + kBRing64 + (uint32_t)(t & 3) * kPanel3 + (uint32_t)(wave + 4 * i) * 1024u, b_off[i % NB_OFF],
               b_base + (B_NN ? (int64_t)t * BK3 * g.ldb : (int64_t)t * BK3));
  };
  // B_PAIR: request i (0..3) of the B pair slot that goes with the A slot at a_slot (steps t, t+1)
  auto request_b_pair = [&](int i, int t, uint32_t a_slot) {
    lds_dma16s(lds_base + kBRing64 + a_slot / 2 + (uint32_t)(wave + 4 * i) * 1024u, b_off[i % NB_OFF], b_base + (int64_t)t * BK3);
  };

  const int fr = lane & 31, fg = lane >> 5;
  const int tr_k = fg * 8 + ((lane & 15) >> 2);
  const int tr_n = (((lane >> 4) & 1) << 4) + ((lane & 3) << 2);
  // The LDS reads of step t (A in half `half` of a_slot) into one register set, with this step's
  // eight fill requests threaded behind the reads of the second sub-step in program order — A
  // request a_first .. a_first+3 of the slot fill_slot (steps ta, ta+1), then the four B requests
  // of step tb — so that the fills leave the wave one at a time over the second half of the step
  // instead of as a burst behind the barrier (the burst form ran the all-zero GEMM 20 % slower).
  auto io_step = [&](int t, uint32_t a_slot, int half, frag_t (&xa)[2][4], frag_t (&xb)[2][NJA], bool fill_a, int ta,
                     uint32_t fill_slot, int a_first, bool fill_b, int tb) __attribute__((always_inline)) {
    const unsigned char* pa = lds + a_slot;
    const unsigned char* pb = B_PAIR ? lds + kBRing64 + a_slot / 2 : lds + kBRing64 + (t & 3) * kPanel3;
    auto fill = [&](int q) __attribute__((always_inline)) {
      if (q < 4) {
        if (fill_a) request_a(a_first + q, ta, fill_slot);
      } else if constexpr (B_PAIR) {  // the B pair follows the A pair: requests 0, 1 with A's 0-3, requests 2, 3 with A's 4-7
        if (fill_a) request_b_pair(a_first / 2 + q - 4, ta, fill_slot);
      } else if (fill_b) {
        request_b(q - 4, tb);
      }
    };
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if constexpr (A_T) {
          const int k = half * 32 + ks * 16 + tr_k;
          const int m = wm * 128 + i * 32 + tr_n;
          const s16x4 lo = lds_read_tr(pa + swz_n(k, m >> 3) + ((m & 7) << 1));
          const s16x4 hi = lds_read_tr(pa + swz_n(k + 4, m >> 3) + ((m & 7) << 1));
          xa[ks][i] = __builtin_bit_cast(frag_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        } else {
          xa[ks][i] = *reinterpret_cast<const frag_t*>(pa + swz_k64(wm * 128 + i * 32 + fr, half * 4 + ks * 2 + fg));
        }
        if (ks == 1) fill(i);
      }
#pragma unroll
      for (int j = 0; j < NJA; ++j) {
        if constexpr (B_NN) {
          const int k = ks * 16 + tr_k;
          const int n = wn * (NJA * 32) + j * 32 + tr_n;
          const int off_lo = NJ == 4 ? swz_n(k, n >> 3) : swz_n128(k, n >> 3);
          const int off_hi = NJ == 4 ? swz_n(k + 4, n >> 3) : swz_n128(k + 4, n >> 3);
          const s16x4 lo = lds_read_tr(pb + off_lo + ((n & 7) << 1));
          const s16x4 hi = lds_read_tr(pb + off_hi + ((n & 7) << 1));
          xb[ks][j] = __builtin_bit_cast(frag_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        } else if constexpr (B_PAIR) {
          xb[ks][j] = *reinterpret_cast<const frag_t*>(pb + swz_k64(wn * (NJA * 32) + j * 32 + fr, half * 4 + ks * 2 + fg));
        } else {
          xb[ks][j] = *reinterpret_cast<const frag_t*>(pb + swz_k32(wn * (NJA * 32) + j * 32 + fr, ks * 2 + fg));
        }
        if (ks == 1) fill(4 + j);
      }
      if constexpr (NJA < NJ)
        if (ks == 1) fill(4 + NJA);  // the fills keep the NJ form: one more B request than column blocks
    }
  };

  f32x16 acc[4][NJA];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < NJA; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  auto mma_step = [&](frag_t (&xa)[2][4], frag_t (&xb)[2][NJA]) __attribute__((always_inline)) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int j = 0; j < NJA; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i][j] = Mfma<T>::run(xb[ks][j], xa[ks][i], acc[i][j]);
  };
  auto next_slot = [](uint32_t s) { return s + kASlot64 == (uint32_t)kBRing64 ? 0u : s + kASlot64; };

  // One step = 32 MFMAs.  The LDS reads are spread over the step (16 reads: one behind every
  // second MFMA; 24 reads with a row-major B: twenty pairs MFMA/read, then every second), and
  // nothing moves across the end of the step (the compiler would otherwise sink MFMAs below the
  // barrier and leave the wait for the last read directly behind it).  NJ = 2: 16 MFMAs, 12
  // reads (16 with a row-major B), all behind the first twelve (eight) MFMAs.
#define MI355_MD __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
#define MI355_MDM MI355_MD __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
#define MI355_X4(X) X X X X
#define MI355_MDD MI355_MD __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
#define MI355_W4_SCHEDULE                                                     \
  if constexpr (NJA == 3 && A_T && B_NN) {     /* 28 reads, 24 MFMAs */       \
    MI355_X4(MI355_MDD) MI355_X4(MI355_X4(MI355_MD)) MI355_X4(MI355_MD)       \
  } else if constexpr (NJA == 3 && (A_T || B_NN)) { /* 22 / 20 reads */       \
    MI355_X4(MI355_X4(MI355_MD)) MI355_X4(MI355_MD) MI355_MD MI355_MD         \
  } else if constexpr (NJA == 3) {             /* 14 reads */                 \
    MI355_X4(MI355_MDM) MI355_X4(MI355_MDM) MI355_X4(MI355_MD) MI355_MD MI355_MD \
  } else if constexpr (NJ == 4 && A_T && B_NN) { /* 32 reads, 32 MFMAs */     \
    MI355_X4(MI355_MDD) MI355_X4(MI355_MDD) MI355_X4(MI355_X4(MI355_MD))      \
  } else if constexpr (NJ == 4 && A_T) {       /* 24 reads */                 \
    MI355_X4(MI355_X4(MI355_MD)) MI355_X4(MI355_MD) MI355_X4(MI355_MDM)       \
  } else if constexpr (NJ == 2 && A_T && B_NN) { /* 24 reads, 16 MFMAs */     \
    MI355_X4(MI355_MDD) MI355_X4(MI355_MDD) MI355_X4(MI355_MDD)               \
  } else if constexpr (NJ == 2 && A_T) {       /* 20 reads */                 \
    MI355_X4(MI355_MDD) MI355_X4(MI355_MDD) MI355_X4(MI355_MD)                \
  } else if constexpr (NJ == 2 && B_NN) {                                     \
    MI355_X4(MI355_MDD) MI355_X4(MI355_MDD)                                   \
  } else if constexpr (NJ == 2) {                                             \
    MI355_X4(MI355_MD) MI355_X4(MI355_MD) MI355_X4(MI355_MD)                  \
  } else if constexpr (B_NN) {                                                \
    MI355_X4(MI355_X4(MI355_MD)) MI355_X4(MI355_MD) MI355_X4(MI355_MDM)       \
  } else {                                                                    \
    MI355_X4(MI355_MDM) MI355_X4(MI355_MDM) MI355_X4(MI355_MDM) MI355_X4(MI355_MDM) \
  }                                                                           \
  __builtin_amdgcn_sched_group_barrier(0x008, 32, 0);                         \
  __builtin_amdgcn_sched_barrier(0);

  // Fragments are read one whole step ahead: while the MFMAs of step t run from one register
  // set, the LDS reads of step t+1 fill the other, so no MFMA of a step waits for LDS.  A panel
  // is therefore read during the step before its own and is free from the barrier that ends
  // that step.  Every step issues eight fills per lane: step t refills the B slot of step t
  // with step t+4; the A slot that held steps u, u+1 (u even) is refilled with steps u+6, u+7,
  // requests 0-3 in step u+1 and 4-7 in step u+2.  At the barrier that ends step t the panels of
  // step t+2 must have landed, all requested in step t-2 or earlier: only the 2 (4 + NJ) loads of
  // steps t-1 and t may still fly.
  const int nk = g.K / BK3;  // even: K % 64 == 0
#pragma unroll
  for (int i = 0; i < 8; ++i) request_a(i, 0, 0);
  if constexpr (B_PAIR) {
#pragma unroll
    for (int i = 0; i < 4; ++i) request_b_pair(i, 0, 0);
    if (nk > 2) {
#pragma unroll
      for (int i = 0; i < 8; ++i) request_a(i, 2, kASlot64);
#pragma unroll
      for (int i = 0; i < 4; ++i) request_b_pair(i, 2, kASlot64);
      if (nk > 4) {  // what the odd step before step 0 would have asked for: the first half of steps 4, 5
#pragma unroll
        for (int i = 0; i < 4; ++i) request_a(i, 4, 2 * kASlot64);
#pragma unroll
        for (int i = 0; i < 2; ++i) request_b_pair(i, 4, 2 * kASlot64);
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < NJ; ++i) request_b(i, 0);
#pragma unroll
    for (int i = 0; i < NJ; ++i) request_b(i, 1);
    if (nk > 2) {
#pragma unroll
      for (int i = 0; i < 8; ++i) request_a(i, 2, kASlot64);
#pragma unroll
      for (int i = 0; i < NJ; ++i) request_b(i, 2);
      if (nk > 4) {
#pragma unroll
        for (int i = 0; i < 4; ++i) request_a(i, 4, 2 * kASlot64);
      }
#pragma unroll
      for (int i = 0; i < NJ; ++i) request_b(i, 3);
    }
  }
  // steps 0 and 1 are in when only the 12 + 2 NJ loads behind them still fly (B_PAIR: the 12 of steps 2, 3 and the 6 of 4, 5)
  if (nk > 4 && NJ == 4) asm volatile("s_waitcnt vmcnt(20)" ::: "memory");
  else if (nk > 4 && B_PAIR) asm volatile("s_waitcnt vmcnt(18)" ::: "memory");
  else if (nk > 4) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
  else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  frag_t fa[2][2][4], fb[2][2][NJA];
  uint32_t cur = 0;  // A slot of steps t, t+1 (t even)
  io_step(0, cur, 0, fa[0], fb[0], false, 0, 0u, 0, false, 0);
  __syncthreads();  // every wave has its fragments of step 0: the B slot of step 0 may be refilled
  int t = 0;
#ifdef MI355_GEMM_TRACE
  // Diagnostic build only (-DMI355_GEMM_TRACE, libmi355_gemm_trace.so): shader-clock stamps
  // (s_memtime, read one step after they are issued, so no wait is added).  Lane 0 of every wave
  // leaves 16 uint64 in the caller's workspace at ((block * 4 + wave) * 16):
  //   [0..5]  sums over the steady-state loop of, for the even and the odd step of an iteration:
  //           ticks issuing the step's MFMAs / reads / fills, ticks in s_waitcnt for the fills,
  //           ticks from there to behind the barrier (the odd one includes the loop's back edge
  //           and ~170 ticks of this bookkeeping);
  //   [6] ticks in the loop   [7] loop iterations   [8], [9] longest single fill wait / barrier wait
  //   [10] stamp at loop entry   [11] HW_ID   [12] stamp at tile entry   [13] at loop exit
  //   [14] behind the remainder and drain steps   [15] when the tile's stores have completed.
  const uint64_t tr_begin = __builtin_readcyclecounter();
  uint64_t tp0 = tr_begin, tp1 = tr_begin, tp2 = tr_begin, tp3 = tr_begin, tp4 = tr_begin, tp5 = tr_begin;
  uint64_t tr_sum[6] = {0, 0, 0, 0, 0, 0};
  uint64_t tr_max[2] = {0, 0};
#define MI355_TR_STAMP(v) asm volatile("s_memtime %0" : "=s"(v)::"memory");
#define MI355_TR_C0 { tr_sum[0] += tp1 - tp0; tr_sum[1] += tp2 - tp1; tr_sum[2] += tp3 - tp2; \
    if (tp2 - tp1 > tr_max[0]) tr_max[0] = tp2 - tp1; if (tp3 - tp2 > tr_max[1]) tr_max[1] = tp3 - tp2; }
#define MI355_TR_C1 { tr_sum[3] += tp4 - tp3; tr_sum[4] += tp5 - tp4; tr_sum[5] += tp0 - tp5; }
#else
#define MI355_TR_STAMP(v)
#define MI355_TR_C0
#define MI355_TR_C1
#endif
  for (; t + 7 < nk; t += 2) {
    const uint32_t nxt = next_slot(cur);
    MI355_TR_C0 MI355_TR_STAMP(tp0)
    // even step t
    io_step(t + 1, cur, 1, fa[1], fb[1], true, t + 4, next_slot(nxt), 4, true, t + 4);
    mma_step(fa[0], fb[0]);
    MI355_W4_SCHEDULE
    MI355_TR_STAMP(tp1)
    if constexpr (NJ == 4) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
    MI355_TR_STAMP(tp2)
    __syncthreads();
    MI355_TR_C1 MI355_TR_STAMP(tp3)
    // odd step t+1
    io_step(t + 2, nxt, 0, fa[0], fb[0], true, t + 6, cur, 0, true, t + 5);
    mma_step(fa[1], fb[1]);
    MI355_W4_SCHEDULE
    MI355_TR_STAMP(tp4)
    if constexpr (NJ == 4) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
    MI355_TR_STAMP(tp5)
    __syncthreads();
    cur = nxt;
  }
#ifdef MI355_GEMM_TRACE
  {
    const uint64_t tr_end = __builtin_readcyclecounter();
    if (lane == 0 && g.ws != nullptr) {
      uint64_t* o = reinterpret_cast<uint64_t*>(g.ws) + ((int64_t)blockIdx.x * 4 + wave) * 16;
      for (int q = 0; q < 6; ++q) o[q] = tr_sum[q];
      o[6] = tr_end - tr_begin; o[7] = (uint64_t)(t / 2); o[8] = tr_max[0]; o[9] = tr_max[1]; o[10] = tr_begin;
      o[11] = __builtin_amdgcn_s_getreg((4 << 0) | (0 << 6) | (31 << 11));  // HW_REG_HW_ID (XCC / SE / CU of this wave)
      o[12] = tr_entry;
      o[13] = tr_end;
    }
  }
#endif
#undef MI355_TR_STAMP
#undef MI355_TR_C0
#undef MI355_TR_C1
  // Last steps: the requests thin out.  fills(s) = loads that step s issues; the barrier that
  // ends step s lets exactly those of steps s-1 and s fly, as in the steady state.
  auto fills = [nk](int s) {
    if constexpr (B_PAIR) return 6 * ((s & 1) ? s + 5 < nk : s + 4 < nk);
    else return (s & 1) ? NJ * (s + 4 < nk) + 4 * (s + 5 < nk) : (4 + NJ) * (s + 4 < nk);
  };
  auto wait_fills = [](int n) {
    switch (n) {
      case 16: asm volatile("s_waitcnt vmcnt(16)" ::: "memory"); break;
      case 14: asm volatile("s_waitcnt vmcnt(14)" ::: "memory"); break;
      case 12: asm volatile("s_waitcnt vmcnt(12)" ::: "memory"); break;
      case 10: asm volatile("s_waitcnt vmcnt(10)" ::: "memory"); break;
      case 8: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
      case 6: asm volatile("s_waitcnt vmcnt(6)" ::: "memory"); break;
      case 4: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
      case 2: asm volatile("s_waitcnt vmcnt(2)" ::: "memory"); break;
      default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    }
  };
  if (nk - t == 6) {
    // The last six steps of any K of 384 and more, written out: which of them still request is known here, so
    // they keep the steady state's order of MFMAs, reads and requests (in the loop below, whose requests sit
    // behind run-time conditions, the compiler reads all fragments first and issues the MFMAs in one block:
    // 1180 clocks a step against 775).  Step t asks for the second half of steps t+4, t+5; step t+1 for b of
    // step t+5 where b is fetched by the step; nothing after that.
    constexpr int kPerStep = 4 + NJ;                 // loads a steady-state step issues
    constexpr int kLateB = B_PAIR ? 0 : NJ;          // loads of step t+1
    const uint32_t s1 = next_slot(cur), s2 = next_slot(s1);
    io_step(t + 1, cur, 1, fa[1], fb[1], true, t + 4, s2, 4, true, t + 4);
    mma_step(fa[0], fb[0]);
    MI355_W4_SCHEDULE
    wait_fills(2 * kPerStep);
    __syncthreads();
    io_step(t + 2, s1, 0, fa[0], fb[0], false, 0, 0u, 0, !B_PAIR, t + 5);
    mma_step(fa[1], fb[1]);
    MI355_W4_SCHEDULE
    wait_fills(kPerStep + kLateB);
    __syncthreads();
    io_step(t + 3, s1, 1, fa[1], fb[1], false, 0, 0u, 0, false, 0);
    mma_step(fa[0], fb[0]);
    MI355_W4_SCHEDULE
    wait_fills(kLateB);
    __syncthreads();
    io_step(t + 4, s2, 0, fa[0], fb[0], false, 0, 0u, 0, false, 0);
    mma_step(fa[1], fb[1]);
    MI355_W4_SCHEDULE
    wait_fills(0);
    __syncthreads();
    io_step(t + 5, s2, 1, fa[1], fb[1], false, 0, 0u, 0, false, 0);
    mma_step(fa[0], fb[0]);
    MI355_W4_SCHEDULE
    __syncthreads();
    mma_step(fa[1], fb[1]);
    t = nk;
  }
  for (; t < nk; t += 2) {
    const uint32_t nxt = next_slot(cur);
    io_step(t + 1, cur, 1, fa[1], fb[1], t + 4 < nk, t + 4, next_slot(nxt), 4, t + 4 < nk, t + 4);
    mma_step(fa[0], fb[0]);
    wait_fills(fills(t - 1) + fills(t));
    __syncthreads();
    if (t + 2 < nk) io_step(t + 2, nxt, 0, fa[0], fb[0], t + 6 < nk, t + 6, cur, 0, t + 5 < nk, t + 5);
    mma_step(fa[1], fb[1]);
    wait_fills(fills(t) + fills(t + 1));
    __syncthreads();
    cur = nxt;
  }
#undef MI355_W4_SCHEDULE
#undef MI355_X4
#undef MI355_MDD
#undef MI355_MDM
#undef MI355_MD
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // (nothing is in flight: the last two steps issue no fills)
#ifdef MI355_GEMM_TRACE
  const uint64_t tr_drained = __builtin_readcyclecounter();
#endif

  store_tile_result<T, 4, 0>(g, acc, lds, wave, lane, bm + wm * 128, bn + wn * (NJA * 32));
  if constexpr (NJA == 4) store_tile_result<T, 4, 2>(g, acc, lds, wave, lane, bm + wm * 128, bn + wn * 128 + 64);
  if constexpr (NJA == 3) store_tile_result<T, 4, 2, 1>(g, acc, lds, wave, lane, bm + wm * 128, bn + wn * 96 + 64);
#ifdef MI355_GEMM_TRACE
  {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const uint64_t tr_stored = __builtin_readcyclecounter();
    if (lane == 0 && g.ws != nullptr) {
      uint64_t* o = reinterpret_cast<uint64_t*>(g.ws) + ((int64_t)blockIdx.x * 4 + wave) * 16;
      o[14] = tr_drained;
      o[15] = tr_stored;
    }
  }
#endif
}

template <typename T, bool B_NN, int NJ, bool A_T>
__global__ __launch_bounds__(256) void gemm_mfma_w4_kernel(GemmArgs g) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  if ((int)blockIdx.x >= g.tiles_m * g.tiles_n) return warm_operands<T, A_T, B_NN>(g, 0, g.K);
  int tm, tn;
  tile_coords<NJ == 2 ? 4 : 8>(g, tm, tn);
  // the fill requests take their bases in SGPRs: the tile origin is uniform, say so
  w4_tile<T, B_NN, NJ, A_T>(g, lds, __builtin_amdgcn_readfirstlane(tm * BM), __builtin_amdgcn_readfirstlane(tn * (NJ * 64)));
}

// The same tiles in two widths in one launch: blocks [0, tiles_m * tiles_n) are 256 x 256 tiles of the
// columns [0, 256 tiles_n); the blocks behind them are 256 x 192 tiles of the columns from there on
// (tiles_m * tail_n of them).  Workgroups are dispatched in block order, so the narrow tiles form
// the last round: a tile count that leaves the last round of 256-wide tiles partly empty (688 tiles
// on 256 CUs: 2.69 rounds, paid as 3) becomes two full rounds plus one round of cheaper tiles.
template <typename T, bool B_NN, bool A_T>
__global__ __launch_bounds__(256) void gemm_mfma_w4_mixed_kernel(GemmArgs g) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int wide = g.tiles_m * g.tiles_n;
  int tm, tn;
  if ((int)blockIdx.x < wide) {
    tile_coords(g.tiles_m, g.tiles_n, blockIdx.x, tm, tn);
    w4_tile<T, B_NN, 4, A_T, 4>(g, lds, __builtin_amdgcn_readfirstlane(tm * BM), __builtin_amdgcn_readfirstlane(tn * 256));
  } else {
    tile_coords(g.tiles_m, g.tail_n, blockIdx.x - wide, tm, tn);
    w4_tile<T, B_NN, 4, A_T, 3>(g, lds, __builtin_amdgcn_readfirstlane(tm * BM), __builtin_amdgcn_readfirstlane(g.tiles_n * 256 + tn * 192));
  }
}


// ---------------------------------------------------------------- MFMA kernel, 128x128 tiles
// For problems that do not fill the chip with 256x256 tiles.  Four waves (2x2), each a 64x64
// corner (2x2 MFMA blocks, 64 accumulators), 32-k steps, a ring of four 16 KB stages
// (A 128x32 + B 32x128) filled by global_load_lds_dwordx4 three steps ahead exactly as in
// gemm_mfma_dma_kernel; 64 KB of LDS, so two workgroups share a CU.  K % 32 == 0.
constexpr int kSPanel = SBM * BK3 * 2;            // 8 KB per operand per stage
constexpr int kSStage = 2 * kSPanel;              // 16 KB
constexpr int kSmallLds = kStages3 * kSStage;     // 64 KB
constexpr int kSmall2Lds = 5 * 2 * SBM * 64 * 2;  // 160 KB: five pairs of (A 128x64 + B 64x128)

template <typename T, bool B_NN, int SPLIT, bool A_T>
__global__ __launch_bounds__(256) void gemm_mfma_small_kernel(GemmArgs g) {
  constexpr int S = kStages3;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  using frag_t = typename Mfma<T>::frag;
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave >> 1, wn = wave & 1;
  int tm, tn;
  tile_coords(g, tm, tn);
  const int bm = tm * SBM, bn = tn * SBN;
  const int kbeg = SPLIT ? (int)blockIdx.y * g.ksplit : 0;
  const int kend = SPLIT ? (kbeg + g.ksplit < g.K ? kbeg + g.ksplit : g.K) : g.K;
  const T* A = static_cast<const T*>(g.a) + (A_T ? (int64_t)kbeg * g.lda : (int64_t)kbeg);
  const T* B = static_cast<const T*>(g.b) + (B_NN ? (int64_t)kbeg * g.ldb : (int64_t)kbeg);
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;

  // Region q = wave + 4 i (i < 2) of a panel is LDS bytes [q * 1024, q * 1024 + 1024).
  const T* a_src[2];
  const T* b_src[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int q = wave + 4 * i;
    if constexpr (A_T) {  // M-contiguous A panel (swz_n128): region q = k rows 4q .. 4q+3, 16 units per row
      const int k = 4 * q + (lane >> 4), pos = lane & 15;
      const int u = (((pos >> 2) ^ (k & 3)) << 2) | (pos & 3);
      int gm = bm + u * 8;
      gm = gm < g.M ? gm : 0;
      a_src[i] = A + (int64_t)k * g.lda + gm;
    } else {  // K-contiguous A panel: region q = rows 16q .. 16q+15, 4 chunks per row
      const int r = 16 * q + (lane >> 2), slot = lane & 3;
      const int c = slot ^ ((r >> 2) & 3);
      int gr = bm + r;
      gr = gr < g.M ? gr : g.M - 1;
      a_src[i] = A + (int64_t)gr * g.lda + c * 8;
    }
    if constexpr (!B_NN) {
      const int r = 16 * q + (lane >> 2), slot = lane & 3;
      const int c = slot ^ ((r >> 2) & 3);
      int gn = bn + r;
      gn = gn < g.N ? gn : g.N - 1;
      b_src[i] = B + (int64_t)gn * g.ldb + c * 8;
    } else {  // N-contiguous B panel: region q = k rows 4q .. 4q+3, 16 units per row
      const int k = 4 * q + (lane >> 4), pos = lane & 15;
      const int u = (((pos >> 2) ^ (k & 3)) << 2) | (pos & 3);
      int gn = bn + u * 8;
      gn = gn < g.N ? gn : 0;
      b_src[i] = B + (int64_t)k * g.ldb + gn;
    }
  }
  auto request_tile = [&](int t) {
    const uint32_t stage = lds_base + (uint32_t)(t % S) * kSStage;
    const int64_t k0 = (int64_t)t * BK3;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const uint32_t region = (uint32_t)(wave + 4 * i) * 1024u;
      lds_dma16(stage + region, a_src[i] + (A_T ? k0 * g.lda : k0));
      if constexpr (!B_NN) lds_dma16(stage + kSPanel + region, b_src[i] + k0);
      else lds_dma16(stage + kSPanel + region, b_src[i] + k0 * g.ldb);
    }
  };

  const int fr = lane & 31, fg = lane >> 5;
  const int tr_k = fg * 8 + ((lane & 15) >> 2);
  const int tr_n = (((lane >> 4) & 1) << 4) + ((lane & 3) << 2);
  auto read_frags = [&](int t, int ks, frag_t (&fa)[2], frag_t (&fb)[2]) {
    const unsigned char* pa = lds + (t % S) * kSStage;
    const unsigned char* pb = pa + kSPanel;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      if constexpr (A_T) {
        const int k = ks * 16 + tr_k;
        const int m = wm * 64 + i * 32 + tr_n;
        const s16x4 lo = lds_read_tr(pa + swz_n128(k, m >> 3) + ((m & 7) << 1));
        const s16x4 hi = lds_read_tr(pa + swz_n128(k + 4, m >> 3) + ((m & 7) << 1));
        fa[i] = __builtin_bit_cast(frag_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      } else {
        fa[i] = *reinterpret_cast<const frag_t*>(pa + swz_k32(wm * 64 + i * 32 + fr, ks * 2 + fg));
      }
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      if constexpr (!B_NN) {
        fb[j] = *reinterpret_cast<const frag_t*>(pb + swz_k32(wn * 64 + j * 32 + fr, ks * 2 + fg));
      } else {
        const int k = ks * 16 + tr_k;
        const int n = wn * 64 + j * 32 + tr_n;
        const s16x4 lo = lds_read_tr(pb + swz_n128(k, n >> 3) + ((n & 7) << 1));
        const s16x4 hi = lds_read_tr(pb + swz_n128(k + 4, n >> 3) + ((n & 7) << 1));
        fb[j] = __builtin_bit_cast(frag_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      }
    }
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  auto mma = [&](frag_t (&fa)[2], frag_t (&fb)[2]) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[i][j] = Mfma<T>::run(fb[j], fa[i], acc[i][j]);
  };

  // Fragments are read one whole step ahead: step `it` computes tile `it` from one register set
  // while the LDS reads of tile it+1 fill the other, so no MFMA waits for LDS and the slot of
  // tile `it`, read during step it-1, is free from the barrier that ends that step.  Step `it`
  // refills it with tile it+4, its four loads issued one at a time behind the LDS reads.  At the
  // barrier that ends step `it` tile it+2 must have landed: the eight loads of tiles it+3 and
  // it+4 may still fly.
  const int nk = (kend - kbeg) / BK3;
  for (int t = 0; t < S && t < nk; ++t) request_tile(t);
  // tiles 0 and 1 are in when only the later ones (at most two) still fly
  if (nk >= 4) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
  else if (nk == 3) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
  else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  frag_t fa[2][2][2], fb[2][2][2];  // [register set][16-k sub-step][block]
  auto request1 = [&](int f, int t) {  // request f (0..3) of tile t: A regions, then B regions
    const uint32_t stage = lds_base + (uint32_t)(t % S) * kSStage;
    const int64_t k0 = (int64_t)t * BK3;
    const int i = f & 1;
    const uint32_t region = (uint32_t)(wave + 4 * i) * 1024u;
    if (f < 2) lds_dma16(stage + region, a_src[i] + (A_T ? k0 * g.lda : k0));
    else if constexpr (!B_NN) lds_dma16(stage + kSPanel + region, b_src[i] + k0);
    else lds_dma16(stage + kSPanel + region, b_src[i] + k0 * g.ldb);
  };
  // LDS reads of tile t into one register set; `after(f)` runs behind fragment group f (0..3).
  auto read_tile = [&](int t, frag_t (&xa)[2][2], frag_t (&xb)[2][2], auto after) __attribute__((always_inline)) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      frag_t ta[2], tb[2];
      read_frags(t, ks, ta, tb);
#pragma unroll
      for (int i = 0; i < 2; ++i) { xa[ks][i] = ta[i]; xb[ks][i] = tb[i]; }
      after(2 * ks);
      after(2 * ks + 1);
    }
  };
  auto mma_tile = [&](frag_t (&xa)[2][2], frag_t (&xb)[2][2]) __attribute__((always_inline)) {
    mma(xa[0], xb[0]);
    mma(xa[1], xb[1]);
  };
  // Eight MFMAs per step; the LDS reads go behind the first four (two each, three with a row-major
  // B), and nothing moves across the end of the step.
#define MI355_SMALL_SCHEDULE                                                                               \
  __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x100, 2 + (B_NN ? 1 : 0) + (A_T ? 1 : 0), 0); \
  __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x100, 2 + (B_NN ? 1 : 0) + (A_T ? 1 : 0), 0); \
  __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x100, 2 + (B_NN ? 1 : 0) + (A_T ? 1 : 0), 0); \
  __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x100, 2 + (B_NN ? 1 : 0) + (A_T ? 1 : 0), 0); \
  __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);                                                       \
  __builtin_amdgcn_sched_barrier(0);
  read_tile(0, fa[0], fb[0], [](int) {});
  __syncthreads();  // every wave has its fragments of tile 0: its slot may be refilled
  int it = 0;
  for (; it + 5 < nk; it += 2) {
    read_tile(it + 1, fa[1], fb[1], [&](int f) { request1(f, it + 4); });
    mma_tile(fa[0], fb[0]);
    MI355_SMALL_SCHEDULE
    asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    __syncthreads();
    read_tile(it + 2, fa[0], fb[0], [&](int f) { request1(f, it + 5); });
    mma_tile(fa[1], fb[1]);
    MI355_SMALL_SCHEDULE
    asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    __syncthreads();
  }
  // Last steps: the requests stop at tile nk-1; each barrier lets the loads of its last two steps fly.
  auto fills = [nk](int q) { return q + 4 < nk ? 4 : 0; };
  auto wait_fills = [](int n) {
    if (n == 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    else if (n == 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  };
  // The last four or five steps of a K loop that reached the steady state, written out: which of them still
  // request (only the first of five) is known at compile time, so they keep the steady state's order of MFMAs
  // and reads; the loop below decides per step.
  auto last_tiles = [&](auto count) __attribute__((always_inline)) {
    constexpr int R = decltype(count)::value;
#pragma unroll
    for (int i = 0; i < R; ++i) {
      if (i + 1 < R) {
        if (i + 4 < R) read_tile(it + i + 1, fa[(i + 1) & 1], fb[(i + 1) & 1], [&](int f) { request1(f, it + i + 4); });
        else read_tile(it + i + 1, fa[(i + 1) & 1], fb[(i + 1) & 1], [](int) {});
      }
      mma_tile(fa[i & 1], fb[i & 1]);
      if (i + 1 < R) {
        MI355_SMALL_SCHEDULE
      }
      wait_fills(4 * ((i - 1 < R - 4) + (i < R - 4)));  // fills(q - 1) + fills(q), q = it + i
      __syncthreads();
    }
  };
  if (nk - it == 5) {
    last_tiles(std::integral_constant<int, 5>{});
    it = nk;
  } else if (nk - it == 4) {
    last_tiles(std::integral_constant<int, 4>{});
    it = nk;
  }
#undef MI355_SMALL_SCHEDULE
  for (; it < nk; it += 2) {
    if (it + 1 < nk) {
      const bool fill = it + 4 < nk;
      read_tile(it + 1, fa[1], fb[1], [&](int f) { if (fill) request1(f, it + 4); });
    }
    mma_tile(fa[0], fb[0]);
    wait_fills(fills(it - 1) + fills(it));
    __syncthreads();
    if (it + 1 < nk) {
      if (it + 2 < nk) {
        const bool fill = it + 5 < nk;
        read_tile(it + 2, fa[0], fb[0], [&](int f) { if (fill) request1(f, it + 5); });
      }
      mma_tile(fa[1], fb[1]);
      wait_fills(fills(it) + fills(it + 1));
      __syncthreads();
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // (nothing is in flight: the last steps issue no fills)

  if constexpr (SPLIT == 1) {
    store_partial_tile<2>(g, acc, lane, bm + wm * 64, bn + wn * 64);
  } else {
    if constexpr (SPLIT == 2) {  // the parts meet inside this launch: the last one sums and stores
      if (blockIdx.y + 1 < gridDim.y) return insplit_leave(g, acc, tid, wave, lane);
      insplit_sum(g, acc, lds, tid, wave, lane);
    }
    store_tile_result<T, 2>(g, acc, lds, wave, lane, bm + wm * 64, bn + wn * 64);
  }
}

// The 128x128 tile for launches with at most one workgroup per CU: nothing else hides a
// workgroup's barrier, LDS and fill latencies there, so it owns the whole 160 KB of LDS (a ring of
// five 64-k pairs, every request a whole 128-byte line), works in 64-k steps (16 MFMAs per wave
// between barriers instead of 8) and reads its fragments a step ahead.
template <typename T, bool B_NN, int SPLIT, bool A_T>
__global__ __launch_bounds__(256) void gemm_mfma_small2_kernel(GemmArgs g) {
  constexpr int S = 5;  // ring depth in 64-k pairs
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  using frag_t = typename Mfma<T>::frag;
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave >> 1, wn = wave & 1;
  int tm, tn;
  tile_coords(g, tm, tn);
  const int bm = tm * SBM, bn = tn * SBN;
  const int kbeg = SPLIT ? (int)blockIdx.y * g.ksplit : 0;
  const int kend = SPLIT ? (kbeg + g.ksplit < g.K ? kbeg + g.ksplit : g.K) : g.K;
  if ((int)blockIdx.x >= g.tiles_m * g.tiles_n) return warm_operands<T, A_T, B_NN>(g, kbeg, kend);
  const T* A = static_cast<const T*>(g.a) + (A_T ? (int64_t)kbeg * g.lda : (int64_t)kbeg);
  const T* B = static_cast<const T*>(g.b) + (B_NN ? (int64_t)kbeg * g.ldb : (int64_t)kbeg);
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;

  // A pair slot (32 KB) holds 64 k of A (128 rows of 128 B, swz_k64) and of B (the same for a
  // K-contiguous B; 64 k-rows of 256 B, swz_n128, for a row-major one), so every request fetches
  // whole 128-byte lines.  Region q = wave + 4 i (i < 4) of a panel is its bytes [1024 q, 1024 q + 1024).
  constexpr int kPairPanel = SBM * 64 * 2;  // 16 KB
  constexpr int kPairSlot = 2 * kPairPanel;
  const T* a_src[4];
  const T* b_src[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int q = wave + 4 * i;
    const int r = 8 * q + (lane >> 3), slot = lane & 7;
    const int c = slot ^ (((r >> 1) & 1) | ((r >> 2) & 6));
    if constexpr (A_T) {  // M-contiguous A: 64 k-rows of 256 B (swz_n128), region q = k rows 4q .. 4q+3
      const int k = 4 * q + (lane >> 4), pos = lane & 15;
      const int u = (((pos >> 2) ^ (k & 3)) << 2) | (pos & 3);
      int gm = bm + u * 8;
      gm = gm < g.M ? gm : 0;
      a_src[i] = A + (int64_t)k * g.lda + gm;
    } else {
      int gr = bm + r;
      gr = gr < g.M ? gr : g.M - 1;
      a_src[i] = A + (int64_t)gr * g.lda + c * 8;
    }
    if constexpr (!B_NN) {
      int gn = bn + r;
      gn = gn < g.N ? gn : g.N - 1;
      b_src[i] = B + (int64_t)gn * g.ldb + c * 8;
    } else {  // region q = k rows 4q .. 4q+3, 16 units per row
      const int k = 4 * q + (lane >> 4), pos = lane & 15;
      const int u = (((pos >> 2) ^ (k & 3)) << 2) | (pos & 3);
      int gn = bn + u * 8;
      gn = gn < g.N ? gn : 0;
      b_src[i] = B + (int64_t)k * g.ldb + gn;
    }
  }
  // Fill request f (0..7) of pair q: the four regions of A, then the four of B.
  auto request = [&](int f, int q) {
    const uint32_t slot = lds_base + (uint32_t)(q % S) * kPairSlot;
    const int64_t k0 = (int64_t)q * 64;
    const int i = f & 3;
    const uint32_t region = (uint32_t)(wave + 4 * i) * 1024u;
    if (f < 4) lds_dma16(slot + region, a_src[i] + (A_T ? k0 * g.lda : k0));
    else if constexpr (!B_NN) lds_dma16(slot + kPairPanel + region, b_src[i] + k0);
    else lds_dma16(slot + kPairPanel + region, b_src[i] + k0 * g.ldb);
  };
  auto request_pair = [&](int q) {
#pragma unroll
    for (int f = 0; f < 8; ++f) request(f, q);
  };

  const int fr = lane & 31, fg = lane >> 5;
  const int tr_k = fg * 8 + ((lane & 15) >> 2);
  const int tr_n = (((lane >> 4) & 1) << 4) + ((lane & 3) << 2);
  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  // One step = one pair of 32-k tiles = 16 MFMAs per wave.  Fragments are read one whole step
  // ahead: step p computes pair p from one register set while the LDS reads of pair p+1 fill the
  // other, so no MFMA waits for LDS; pair p is therefore read during step p-1 and its two slots
  // are free from the barrier that ends that step.  Step p requests pair p+5 into them, its
  // eight loads issued one at a time behind the LDS reads (a burst behind the barrier stalls the
  // whole workgroup on its slowest wave).  At the barrier that ends step p the pairs up to p+2
  // must have landed: the 24 loads of steps p-2 .. p may still fly.  With one workgroup per CU
  // the kernel is bound by the latency of these fills; four pairs (128 KB) in flight are what the
  // LDS of a CU can hold.  K % 64 == 0.
  const int np = (kend - kbeg) / (2 * BK3);
  for (int q = 0; q < S && q < np; ++q) request_pair(q);
  // pairs 0 and 1 are in when only the later ones (at most three) still fly
  if (np >= 5) asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
  else if (np == 4) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
  else if (np == 3) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
  else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  frag_t fa[2][4][2], fb[2][4][2];  // [register set][tile of the pair * 2 + 16-k sub-step][block]
  // LDS reads of pair q into one register set; `after(f)` runs behind fragment group f (0..7).
  auto read_pair = [&](int q, frag_t (&xa)[4][2], frag_t (&xb)[4][2], auto after) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {  // 16-k sub-step u of the pair: chunks 2u, 2u+1 of the 128-byte rows
      const unsigned char* pa = lds + (q % S) * kPairSlot;
      const unsigned char* pb = pa + kPairPanel;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        if constexpr (A_T) {
          const int k = u * 16 + tr_k;
          const int m = wm * 64 + i * 32 + tr_n;
          const s16x4 lo = lds_read_tr(pa + swz_n128(k, m >> 3) + ((m & 7) << 1));
          const s16x4 hi = lds_read_tr(pa + swz_n128(k + 4, m >> 3) + ((m & 7) << 1));
          xa[u][i] = __builtin_bit_cast(frag_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        } else {
          xa[u][i] = *reinterpret_cast<const frag_t*>(pa + swz_k64(wm * 64 + i * 32 + fr, u * 2 + fg));
        }
      }
      after(2 * u);
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        if constexpr (!B_NN) {
          xb[u][j] = *reinterpret_cast<const frag_t*>(pb + swz_k64(wn * 64 + j * 32 + fr, u * 2 + fg));
        } else {
          const int k = u * 16 + tr_k;
          const int n = wn * 64 + j * 32 + tr_n;
          const s16x4 lo = lds_read_tr(pb + swz_n128(k, n >> 3) + ((n & 7) << 1));
          const s16x4 hi = lds_read_tr(pb + swz_n128(k + 4, n >> 3) + ((n & 7) << 1));
          xb[u][j] = __builtin_bit_cast(frag_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        }
      }
      after(2 * u + 1);
    }
  };
  auto mma_pair = [&](frag_t (&xa)[4][2], frag_t (&xb)[4][2]) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = Mfma<T>::run(xb[u][j], xa[u][i], acc[i][j]);
  };
  // The LDS reads go behind the first eight MFMAs of a step (two each, three with a row-major
  // B), the other eight MFMAs cover the latency of the last read, and nothing moves across the
  // end of the step.
#define MI355_MDD                                                                             \
  __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x100, 2 + (B_NN ? 1 : 0) + (A_T ? 1 : 0), 0);
#define MI355_X4(X) X X X X
#define MI355_PAIR_SCHEDULE                                                   \
  MI355_X4(MI355_MDD) MI355_X4(MI355_MDD)                                     \
  __builtin_amdgcn_sched_group_barrier(0x008, 16, 0);                         \
  __builtin_amdgcn_sched_barrier(0);

  read_pair(0, fa[0], fb[0], [](int) {});
  __syncthreads();  // every wave has its fragments of pair 0: its slots may be refilled
  int p = 0;
  for (; p + 6 < np; p += 2) {
    read_pair(p + 1, fa[1], fb[1], [&](int f) { request(f, p + 5); });
    mma_pair(fa[0], fb[0]);
    MI355_PAIR_SCHEDULE
    asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
    __syncthreads();
    read_pair(p + 2, fa[0], fb[0], [&](int f) { request(f, p + 6); });
    mma_pair(fa[1], fb[1]);
    MI355_PAIR_SCHEDULE
    asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
    __syncthreads();
  }
  // Last steps: the requests stop at pair np-1; each barrier lets the loads of its last three steps fly.
  auto fills = [np](int q) { return q + 5 < np ? 8 : 0; };
  auto wait_fills = [](int n) {
    if (n == 24) asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
    else if (n == 16) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
    else if (n == 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  };
  // The last five or six pairs of a K loop that reached the steady state, written out: which of them still
  // request (only the first of six) is known at compile time, so they keep the steady state's order of MFMAs and
  // reads; the loop below decides per step and leaves the order to the compiler.
  auto last_pairs = [&](auto count) __attribute__((always_inline)) {
    constexpr int R = decltype(count)::value;
#pragma unroll
    for (int i = 0; i < R; ++i) {
      if (i + 1 < R) {
        if (i + 5 < R) read_pair(p + i + 1, fa[(i + 1) & 1], fb[(i + 1) & 1], [&](int f) { request(f, p + i + 5); });
        else read_pair(p + i + 1, fa[(i + 1) & 1], fb[(i + 1) & 1], [](int) {});
      }
      mma_pair(fa[i & 1], fb[i & 1]);
      if (i + 1 < R) {
        MI355_PAIR_SCHEDULE
      }
      wait_fills(8 * ((i - 2 < R - 5) + (i - 1 < R - 5) + (i < R - 5)));  // fills(q - 2) + fills(q - 1) + fills(q), q = p + i
      __syncthreads();
    }
  };
  if (np - p == 6) {
    last_pairs(std::integral_constant<int, 6>{});
    p = np;
  } else if (np - p == 5) {
    last_pairs(std::integral_constant<int, 5>{});
    p = np;
  }
#undef MI355_PAIR_SCHEDULE
#undef MI355_X4
#undef MI355_MDD
  for (; p < np; p += 2) {
    if (p + 1 < np) {
      const bool fill = p + 5 < np;
      read_pair(p + 1, fa[1], fb[1], [&](int f) { if (fill) request(f, p + 5); });
    }
    mma_pair(fa[0], fb[0]);
    wait_fills(fills(p - 2) + fills(p - 1) + fills(p));
    __syncthreads();
    if (p + 1 < np) {
      if (p + 2 < np) {
        const bool fill = p + 6 < np;
        read_pair(p + 2, fa[0], fb[0], [&](int f) { if (fill) request(f, p + 6); });
      }
      mma_pair(fa[1], fb[1]);
      wait_fills(fills(p - 1) + fills(p) + fills(p + 1));
      __syncthreads();
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // (nothing is in flight: the last steps issue no fills)

  if constexpr (SPLIT == 1) {
    store_partial_tile<2>(g, acc, lane, bm + wm * 64, bn + wn * 64);
  } else {
    if constexpr (SPLIT == 2) {  // the parts meet inside this launch: the last one sums and stores
      if (blockIdx.y + 1 < gridDim.y) return insplit_leave(g, acc, tid, wave, lane);
      insplit_sum(g, acc, lds, tid, wave, lane);
    }
    store_tile_result<T, 2>(g, acc, lds, wave, lane, bm + wm * 64, bn + wn * 64);
  }
}

// The deep-ring 128x128 kernel with the fills taken out of the computing waves' instruction streams: eight
// waves, two per SIMD.  Waves 0 - 3 compute as in gemm_mfma_small2_kernel (fragments of pair p + 1 read during
// step p, sixteen MFMAs per step) and never touch global memory in the K loop; waves 4 - 7 ("loaders") issue
// every fill request - wave 4 + w the regions that wave w fills in the four-wave form - wait for them
// (s_waitcnt vmcnt) and meet the others at the one barrier per step.  Why: a CU takes fills in at about 80 GB/s,
// which is what a 128x128 tile asks for (32 KB per 64-k step of 0.4 us); at that rate the memory pipeline
// pushes back, a wave stalls at its next request, and on a SIMD with a single wave the MFMAs behind the
// request wait with it - fills and MFMAs took turns instead of overlapping (measured on [2048,4096]x
// [2048,4096]^T, ns per k: 12.5 as built, 6.4 without the fills, 6.3 with the fills alone).  A loader stalls
// alone.  The loaders end after the last step's barrier; s_barrier counts the waves that are left, so the
// epilogue's barriers (the in-launch split's exchange) are met by the four computing waves only.
template <typename T, bool B_NN, int SPLIT, bool A_T>
__global__ __launch_bounds__(512) void gemm_mfma_small3_kernel(GemmArgs g) {
  constexpr int S = 5;  // ring depth in 64-k pairs
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  using frag_t = typename Mfma<T>::frag;
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave8 = __builtin_amdgcn_readfirstlane(tid / kWave);
  const bool loader = wave8 >= 4;
  const int wave = wave8 & 3;
  const int wm = wave >> 1, wn = wave & 1;
  int tm, tn;
  tile_coords(g, tm, tn);
  const int bm = tm * SBM, bn = tn * SBN;
  const int kbeg = SPLIT ? (int)blockIdx.y * g.ksplit : 0;
  const int kend = SPLIT ? (kbeg + g.ksplit < g.K ? kbeg + g.ksplit : g.K) : g.K;
  const int np = (kend - kbeg) / (2 * BK3);
  constexpr int kPairPanel = SBM * 64 * 2;  // 16 KB
  constexpr int kPairSlot = 2 * kPairPanel;
  if ((int)blockIdx.x >= g.tiles_m * g.tiles_n) return warm_operands<T, A_T, B_NN>(g, kbeg, kend);

  if (loader) {
    const T* A = static_cast<const T*>(g.a) + (A_T ? (int64_t)kbeg * g.lda : (int64_t)kbeg);
    const T* B = static_cast<const T*>(g.b) + (B_NN ? (int64_t)kbeg * g.ldb : (int64_t)kbeg);
    const uint32_t lds_base = (uint32_t)(uintptr_t)lds;
    // Region q = wave + 4 i (i < 4) of a panel is its bytes [1024 q, 1024 q + 1024); layouts as in the
    // four-wave form (swz_k64 rows for a K-contiguous operand, swz_n128 k-rows otherwise).
    const T* a_src[4];
    const T* b_src[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int q = wave + 4 * i;
      const int r = 8 * q + (lane >> 3), slot = lane & 7;
      const int c = slot ^ (((r >> 1) & 1) | ((r >> 2) & 6));
      if constexpr (A_T) {
        const int k = 4 * q + (lane >> 4), pos = lane & 15;
        const int u = (((pos >> 2) ^ (k & 3)) << 2) | (pos & 3);
        int gm = bm + u * 8;
        gm = gm < g.M ? gm : 0;
        a_src[i] = A + (int64_t)k * g.lda + gm;
      } else {
        int gr = bm + r;
        gr = gr < g.M ? gr : g.M - 1;
        a_src[i] = A + (int64_t)gr * g.lda + c * 8;
      }
      if constexpr (!B_NN) {
        int gn = bn + r;
        gn = gn < g.N ? gn : g.N - 1;
        b_src[i] = B + (int64_t)gn * g.ldb + c * 8;
      } else {
        const int k = 4 * q + (lane >> 4), pos = lane & 15;
        const int u = (((pos >> 2) ^ (k & 3)) << 2) | (pos & 3);
        int gn = bn + u * 8;
        gn = gn < g.N ? gn : 0;
        b_src[i] = B + (int64_t)k * g.ldb + gn;
      }
    }
    auto request_pair = [&](int q, uint32_t slot) __attribute__((always_inline)) {
      const int64_t k0 = (int64_t)q * 64;
#pragma unroll
      for (int i = 0; i < 4; ++i) lds_dma16(slot + (uint32_t)(wave + 4 * i) * 1024u, a_src[i] + (A_T ? k0 * g.lda : k0));
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if constexpr (!B_NN) lds_dma16(slot + kPairPanel + (uint32_t)(wave + 4 * i) * 1024u, b_src[i] + k0);
        else lds_dma16(slot + kPairPanel + (uint32_t)(wave + 4 * i) * 1024u, b_src[i] + k0 * g.ldb);
      }
    };
    // at most `n` of this wave's requests still in flight (n a multiple of 8: whole pairs)
    auto wait_fills = [](int n) {
      if (n >= 24) asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
      else if (n == 16) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
      else if (n == 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    };
    uint32_t slot = lds_base;
    for (int q = 0; q < S && q < np; ++q) request_pair(q, lds_base + (uint32_t)q * kPairSlot);
    wait_fills(8 * ((np < S ? np : S) - 2 > 0 ? (np < S ? np : S) - 2 : 0));  // pairs 0 and 1 are in
    __syncthreads();
    __syncthreads();  // the computing waves hold pair 0: its slot may be refilled
    // Step p: pair p + 5 goes into the slot pair p left; when the step ends the pairs up to p + 2 are in (the
    // requests of pairs p + 3 .. p + 5, those that exist, may still fly).
    for (int p = 0; p < np; ++p) {
      if (p + S < np) request_pair(p + S, slot);
      slot = slot + kPairSlot == lds_base + S * kPairSlot ? lds_base : slot + kPairSlot;
      const int ahead = np - 1 - (p + 2);  // pairs behind p + 2 that have been requested
      wait_fills(8 * (ahead < 0 ? 0 : ahead > 3 ? 3 : ahead));
      __syncthreads();
    }
    return;
  }

  const int fr = lane & 31, fg = lane >> 5;
  const int tr_k = fg * 8 + ((lane & 15) >> 2);
  const int tr_n = (((lane >> 4) & 1) << 4) + ((lane & 3) << 2);
  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  frag_t fa[2][4][2], fb[2][4][2];  // [register set][tile of the pair * 2 + 16-k sub-step][block]
  auto read_pair = [&](int slot_index, frag_t (&xa)[4][2], frag_t (&xb)[4][2]) __attribute__((always_inline)) {
    const unsigned char* pa = lds + slot_index * kPairSlot;
    const unsigned char* pb = pa + kPairPanel;
#pragma unroll
    for (int u = 0; u < 4; ++u) {  // 16-k sub-step u of the pair: chunks 2u, 2u+1 of the 128-byte rows
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        if constexpr (A_T) {
          const int k = u * 16 + tr_k;
          const int m = wm * 64 + i * 32 + tr_n;
          const s16x4 lo = lds_read_tr(pa + swz_n128(k, m >> 3) + ((m & 7) << 1));
          const s16x4 hi = lds_read_tr(pa + swz_n128(k + 4, m >> 3) + ((m & 7) << 1));
          xa[u][i] = __builtin_bit_cast(frag_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        } else {
          xa[u][i] = *reinterpret_cast<const frag_t*>(pa + swz_k64(wm * 64 + i * 32 + fr, u * 2 + fg));
        }
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        if constexpr (!B_NN) {
          xb[u][j] = *reinterpret_cast<const frag_t*>(pb + swz_k64(wn * 64 + j * 32 + fr, u * 2 + fg));
        } else {
          const int k = u * 16 + tr_k;
          const int n = wn * 64 + j * 32 + tr_n;
          const s16x4 lo = lds_read_tr(pb + swz_n128(k, n >> 3) + ((n & 7) << 1));
          const s16x4 hi = lds_read_tr(pb + swz_n128(k + 4, n >> 3) + ((n & 7) << 1));
          xb[u][j] = __builtin_bit_cast(frag_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        }
      }
    }
  };
  auto mma_pair = [&](frag_t (&xa)[4][2], frag_t (&xb)[4][2]) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = Mfma<T>::run(xb[u][j], xa[u][i], acc[i][j]);
  };
  // The LDS reads go behind the first eight MFMAs of a step (two each, three with a row-major B), the other
  // eight MFMAs cover the latency of the last read, and nothing moves across the end of the step.
#define MI355_MDD                                                                             \
  __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x100, 2 + (B_NN ? 1 : 0) + (A_T ? 1 : 0), 0);
#define MI355_X4(X) X X X X
#define MI355_PAIR_SCHEDULE                                                   \
  MI355_X4(MI355_MDD) MI355_X4(MI355_MDD)                                     \
  __builtin_amdgcn_sched_group_barrier(0x008, 16, 0);                         \
  __builtin_amdgcn_sched_barrier(0);

  __syncthreads();  // pairs 0 and 1 are in
  read_pair(0, fa[0], fb[0]);
  __syncthreads();  // every wave has its fragments of pair 0
  int p = 0, rs = 1;  // rs: the ring slot of pair p + 1
  auto next_slot = [](int v) { return v + 1 == S ? 0 : v + 1; };
  for (; p + 2 < np; p += 2) {
    read_pair(rs, fa[1], fb[1]);
    mma_pair(fa[0], fb[0]);
    MI355_PAIR_SCHEDULE
    __syncthreads();
    rs = next_slot(rs);
    read_pair(rs, fa[0], fb[0]);
    mma_pair(fa[1], fb[1]);
    MI355_PAIR_SCHEDULE
    __syncthreads();
    rs = next_slot(rs);
  }
#undef MI355_PAIR_SCHEDULE
#undef MI355_X4
#undef MI355_MDD
  for (; p < np; p += 2) {  // the last one or two steps
    if (p + 1 < np) read_pair(rs, fa[1], fb[1]);
    mma_pair(fa[0], fb[0]);
    __syncthreads();
    if (p + 1 < np) {
      mma_pair(fa[1], fb[1]);
      __syncthreads();
    }
  }

  if constexpr (SPLIT == 1) {
    store_partial_tile<2>(g, acc, lane, bm + wm * 64, bn + wn * 64);
  } else {
    if constexpr (SPLIT == 2) {  // the parts meet inside this launch: the last one sums and stores
      if (blockIdx.y + 1 < gridDim.y) return insplit_leave(g, acc, tid, wave, lane);
      insplit_sum(g, acc, lds, tid, wave, lane);
    }
    store_tile_result<T, 2>(g, acc, lds, wave, lane, bm + wm * 64, bn + wn * 64);
  }
}

// ---------------------------------------------------------------- MFMA kernel, 64x64 tiles
// bf16 / f16 products whose 128x128 tiles would leave most CUs without work (a 197-token ViT
// layer against a 768-wide weight: 12 tiles; 1024^3: 64) and whose K loop is too short to split:
// 64x64 tiles, four waves (2x2) of one 32x32 MFMA block each, 64-k stages (A 64x64 + B 64x64 =
// 16 KB, whole 128-byte lines for both operands) in a ring of S stages filled S-1 stages ahead by
// global_load_lds_dwordx4 (four requests per wave and stage, scalar base + 32-bit lane offset).
// One barrier per stage; the per-stage work is four MFMAs per wave, so the kernel lives on how
// many stages it keeps in flight: S = 8 (128 KB) when a CU gets one workgroup, else S = 4 (two
// per CU).  K % 64 == 0.  A K-contiguous; B K-contiguous (swz_k64 rows) or N-contiguous (128-byte
// k-rows, transposed by the LDS read).
constexpr int TBM = 64, TBN = 64;
constexpr int kTPanel = TBM * 64 * 2;  // 8 KB per operand per stage
constexpr int kTStage = 2 * kTPanel;   // 16 KB
// N-contiguous 64-wide panel: 128 B per k row, the two 64-byte halves swapped on k rows 2, 3 mod 4
// so that the four k rows of a transposing read fall into four different 64-byte bank groups.
__device__ __forceinline__ int swz_n64(int k, int u) {
  return k * 128 + ((((u >> 2) ^ ((k >> 1) & 1))) << 6) + ((u & 3) << 4);
}

// SPLIT: blockIdx.y owns the k range [blockIdx.y * ksplit, + ksplit) (whole 64-k stages) and leaves its raw fp32
// tile in plane blockIdx.y of the workspace, as the 128x128 kernels do; gemm_splitk_finish_kernel sums the planes.
template <typename T, bool B_NN, int S, int SPLIT = 0>
__global__ __launch_bounds__(256) void gemm_mfma_t64_kernel(GemmArgs g) {
  static_assert(S == 4 || S == 8, "ring of four or eight stages");
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  using frag_t = typename Mfma<T>::frag;
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave >> 1, wn = wave & 1;
  int tm, tn;
  tile_coords(g, tm, tn);
  const int bm = tm * TBM, bn = tn * TBN;
  const int kbeg = SPLIT ? (int)blockIdx.y * g.ksplit : 0;
  const int kend = SPLIT ? (kbeg + g.ksplit < g.K ? kbeg + g.ksplit : g.K) : g.K;
  if ((int)blockIdx.x >= g.tiles_m * g.tiles_n) return warm_operands<T, false, B_NN>(g, kbeg, kend);
  const T* a_base = static_cast<const T*>(g.a) + (int64_t)bm * g.lda + kbeg;
  const T* b_base = static_cast<const T*>(g.b) + (B_NN ? (int64_t)kbeg * g.ldb : (int64_t)bn * g.ldb + kbeg);
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;

  // Region q = wave + 4 i (i < 2) of a panel is LDS bytes [q * 1024, q * 1024 + 1024): eight rows of 128 B.
  uint32_t a_off[2], b_off[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int q = wave + 4 * i;
    const int r = 8 * q + (lane >> 3), slot = lane & 7;
    {
      const int c = slot ^ (((r >> 1) & 1) | ((r >> 2) & 6));
      const int lr = bm + r < g.M ? r : g.M - 1 - bm;  // rows past M re-read the last row
      a_off[i] = ((uint32_t)lr * (uint32_t)g.lda + (uint32_t)c * 8u) * 2u;
    }
    if constexpr (!B_NN) {
      const int c = slot ^ (((r >> 1) & 1) | ((r >> 2) & 6));
      const int ln = bn + r < g.N ? r : g.N - 1 - bn;
      b_off[i] = ((uint32_t)ln * (uint32_t)g.ldb + (uint32_t)c * 8u) * 2u;
    } else {  // k row r of the stage, LDS position `slot` holds unit u
      const int u = (((slot >> 2) ^ ((r >> 1) & 1)) << 2) | (slot & 3);
      int gn = bn + u * 8;
      gn = gn < g.N ? gn : 0;
      b_off[i] = ((uint32_t)r * (uint32_t)g.ldb + (uint32_t)gn) * 2u;
    }
  }
  auto request_stage = [&](int t) {
    const uint32_t stage = lds_base + (uint32_t)(t % S) * kTStage;
    const T* pa = a_base + (int64_t)t * 64;
    const T* pb = b_base + (B_NN ? (int64_t)t * 64 * g.ldb : (int64_t)t * 64);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const uint32_t region = (uint32_t)(wave + 4 * i) * 1024u;
      lds_dma16s(stage + region, a_off[i], pa);
      lds_dma16s(stage + kTPanel + region, b_off[i], pb);
    }
  };
  auto wait_younger = [](int stages) {  // stages requested behind the one about to be read: 4 loads each
    switch (stages) {
      case 0: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
      case 1: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
      case 2: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
      case 3: asm volatile("s_waitcnt vmcnt(12)" ::: "memory"); break;
      case 4: asm volatile("s_waitcnt vmcnt(16)" ::: "memory"); break;
      case 5: asm volatile("s_waitcnt vmcnt(20)" ::: "memory"); break;
      case 6: asm volatile("s_waitcnt vmcnt(24)" ::: "memory"); break;
      default: asm volatile("s_waitcnt vmcnt(28)" ::: "memory"); break;  // seven: the whole ring behind stage 0
    }
  };

  const int fr = lane & 31, fg = lane >> 5;
  const int tr_k = fg * 8 + ((lane & 15) >> 2);
  const int tr_n = (((lane >> 4) & 1) << 4) + ((lane & 3) << 2);
  // Two accumulators (even / odd 16-k sub-steps) halve the chain of dependent MFMAs, the only
  // arithmetic of a stage; they are added once at the end.
  f32x16 acc[1][1], acc_odd;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[0][0][e] = acc_odd[e] = 0.f;

  const int nk = (kend - kbeg) / 64;
  // Fragments are read one stage ahead: step t computes stage t from one register set while the LDS reads of
  // stage t + 1 fill the other, so the four MFMAs of a step - all its arithmetic - wait for nothing, and the slot
  // of stage t, read during step t - 1, takes the request for stage t + S behind the barrier of step t (the ring
  // is S stages deep in flight).  Two steps per iteration, one per register set.
  auto read_frags = [&](int t, frag_t (&fa)[4], frag_t (&fb)[4]) __attribute__((always_inline)) {
    const unsigned char* pa = lds + (t % S) * kTStage;
    const unsigned char* pb = pa + kTPanel;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      fa[ks] = *reinterpret_cast<const frag_t*>(pa + swz_k64(wm * 32 + fr, ks * 2 + fg));
      if constexpr (!B_NN) {
        fb[ks] = *reinterpret_cast<const frag_t*>(pb + swz_k64(wn * 32 + fr, ks * 2 + fg));
      } else {
        const int k = ks * 16 + tr_k;
        const int n = wn * 32 + tr_n;
        const s16x4 lo = lds_read_tr(pb + swz_n64(k, n >> 3) + ((n & 7) << 1));
        const s16x4 hi = lds_read_tr(pb + swz_n64(k + 4, n >> 3) + ((n & 7) << 1));
        fb[ks] = __builtin_bit_cast(frag_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      }
    }
  };
  auto mma_stage = [&](frag_t (&fa)[4], frag_t (&fb)[4]) __attribute__((always_inline)) {
    acc[0][0] = Mfma<T>::run(fb[0], fa[0], acc[0][0]);
    acc_odd = Mfma<T>::run(fb[1], fa[1], acc_odd);
    acc[0][0] = Mfma<T>::run(fb[2], fa[2], acc[0][0]);
    acc_odd = Mfma<T>::run(fb[3], fa[3], acc_odd);
  };
  // One step: stage `t` from `cur`; stage t + 1 (when there is one) lands, is read into `nxt`, and stage t + S is
  // requested into the slot stage t leaves.  Requests so far reach stage min(t + S - 1, nk - 1).
  auto step = [&](int t, frag_t (&ca)[4], frag_t (&cb)[4], frag_t (&na)[4], frag_t (&nb)[4]) __attribute__((always_inline)) {
    const bool more = t + 1 < nk;
    if (more) wait_younger((t + S - 1 < nk - 1 ? t + S - 1 : nk - 1) - (t + 1));
    __syncthreads();  // stage t + 1 has landed for every wave, and every wave has read stage t
    if (more) read_frags(t + 1, na, nb);
    if (t + S < nk) request_stage(t + S);
    mma_stage(ca, cb);
  };
  for (int t = 0; t < S && t < nk; ++t) request_stage(t);
  wait_younger((S < nk ? S : nk) - 1);
  __syncthreads();
  frag_t fa[2][4], fb[2][4];
  read_frags(0, fa[0], fb[0]);
  int t = 0;
  // Steady state without a branch (with branches around them the accumulators travel between their registers and
  // the VGPRs in every step): while both steps of an iteration still request a stage, S - 2 stages stay in flight
  // behind the one that is waited for.
  for (; t + S + 1 < nk; t += 2) {
    if constexpr (S == 8) asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    __syncthreads();
    read_frags(t + 1, fa[1], fb[1]);
    request_stage(t + S);
    mma_stage(fa[0], fb[0]);
    if constexpr (S == 8) asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    __syncthreads();
    read_frags(t + 2, fa[0], fb[0]);
    request_stage(t + 1 + S);
    mma_stage(fa[1], fb[1]);
  }
  // The last S or S + 1 steps of a K loop that reached the steady state, written out: what each of them still
  // waits for, reads and requests is known at compile time (the loop below decides it per step with a dozen
  // branches, which cost a 64-k step about as much as its four MFMAs).
  auto last_steps = [&](auto count) __attribute__((always_inline)) {
    constexpr int R = decltype(count)::value;
#pragma unroll
    for (int i = 0; i < R; ++i) {
      const int left = R - i;  // steps to go, this one included
      if (left > 1) wait_younger(left > S ? S - 2 : left - 2);
      __syncthreads();
      if (left > 1) read_frags(t + i + 1, fa[(i + 1) & 1], fb[(i + 1) & 1]);
      if (left > S) request_stage(t + i + S);
      mma_stage(fa[i & 1], fb[i & 1]);
    }
  };
  if (nk - t == S + 1) {
    last_steps(std::integral_constant<int, S + 1>{});
    t = nk;
  } else if (nk - t == S) {
    last_steps(std::integral_constant<int, S>{});
    t = nk;
  }
  for (; t < nk; t += 2) {  // a K loop shorter than the ring: requests and reads run out
    step(t, fa[0], fb[0], fa[1], fb[1]);
    if (t + 1 < nk) step(t + 1, fa[1], fb[1], fa[0], fb[0]);
  }
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[0][0][e] += acc_odd[e];
  if constexpr (SPLIT == 1) {
    store_partial_tile<1, 1>(g, acc, lane, bm + wm * 32, bn + wn * 32);
    return;
  }
  if constexpr (SPLIT == 2) {  // the parts meet inside this launch: the last one sums and stores
    if (blockIdx.y + 1 < gridDim.y) return insplit_leave(g, acc, tid, wave, lane);
    insplit_sum(g, acc, lds, tid, wave, lane);
  }
  __syncthreads();  // the ring becomes the epilogue's staging area
  store_tile_result<T, 1, 0, 1>(g, acc, lds, wave, lane, bm + wm * 32, bn + wn * 32);
}

// ---------------------------------------------------------------- MFMA kernel, fp32
// v_mfma_f32_32x32x2_f32 (fp32 in, fp32 accumulate; 157 TFLOP/s dense peak).  Same shape as the
// 128x128 half-precision kernel in bytes: four waves (2x2) of 64x64, 16-k steps (64-byte rows),
// a ring of S 16 KB stages (A 128x16 + B 16x128 fp32) filled by global_load_lds_dwordx4
// S - 1 steps ahead (S = 4: 64 KB, two workgroups per CU; S = 8: 128 KB for problems that leave
// a CU one workgroup anyway, where the deeper ring is what hides the fill latency).  A lane reads one 16-byte chunk (4 consecutive k) per operand block and
// feeds MFMA e (e = 0..3) with its element e: the two k slots of that MFMA are then k = e of
// the lower chunk (lanes 0-31) and of the upper chunk (lanes 32-63) — any pairing works as long
// as both operands use the same one.  Row-major B has no transposing LDS read at 32 bits: a
// lane gathers its four k with four ds_read_b32, rows of the panel offset by 128 bytes every
// four k so that the two lane halves use different banks.  K % 16 == 0, N % 4 == 0.
constexpr int FBK = 16;
// [k][n] fp32 panel, 4 TILE bytes per k row; 16-byte unit u of row k sits at u ^ (8 * ((k / 4) % 2)).
template <int TILE> __device__ __forceinline__ int swz_nf(int k, int n) {
  return k * (TILE * 4) + (((n >> 2) ^ (((k >> 2) & 1) << 3)) << 4) + ((n & 3) << 2);
}

template <bool B_NN, bool SPLIT, int S, int TILE>
__global__ __launch_bounds__(256) void gemm_mfma_f32_kernel(GemmArgs g) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  static_assert(TILE == 128 || TILE == 64, "128x128 or 64x64 tiles");
  constexpr int MI = TILE / 64;                 // 32x32 blocks per wave and dim; also 1 KB regions per wave and panel
  constexpr int kPanel = TILE * FBK * 4;        // bytes per operand per stage
  constexpr int kStage = 2 * kPanel;
  constexpr int UPR = TILE / 4;                 // 16-byte units per k row of a row-major B panel
  const int wm = wave >> 1, wn = wave & 1;
  int tm, tn;
  tile_coords(g, tm, tn);
  const int bm = tm * TILE, bn = tn * TILE;
  const int kbeg = SPLIT ? (int)blockIdx.y * g.ksplit : 0;
  const int kend = SPLIT ? (kbeg + g.ksplit < g.K ? kbeg + g.ksplit : g.K) : g.K;
  const float* A = static_cast<const float*>(g.a) + kbeg;
  const float* B = static_cast<const float*>(g.b) + (B_NN ? (int64_t)kbeg * g.ldb : (int64_t)kbeg);
  const uint32_t lds_base = (uint32_t)(uintptr_t)lds;

  const float* a_src[MI];
  const float* b_src[MI];
#pragma unroll
  for (int i = 0; i < MI; ++i) {
    const int q = wave + 4 * i;
    {  // K-contiguous panel: region q = rows 16q .. 16q+15, 4 chunks of 4 floats per row
      const int r = 16 * q + (lane >> 2), slot = lane & 3;
      const int c = slot ^ ((r >> 2) & 3);
      int gr = bm + r;
      gr = gr < g.M ? gr : g.M - 1;
      a_src[i] = A + (int64_t)gr * g.lda + c * 4;
    }
    if constexpr (!B_NN) {
      const int r = 16 * q + (lane >> 2), slot = lane & 3;
      const int c = slot ^ ((r >> 2) & 3);
      int gn = bn + r;
      gn = gn < g.N ? gn : g.N - 1;
      b_src[i] = B + (int64_t)gn * g.ldb + c * 4;
    } else {  // N-contiguous panel: region q = 64 / UPR k rows of UPR units of 4 floats
      const int k = (64 / UPR) * q + lane / UPR, pos = lane % UPR;
      const int u = pos ^ (((k >> 2) & 1) << 3);
      int gn = bn + u * 4;
      gn = gn < g.N ? gn : 0;
      b_src[i] = B + (int64_t)k * g.ldb + gn;
    }
  }
  auto request_tile = [&](int t) {
    const uint32_t stage = lds_base + (uint32_t)(t % S) * kStage;
    const int64_t k0 = (int64_t)t * FBK;
#pragma unroll
    for (int i = 0; i < MI; ++i) {
      const uint32_t region = (uint32_t)(wave + 4 * i) * 1024u;
      lds_dma16(stage + region, a_src[i] + k0);
      if constexpr (!B_NN) lds_dma16(stage + kPanel + region, b_src[i] + k0);
      else lds_dma16(stage + kPanel + region, b_src[i] + k0 * g.ldb);
    }
  };

  const int fr = lane & 31, fg = lane >> 5;
  // Operand blocks of 8-k sub-step ks (0, 1) of step t: 4 floats per lane and block.
  auto read_frags = [&](int t, int ks, f32x4 (&fa)[MI], f32x4 (&fb)[MI]) {
    const unsigned char* pa = lds + (t % S) * kStage;
    const unsigned char* pb = pa + kPanel;
#pragma unroll
    for (int i = 0; i < MI; ++i)
      fa[i] = *reinterpret_cast<const f32x4*>(pa + swz_k32(wm * 32 * MI + i * 32 + fr, ks * 2 + fg));
#pragma unroll
    for (int j = 0; j < MI; ++j) {
      if constexpr (!B_NN) {
        fb[j] = *reinterpret_cast<const f32x4*>(pb + swz_k32(wn * 32 * MI + j * 32 + fr, ks * 2 + fg));
      } else {
        const int n = wn * 32 * MI + j * 32 + fr;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          fb[j][e] = *reinterpret_cast<const float*>(pb + swz_nf<TILE>(ks * 8 + fg * 4 + e, n));
      }
    }
  };

  f32x16 acc[MI][MI];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < MI; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  auto mma = [&](f32x4 (&fa)[MI], f32x4 (&fb)[MI]) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < MI; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[j][e], fa[i][e], acc[i][j], 0, 0, 0);
  };

  const int nk = (kend - kbeg) / FBK;
  for (int t = 0; t < S - 1 && t < nk; ++t) request_tile(t);
  // Step t reads tile t and the first half of tile t + 1: all but the newest S - 3 tiles must
  // have landed (2 MI requests per thread and tile).
  if (nk >= S - 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * MI * (S - 3)) : "memory");
  else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  f32x4 fa0[MI], fb0[MI], fa1[MI], fb1[MI];
  read_frags(0, 0, fa0, fb0);
  int it = 0;
  for (; it + S - 1 < nk; ++it) {
    request_tile(it + S - 1);
    read_frags(it, 1, fa1, fb1);
    mma(fa0, fb0);
    read_frags(it + 1, 0, fa0, fb0);
    mma(fa1, fb1);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * MI * (S - 3)) : "memory");
    __syncthreads();
  }
  for (; it < nk; ++it) {
    read_frags(it, 1, fa1, fb1);
    mma(fa0, fb0);
    if (it + 1 < nk) read_frags(it + 1, 0, fa0, fb0);
    mma(fa1, fb1);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  }

  if constexpr (SPLIT) {
    store_partial_tile<MI, MI>(g, acc, lane, bm + wm * 32 * MI, bn + wn * 32 * MI);
    return;
  }
  // Register r of acc[i][j] in lane l is C[m0 + 32 i + l%32][n0 + 32 j + 8 (r/4) + 4 (l/32) + r%4]:
  // four consecutive n per lane and r/4, stored as one 16-byte vector.
  const float* C = static_cast<const float*>(g.c);
  const bool use_c = C != nullptr && g.beta != 0.f;
  float* D = static_cast<float*>(g.out);
#pragma unroll
  for (int i = 0; i < MI; ++i) {
    const int m = bm + wm * 32 * MI + i * 32 + fr;
    if (m >= g.M) continue;
#pragma unroll
    for (int j = 0; j < MI; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = bn + wn * 32 * MI + j * 32 + q * 8 + fg * 4;
        if (n >= g.N) continue;
        f32x4 r;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float v = g.alpha * acc[i][j][q * 4 + e];
          const int ne = n + e < g.N ? n + e : g.N - 1;
          if (use_c) v += g.beta * C[(int64_t)m * g.c_rs + (int64_t)ne * g.c_cs];
          r[e] = v;
        }
        if (g.out_vec) {
          *reinterpret_cast<f32x4*>(D + (int64_t)m * g.N + n) = r;
        } else {  // N % 4 != 0: misaligned rows, element stores
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < g.N) D[(int64_t)m * g.N + n + e] = r[e];
        }
      }
  }
}

// ---------------------------------------------------------------- generic fallback
// Any strides; accumulates in fp32 (fp64 products run on the MFMA kernel of gemm_f64.hip; instantiated
// for double, this kernel would accumulate in fp64).  A block of 256 threads owns
// a (16 TT) x (16 TT) tile, TT x TT outputs per thread (rows ty TT + i, columns tx + 16 j: lanes
// along n, so LDS reads of B and the stores are conflict-free and coalesced), GK-k steps.  TT = 4:
// 64x64 tiles, 32-k steps; TT = 8: 128x128 tiles, 16-k steps, half the LDS reads per FMA.  The loads of step t + 1 are issued into registers before the FMAs of step t,
// so a step costs its arithmetic and not a round trip to memory; the element-to-thread mapping
// of each operand's loads follows its contiguous dim.
template <typename T, int TT>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const T* __restrict__ A, int64_t a_rs, int64_t a_cs,
                                                          const T* __restrict__ B, int64_t b_rs, int64_t b_cs,
                                                          const T* __restrict__ C, int64_t c_rs, int64_t c_cs,
                                                          T* __restrict__ D, int64_t M, int64_t N, int64_t K,
                                                          typename std::conditional<std::is_same<T, double>::value, double, float>::type alpha,
                                                          typename std::conditional<std::is_same<T, double>::value, double, float>::type beta) {
  using Acc = typename std::conditional<std::is_same<T, double>::value, double, float>::type;
  constexpr int GT = 16 * TT, GK = 128 / TT;
  constexpr int PER = GT * GK / 256;  // elements of each operand a thread moves per step
  __shared__ Acc As[GK][GT + 1], Bs[GK][GT + 1];
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  const int64_t bm = (int64_t)blockIdx.y * GT, bn = (int64_t)blockIdx.x * GT;
  const bool a_k_fast = a_cs == 1 || a_rs != 1;  // consecutive threads along k, unless A is M-contiguous
  const bool b_n_fast = b_cs == 1 || b_rs != 1;  // consecutive threads along n, unless B is K-contiguous
  Acc ra[PER], rb[PER];
  auto fetch = [&](int64_t k0) {
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int e = threadIdx.x + 256 * u;
      const int r = a_k_fast ? e / GK : e % GT, kk = a_k_fast ? e % GK : e / GT;
      const int64_t m = bm + r, k = k0 + kk;
      ra[u] = (m < M && k < K) ? static_cast<Acc>(A[m * a_rs + k * a_cs]) : Acc(0);
      const int c = b_n_fast ? e % GT : e / GK, kk2 = b_n_fast ? e / GT : e % GK;
      const int64_t n = bn + c, k2 = k0 + kk2;
      rb[u] = (n < N && k2 < K) ? static_cast<Acc>(B[k2 * b_rs + n * b_cs]) : Acc(0);
    }
  };
  Acc acc[TT][TT] = {};
  fetch(0);
  for (int64_t k0 = 0; k0 < K; k0 += GK) {
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int e = threadIdx.x + 256 * u;
      As[a_k_fast ? e % GK : e / GT][a_k_fast ? e / GK : e % GT] = ra[u];
      Bs[b_n_fast ? e / GT : e % GK][b_n_fast ? e % GT : e / GK] = rb[u];
    }
    __syncthreads();
    if (k0 + GK < K) fetch(k0 + GK);
#pragma unroll
    for (int kk = 0; kk < GK; ++kk) {
      Acc av[TT], bv[TT];
#pragma unroll
      for (int i = 0; i < TT; ++i) av[i] = As[kk][ty * TT + i];
#pragma unroll
      for (int j = 0; j < TT; ++j) bv[j] = Bs[kk][tx + 16 * j];
#pragma unroll
      for (int i = 0; i < TT; ++i)
#pragma unroll
        for (int j = 0; j < TT; ++j) acc[i][j] += av[i] * bv[j];
    }
    __syncthreads();
  }
  const bool use_c = C != nullptr && beta != Acc(0);  // tested in the accumulation type: a tiny f64 beta still counts
#pragma unroll
  for (int i = 0; i < TT; ++i) {
    const int64_t m = bm + ty * TT + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < TT; ++j) {
      const int64_t n = bn + tx + 16 * j;
      if (n >= N) continue;
      Acc v = alpha * acc[i][j];
      if (use_c) v += beta * static_cast<Acc>(C[m * c_rs + n * c_cs]);
      D[m * N + n] = static_cast<T>(v);
    }
  }
}

// Split-K plan for problems with fewer 128x128 tiles than CUs and a long K: how many splits,
// and the k extent of each (a multiple of the kernel's k step).  The split count minimises a
// small cost model fitted to this chip: a 128x128 workgroup alone on a CU spends ~12.8 ns per k
// (fp32: ~70 ns), two on a CU ~0.7 of that each, and a split adds a finishing launch (~3 us)
// plus the fp32 partial planes written and read once at ~4 TB/s.  Each split keeps >= 8 k steps
// (>= 4 when the output is one or two tiles).
struct SplitPlan {
  int nsplit, ksplit;
  int mode;  // how the parts meet: 1 in a summing launch, 2 inside the one launch (insplit_sum; bf16 / f16 only)
};
// What the meeting costs, in ns, on top of the longest part's K loop.  A summing launch: 3 us and every plane
// written and read once at ~4 TB/s.  Inside the launch: the producers' planes go out in ~1.5 us, and the summing
// workgroup takes them in two (128x128 tiles, 64 KB each: ~1.0 us a plane) or four (64x64, 16 KB: ~0.6 us) at a time.
static double split_meet_ns(int mode, int64_t ns, int64_t M, int64_t N, int tile) {
  if (ns <= 1) return 0.0;
  if (mode == 2) return 1500.0 + (tile == 64 ? 600.0 : 1000.0) * (double)(ns - 1);
  return 3000.0 + (double)ns * (double)M * (double)N * 8.0 / 4000.0;  // 4 TB/s = 4000 B/ns
}
// The modes the plan may choose from: both for bf16 / f16 unless the gemm_split knob names one.
static void split_modes(int elem_size, bool (&allowed)[3]) {
  const Knobs& kn = knobs();
  allowed[1] = elem_size == 4 || strcmp(kn.gemm_split, "inlaunch") != 0;
  allowed[2] = elem_size == 2 && strcmp(kn.gemm_split, "launch2") != 0;
}
// Workspace a plan needs: planes of whole rows (a summing launch), or (nsplit - 1) planes of whole tiles and a
// 64-bit flag each (inside the launch).
static int64_t split_ws_bytes(const SplitPlan& p, int64_t M, int64_t N, int tile) {
  if (p.nsplit <= 1) return 0;
  if (p.mode == 2) {
    const int64_t tiles = ((M + tile - 1) / tile) * ((N + tile - 1) / tile);
    return (int64_t)(p.nsplit - 1) * tiles * ((int64_t)tile * tile * 4 + 8);
  }
  return (int64_t)p.nsplit * M * ((N + 3) / 4 * 4) * 4;
}
// fp32 products that leave most CUs without a 128x128 tile run on 64x64 tiles.
static int f32_tile(int64_t M, int64_t N) {
  return ((M + SBM - 1) / SBM) * ((N + SBN - 1) / SBN) < kNumCU * 3 / 4 ? 64 : 128;
}
// What a 128x128 workgroup of the bf16 / f16 kernels adds per k, in ns, when `wgs` of them run in one launch: the
// slope between K = 1024 and K = 4096 of [128 tm, K] x [128 tn, K]^T without a split, on inputs that no cache
// holds.  Up to 128 workgroups the K loop runs at the latency of fills that the warming workgroups have sent ahead
// (warm_operands; 7.9 ns without them, whatever the count); towards 224 there are fewer CUs left for those and
// the fills start to queue; beyond one per CU two share a CU's LDS and fill path.
static double small_ns_per_k(int64_t wgs) {
  // (between a transposed b - 5.5 ns up to 128 workgroups, 6.6 at 192, 8.45 at 256 - and a row-major one - 6.7, 8.0,
  // 9.5: the plan is made before the layouts are known, mi355_gemm_workspace_bytes has to agree with it)
  static const struct { int wgs; double ns; } pts[] = {{64, 6.0}, {128, 6.3}, {160, 6.55}, {192, 7.3}, {208, 7.4}, {224, 8.2},
                                                       {240, 8.6}, {256, 9.0}, {320, 16.4}, {384, 18.0}, {512, 22.3}};
  constexpr int n = sizeof(pts) / sizeof(pts[0]);
  if (wgs <= pts[0].wgs) return pts[0].ns;
  if (wgs > pts[n - 1].wgs) return pts[n - 1].ns * (double)((wgs + 511) / 512);  // rounds of two per CU
  for (int i = 1; i < n; ++i)
    if (wgs <= pts[i].wgs)
      return pts[i - 1].ns + (pts[i].ns - pts[i - 1].ns) * (double)(wgs - pts[i - 1].wgs) / (double)(pts[i].wgs - pts[i - 1].wgs);
  return pts[n - 1].ns;
}
static SplitPlan plan_splitk(int64_t M, int64_t N, int64_t K, int elem_size) {
  // Parts of whole steps: 64 k where K allows it, so that every part keeps the deep-ring kernel's 64-k pairs
  // (a part of 3680 k fell back to the 32-k kernel: [1024,11008]x[11008,1024] in three parts 56 us, in four 44).
  const int bk = elem_size == 4 ? FBK : K % 64 == 0 ? 64 : BK3;
  const int tile = elem_size == 4 ? f32_tile(M, N) : SBM;
  const int64_t tiles = ((M + tile - 1) / tile) * ((N + tile - 1) / tile);
  SplitPlan p{1, (int)K, 1};
  if (tiles >= kNumCU || K % bk != 0) return p;
  const double ns_per_k = elem_size == 4 ? (tile == 64 ? 20.0 : 70.0) : 12.8;
  const int min_steps = tiles <= 2 ? 4 : 8;  // one or two tiles: the launch is all latency, shorter splits still pay
  const int64_t min_k = (int64_t)min_steps * (elem_size == 4 ? FBK : BK3);  // (steps of the 32-k kernels, as measured)
  const int64_t max_ns = K / min_k < 64 ? K / min_k : 64;
  bool allowed[3];
  split_modes(elem_size, allowed);
  double best = 1e30;
  int64_t best_ns = 1;
  int best_mode = 1;
  for (int64_t ns = 1; ns <= max_ns; ++ns) {
    int64_t ks = (K + ns - 1) / ns;
    ks = (ks + bk - 1) / bk * bk;
    const int64_t real_ns = (K + ks - 1) / ks;
    if (real_ns != ns) continue;  // this count rounds to one already tried
    if (K - (ns - 1) * ks < min_k) continue;  // the last split would fall under the minimum
    const int64_t per_cu = (tiles * ns + kNumCU - 1) / kNumCU;
    // (A few rows against a weight that is streamed once - decoding - are bound by that stream, not by the tiles'
    // K loops: they keep the older figures, under which more, shorter parts win: [8,8192]x[8192,8192]^T 30.9 us
    // against 37.1.)
    const double t_k = elem_size == 2 && M > 32 ? (double)ks * small_ns_per_k(tiles * ns)
                                      : (double)per_cu * (per_cu >= 2 ? 0.7 : 1.0) * (double)ks * ns_per_k;
    if (ns == 1) {  // the unsplit product: what a split has to beat
      best = t_k;
      continue;
    }
    // The parts meet whichever way is cheaper for this count.
    const int mode = allowed[2] && (!allowed[1] || split_meet_ns(2, ns, M, N, tile) < split_meet_ns(1, ns, M, N, tile)) ? 2 : 1;
    const double t = t_k + split_meet_ns(elem_size == 2 ? mode : 1, ns, M, N, tile);
    if (t < best) {
      best = t;
      best_ns = ns;
      best_mode = mode;
    }
  }
  if (best_ns <= 1) return p;
  int64_t ks = (K + best_ns - 1) / best_ns;
  ks = (ks + bk - 1) / bk * bk;
  p.ksplit = (int)ks;
  p.nsplit = (int)((K + ks - 1) / ks);
  p.mode = best_mode;
  return p;
}

// Split-K for the 64x64-tile kernel: a handful of tiles with a long K (one image's 197 tokens against a
// 3072 x 768 weight) leave most CUs idle and walk K at about 0.21 us per 64-k stage.  Splits of whole stages, at
// least four each; the cost model is the one of plan_splitk with this kernel's figures (2 us to get going,
// 0.21 us per stage - [896,3584]x[896,3584]^T, 196 tiles: 15.7 us for 56 stages - and 1.1 x that per workgroup
// when several share a CU, 3 us and the partial planes for the summing launch).
static SplitPlan plan_t64_split(int64_t M, int64_t N, int64_t K) {
  SplitPlan p{1, (int)K, 1};
  const int64_t tiles = ((M + TBM - 1) / TBM) * ((N + TBN - 1) / TBN);
  if (K % 64 != 0 || K < 1024 || tiles > kNumCU / 2) return p;
  const int64_t stages = K / 64;
  bool allowed[3];
  split_modes(2, allowed);
  double best = 1e30;
  int64_t best_ks = stages;
  int best_mode = 1;
  for (int64_t ns = 1; ns <= stages / 4 && ns <= 64; ++ns) {
    const int64_t ks = (stages + ns - 1) / ns;
    if ((stages + ks - 1) / ks != ns || stages - (ns - 1) * ks < 4) continue;
    const int64_t per_cu = (tiles * ns + kNumCU - 1) / kNumCU;
    const double t_k = 2000.0 + 210.0 * (double)ks * (per_cu >= 2 ? 1.1 * (double)per_cu : 1.0);
    if (ns == 1) {  // the unsplit product: what a split has to beat
      best = t_k;
      continue;
    }
    const double t = t_k + split_meet_ns(1, ns, M, N, 64);  // (part count against the summing launch, as in plan_splitk)
    if (t < best) {
      best = t;
      best_ks = ks;
      best_mode = allowed[2] && (!allowed[1] || split_meet_ns(2, ns, M, N, 64) < split_meet_ns(1, ns, M, N, 64)) ? 2 : 1;
    }
  }
  p.ksplit = (int)(best_ks * 64);
  p.nsplit = (int)((stages + best_ks - 1) / best_ks);
  p.mode = p.nsplit > 1 ? best_mode : 1;
  return p;
}

// Split-K inside one launch of the 16x16x32 kernel (gemm_mfma_x16_splitk_kernel): for products with 65 - 128
// tiles of 256x256 (a quarter to half of the CUs) and K >= 2048 (1536 for 96 - 112 tiles, 3072 from 113 on), two workgroups per tile,
// each with about half of K.  The caller's workspace holds one fp32 plane of 256 KB per tile and a 64-bit flag per
// plane.  Measured against one workgroup per tile ([M,K]x[N,K]^T, us; the stock kernel in brackets): 96 tiles at
// K = 1536 36.7 -> 34.6 (27.7; the 128x128 kernels 34.7; 72 tiles: 36.0 -> 32.5, the 128x128 kernels 30.4), at K = 2048 44 -> 40 (33), at 3072 63 -> 50 (47), at 4096 77 -> 60 (58), at 8192 143 -> 97 (106); 128 tiles at K =
// 2048 46 -> 45 (40), at 3072 65 -> 56 (56), at 4096 80 -> 69 (69), at 8192 148 -> 114 (126).  The exchange costs
// a producer 3 us (its plane, 16 bytes a lane and instruction) and the summing workgroup 4 us on top of its
// epilogue; a CU takes a plane in at 50 - 60 GB/s, so more workgroups per tile do not pay - the one that sums
// reads all the other planes (48 tiles at K = 8192: two parts 86 us, three 78, four 83; the 128x128 kernels 90),
// which is why the plan knows only two; the kernel takes up to four (a test knob: x16split3, x16split4).
struct X16SplitPlan {
  int splits, tiles8;
  int64_t ws_bytes;
};
constexpr int64_t kX16SplitMinK = 2048, kX16SplitMinKMid = 1536, kX16SplitMinKFull = 3072;
constexpr int kX16MaxSplits = 4;  // the summing workgroup's epilogue exists for one to three producers
static X16SplitPlan plan_x16_split(int64_t M, int64_t N, int64_t K) {
  X16SplitPlan p{1, 0, 0};
  const int64_t tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  if (K % kX16SplitUnit != 0) return p;
  const Knobs& kn = knobs();
  int splits = 0;
  if (strncmp(kn.gemm_tile, "x16split", 8) == 0 && kn.gemm_tile[8] >= '2' && kn.gemm_tile[8] <= '0' + kX16MaxSplits && kn.gemm_tile[9] == 0) {
    splits = kn.gemm_tile[8] - '0';  // a test knob: this many workgroups per tile at any tile count
  } else {
    if (tiles <= kNumCU / 4 || tiles > kNumCU / 2 || K < (tiles > 112 ? kX16SplitMinKFull : tiles >= 96 ? kX16SplitMinKMid : kX16SplitMinK)) return p;
    splits = 2;
  }
  // every share is at least two units (the kernel's K loop needs 256): the producers share what the summing
  // workgroup leaves
  const int units = (int)(K / kX16SplitUnit);
  if ((units - x16_split_summing_units(units, splits)) / (splits - 1) < 2) return p;
  p.splits = splits;
  p.tiles8 = (int)((tiles + 7) / 8 * 8);
  p.ws_bytes = (p.splits - 1) * tiles * (int64_t)(BM * BN * 4 + 8);
  return p;
}

// Widths for the four-wave kernel's tile columns: `wide` columns of 256 followed by `narrow` columns
// of 192 (gemm_mfma_w4_mixed_kernel), chosen to minimise the time of the launch when workgroups
// go to the CUs in block order, one per CU; narrow == 0 is the plain 256-wide grid.  A 192-wide
// tile is priced at kNarrowCost of a 256-wide one (three quarters of the MFMAs on the same fills).
struct MixedPlan {
  int wide, narrow;
};
constexpr double kNarrowCost = 0.85;  // measured: 0.78 of the K loop's ticks, the per-tile prologue and epilogue in full
constexpr int64_t kMixedMinK = 4096;  // shorter K loops: the per-tile overhead of the extra tiles eats the gain
static double mixed_makespan(int64_t n_wide, int64_t n_narrow) {
  // wide tiles first: after them `late` CUs are free at time rounds + 1, the others at `rounds`
  const int64_t rounds = n_wide / kNumCU, late = n_wide % kNumCU;
  double t[2] = {(double)rounds, (double)rounds + 1.0};
  int64_t cnt[2] = {kNumCU - late, late};
  double end = late ? t[1] : t[0];
  if (n_wide == 0) end = 0.0;
  while (n_narrow > 0) {
    const int e = (cnt[1] > 0 && t[1] < t[0]) || cnt[0] == 0 ? 1 : 0;
    const int64_t take = n_narrow < cnt[e] ? n_narrow : cnt[e];
    n_narrow -= take;
    const double fin = t[e] + kNarrowCost;
    if (fin > end) end = fin;
    if (take == cnt[e]) {
      t[e] = fin;
    } else {  // last, partial batch: nothing is scheduled behind it
      break;
    }
  }
  return end;
}
static MixedPlan plan_mixed(int64_t tiles_m, int64_t N) {
  static thread_local int64_t key_m = -1, key_n = -1;
  static thread_local MixedPlan cached{0, 0};
  if (key_m == tiles_m && key_n == N) return cached;
  const int64_t all_wide = (N + 255) / 256;
  MixedPlan best{(int)all_wide, 0};
  double best_t = mixed_makespan(tiles_m * all_wide, 0);
  for (int64_t narrow = 1; narrow * 192 < N + 192; ++narrow) {
    const int64_t rest = N - narrow * 192;
    const int64_t wide = rest > 0 ? (rest + 255) / 256 : 0;
    if (wide * 256 + (narrow - 1) * 192 >= N) continue;  // the last narrow column would start past the matrix
    const double t = mixed_makespan(tiles_m * wide, tiles_m * narrow);
    if (t < best_t - 0.1) {  // a mixed grid has to pay for itself
      best_t = t;
      best = MixedPlan{(int)wide, (int)narrow};
    }
  }
  key_m = tiles_m; key_n = N; cached = best;
  return best;
}

template <typename T>
static int finish_splitk(const GemmArgs& g, int nsplit, hipStream_t st) {
  const int64_t quads = (int64_t)g.M * g.ws_ld / 4;
  if (quads < (int64_t)kNumCU * 256 * 2 && nsplit >= 4) {  // under two blocks per CU: four lanes per group of columns
    const int grid = grid_for(quads, 64, kNumCU * 8);
    hipLaunchKernelGGL((gemm_splitk_finish4_kernel<T>), dim3(grid), dim3(256), 0, st, g, nsplit);
  } else {
    const int grid = grid_for(quads, 256, kNumCU * 8);
    hipLaunchKernelGGL((gemm_splitk_finish_kernel<T>), dim3(grid), dim3(256), 0, st, g, nsplit);
  }
  return check_launch("mi355_gemm(split-k finish)");
}

// A flag value of its own for every launch whose workgroups meet through flags in the workspace: odd, and
// stepped by two - never 0, which is what a flag holds between launches.
static unsigned long long next_split_epoch() {
  static std::atomic<unsigned long long> epoch{0x5bd1e9955bd1e995ull};
  return epoch.fetch_add(2);
}

// mi355_gemm_plan: run_gemm stops in front of its launch and leaves what it would have launched here.
static thread_local char* g_plan_text = nullptr;
static thread_local int64_t g_plan_cap = 0;
static int describe_plan(const char* form, int tiles_m, int tiles_n, int64_t grid_x, int grid_y, int threads, int lds_bytes,
                         int parts, const char* meet, int warm) {
  snprintf(g_plan_text, (size_t)g_plan_cap, "form=%s tiles=%dx%d grid=%lldx%d threads=%d lds=%d parts=%d meet=%s warm=%d", form, tiles_m,
           tiles_n, (long long)grid_x, grid_y, threads, lds_bytes, parts, meet, warm);
  return MI355_OK;
}

template <typename T>
static int run_gemm(const void* a, int64_t a_rs, int64_t a_cs, const void* b, int64_t b_rs, int64_t b_cs,
                    const void* c, int64_t c_rs, int64_t c_cs, void* out, int64_t M, int64_t N, int64_t K,
                    double alpha, double beta, void* workspace, int64_t workspace_bytes, hipStream_t st) {
  constexpr bool can_mfma = sizeof(T) == 2;
  if constexpr (can_mfma) {
    const bool a_ok = a_cs == 1 && a_rs % 8 == 0 && aligned16(a);
    const bool b_nt = b_rs == 1 && b_cs % 8 == 0 && aligned16(b);
    const bool b_nn = b_cs == 1 && b_rs % 8 == 0 && aligned16(b);
    const bool fits = M < (1 << 30) && N < (1 << 30) && K < (1 << 30);
    // Tiny outputs with a short K are cheaper on the generic kernel than on a mostly empty MFMA
    // tile.  Anything with a K loop worth pipelining is not: [64, 512] x [512, 64] takes 72 us there
    // and 8 us here, and a single row against a large weight (decoding one token) streams the
    // whole weight.
    const bool worth = K >= 32 && (M * N >= 32 * 32 || K >= 256 || M * N * K >= (int64_t(1) << 22));
    // Row-major B needs N % 8 == 0 (its rows must start on 16-byte boundaries); transposed B takes
    // any N — a 50257-wide vocabulary projection stores its misaligned output rows element-wise.
    const bool b_nn_ok = b_nn && N % 8 == 0;
    // An M-contiguous left operand (a transposed view) is taken as it is by the four-wave and the
    // 128x128 kernels when its k-rows start on 16-byte boundaries and K is a multiple of 64.
    // The four-wave kernels address their fills with 32-bit byte offsets from a per-tile base:
    // up to 256 rows of either operand must span less than 4 GB.
    const bool ld32 = (a_ok ? a_rs : a_cs) < (1 << 22) && (b_nt ? b_cs : b_rs) < (1 << 22);
    const bool a_t = !a_ok && a_rs == 1 && a_cs % 8 == 0 && aligned16(a) && M % 8 == 0 && K % 64 == 0 && ld32;
    if ((a_ok || a_t) && (b_nt || b_nn_ok) && K % 8 == 0 && fits && worth && K > 0) {
      GemmArgs g{};
      g.a = a; g.b = b; g.c = c; g.out = out;
      g.lda = a_t ? a_cs : a_rs;
      g.ldb = b_nt ? b_cs : b_rs;
      g.c_rs = c_rs; g.c_cs = c_cs;
      g.c_vec = c != nullptr && c_cs == 1 && c_rs % 4 == 0 && reinterpret_cast<uintptr_t>(c) % 8 == 0 && N % 4 == 0;
      g.out_vec = N % 8 == 0 && aligned16(out);
      g.bias_vec = c != nullptr && c_rs == 0 && c_cs == 1 && reinterpret_cast<uintptr_t>(c) % 8 == 0;
      g.M = (int32_t)M; g.N = (int32_t)N; g.K = (int32_t)K;
      g.alpha = (float)alpha; g.beta = (float)beta;
      g.tiles_m = (int32_t)((M + BM - 1) / BM);
      g.tiles_n = (int32_t)((N + BN - 1) / BN);
      int64_t nblocks = (int64_t)g.tiles_m * g.tiles_n;
      MI355_REQUIRE(nblocks < (int64_t(1) << 31), "mi355_gemm: too many tiles");
      const bool ktail = K % BK3 != 0;
      const void* kern;
      int lds_bytes = kGemmLds;
      int threads = 512;
      int nsplit = 1;
      int warm_blocks = 0;  // workgroups behind the tiles that only warm the last-level cache (warm_operands)
      const char* form = "";  // the kernel form, for mi355_gemm_plan
      // Per part of K, for a launch of one workgroup per CU: up to 32 of the CUs it leaves idle, when a part's K
      // loop has `min_k` and more (a ring holds the first stages of a K loop itself).  gemm_prefetch = N forces N
      // (0: none): a measurement knob.
      auto warm_for = [&](int64_t tiles, int64_t min_k) {
        const int64_t idle = (kNumCU - tiles * nsplit) / nsplit;
        const int64_t want = knobs().gemm_prefetch >= 0 ? knobs().gemm_prefetch : K / nsplit >= min_k ? 32 : 0;
        if (knobs().gemm_prefetch < 0 && idle < 16) return 0;  // too few to stay ahead of the tiles
        return (int)(idle < 0 ? 0 : idle < want ? idle : want);
      };
      auto pick_w4 = [&](auto nj) -> const void* {
        constexpr int NJ = decltype(nj)::value;
        if (a_t) return b_nt ? (const void*)gemm_mfma_w4_kernel<T, false, NJ, true> : (const void*)gemm_mfma_w4_kernel<T, true, NJ, true>;
        return b_nt ? (const void*)gemm_mfma_w4_kernel<T, false, NJ, false> : (const void*)gemm_mfma_w4_kernel<T, true, NJ, false>;
      };
      // The parts of a split K meet inside the launch (SplitPlan::mode 2): planes of whole tiles at the start of the
      // workspace, one flag per plane behind them.
      bool meet_inside = false;
      auto arm_insplit = [&](int64_t tiles, int tile) {
        meet_inside = true;
        g.sk_flags = reinterpret_cast<unsigned long long*>(static_cast<unsigned char*>(workspace) + (int64_t)(nsplit - 1) * tiles * tile * tile * 4);
        g.sk_epoch = next_split_epoch();
        g.sk_spin_limit = knobs().x16_spin_limit;
      };
      // The deep-ring 128x128 kernel: with loader waves where an operand is transposed by the LDS reads (a row-major
      // b, an M-contiguous a: three or four DS instructions per MFMA leave the computing waves no slot for
      // the requests: [2048,4096]x[4096,2048] 43.9 -> 41.7 us, [128,1024]x[1024,128] 12.7 -> 10.6), the four-wave
      // form otherwise (level or 1 - 3 % ahead there).  gemm_tile = ring4 / ring8 forces one (measurement knobs).
      const bool four_wave_ring = strcmp(knobs().gemm_tile, "ring4") == 0 || (b_nt && !a_t && strcmp(knobs().gemm_tile, "ring8") != 0);
      auto pick_small = [&](auto deep, auto split_c) -> const void* {
        constexpr int SP = decltype(split_c)::value;
        if constexpr (decltype(deep)::value) {
          if (four_wave_ring) {
            if (a_t) return b_nt ? (const void*)gemm_mfma_small2_kernel<T, false, SP, true> : (const void*)gemm_mfma_small2_kernel<T, true, SP, true>;
            return b_nt ? (const void*)gemm_mfma_small2_kernel<T, false, SP, false> : (const void*)gemm_mfma_small2_kernel<T, true, SP, false>;
          }
          if (a_t) return b_nt ? (const void*)gemm_mfma_small3_kernel<T, false, SP, true> : (const void*)gemm_mfma_small3_kernel<T, true, SP, true>;
          return b_nt ? (const void*)gemm_mfma_small3_kernel<T, false, SP, false> : (const void*)gemm_mfma_small3_kernel<T, true, SP, false>;
        } else {
          if (a_t) return b_nt ? (const void*)gemm_mfma_small_kernel<T, false, SP, true> : (const void*)gemm_mfma_small_kernel<T, true, SP, true>;
          return b_nt ? (const void*)gemm_mfma_small_kernel<T, false, SP, false> : (const void*)gemm_mfma_small_kernel<T, true, SP, false>;
        }
      };
      // Too few 256x256 tiles for the chip but close to one full round of 256x128 tiles, and a K loop
      // long enough to amortise the one-workgroup-per-CU pipeline: the four-wave kernel on 256x128
      // tiles.  Its time does not depend on the tile count up to 256, while the 128x128 kernel's grows
      // with it; measured crossover at about 230 tiles for K = 3072 and 250 for K = 1024.
      // MI355_GEMM_TILE=256x128 forces it (a test knob).
      const int64_t tiles_mid = (int64_t)g.tiles_m * ((N + 127) / 128);
      const Knobs& kn = knobs();
      const char* forced_tile = kn.gemm_tile[0] ? kn.gemm_tile : nullptr;
      const char* forced_waves = kn.gemm_waves[0] ? kn.gemm_waves : nullptr;
      const bool mid = !ktail && K % 64 == 0 && ld32 &&
                       (forced_tile != nullptr ? strcmp(forced_tile, "256x128") == 0
                                               : nblocks < kNumCU * 3 / 4 && tiles_mid <= kNumCU &&
                                                     ((K >= 1024 && tiles_mid > (K >= 2048 ? 228 : 248)) ||
                                                      // More 128x128 tiles than one round of them, few enough 256x128 tiles to leave CUs for
                                                      // warm_operands: this kernel runs at fill latency, and with the operands on their way
                                                      // into the last-level cache it is ahead of the 128x128 kernels with two workgroups on
                                                      // a CU and of two parts of K on 256x256 tiles ([4096,1536]x[1536,1536]^T 35.1 ->
                                                      // 29.4 us, [2048,1536]x[1536,2304] 32.9 -> 25.7, [3072,768]x[2048,768]^T 21.6 -> 18.9;
                                                      // level from K = 4096 on.  Below K = 768 no warming workgroups are added,
                                                      // and with the last six steps of its K loop written out this form is 17 - 30 %
                                                      // ahead of two 128x128 workgroups per CU there too, on either layout of b:
                                                      // [2048,512]x[512,3072] 20.1 -> 15.4 us, [4096,256]x[1536,256]^T 14.3 -> 11.4,
                                                      // [1024,640]x[640,6144] 24.4 -> 17.5; 85 shapes, K = 256 .. 704).
                                                      (K >= 256 && K <= 3072 && tiles_mid > kNumCU / 2)) &&
                                                     4 * M >= 3 * (int64_t)g.tiles_m * BM);  // rows that are mostly output ([128,4096]x[4096,32000]: 74 us here, 61 on 128x128 tiles)
      // Fewer 128x128 tiles than half the CUs: 64x64 tiles reach four times as many (measured on this
      // chip: [197,768]x[768,768] 11.6 -> 7.5 us, 1024^3 14.6 -> 9.4 us).  A 64x64 workgroup walks K at
      // about 0.3 us per 64 k, so a few tiles with a long K stay on the 128x128 kernels, which split K
      // over the chip.  A single row of tiles (M <= 64) also takes them at larger N: half of a 128-row
      // tile would be padding ([32,768]x[768,32000]: 17.5 -> 13.3 us).  MI355_GEMM_TILE=64x64 forces them, =128x128 keeps them off: test knobs.
      const int64_t nb128 = ((M + SBM - 1) / SBM) * ((N + SBN - 1) / SBN);
      const int64_t nb64 = ((M + TBM - 1) / TBM) * ((N + TBN - 1) / TBN);
      // With scratch for its split-K form (plan_t64_split) they also take the few tiles with a long K
      // ([197,3072]x[3072,768]: 15.4 -> 12.1 us, [64,4096]x[4096,4096]: 17.6 -> 15.2, [64,11008]x[11008,4096]: 32.8 ->
      // 28.4; not a handful of rows against a weight that takes longer to stream than to multiply:
      // [8,8192]x[8192,8192] 32.1 us on the 128x128 kernels, 35.8 here split, 42.4 unsplit).
      const SplitPlan ts = plan_t64_split(M, N, K);
      // ... nor 16 - 32 rows against 128 MB of weight ([16,8192]x[8192,8192]: 32.4 us there, 35.8 here).
      const bool light_b = (int64_t)N * K * (int64_t)sizeof(T) <= 100000000;
      const bool t64_split = ts.nsplit > 1 && M >= 16 && light_b && workspace != nullptr &&
                             reinterpret_cast<uintptr_t>(workspace) % 16 == 0 &&
                             workspace_bytes >= split_ws_bytes(ts, M, N, TBM);
      // More 64x64 tiles than CUs put two workgroups on some CUs, and with a row-major b wider than 1536 columns
      // (64 columns of a k row are one 128-byte line, 2 N bytes from the next) those then fall behind the 128x128
      // kernels with K in two parts from K = 2048 on ([512,2048]x[2048,2560] 22.0 -> 17.6 us, [768,2048]x[2048,2560]
      // 23.2 -> 19.6, [1024,2048]x[2048,1792] 19.9 -> 18.7; at K = 1536 the 64x64 tiles are level or up to 20 % ahead),
      // with 65 - 256 rows from K = 1536 on ([256,2048]x[2048,5120] 25.7 -> 18.0 us, [256,1536]x[1536,5120] 20.4 ->
      // 16.8, [128,2048]x[2048,11008] 24.0 -> 20.7).  Narrow products ([3072,2048]x[2048,512]) and a transposed b stay here.
      const bool t64_crowded_nn = !b_nt && nb64 > kNumCU && N >= 1536 && M > 64;
      const int64_t t64_k_max = M <= 32 ? 1024 : t64_crowded_nn ? (M <= 256 ? 1024 : 1536) : 2048;
      const bool t64 = !ktail && K % 64 == 0 && !a_t && ld32 &&
                       (forced_tile != nullptr ? strcmp(forced_tile, "64x64") == 0
                                               : (nb128 < kNumCU / 2 || (nb128 == kNumCU / 2 && K < 2048) ||  // (exactly 128 tiles: K = 512 10.0 -> 7.0 us; at K = 2048 the deep-ring 128x128 kernel with its warming workgroups is level on a transposed b, 19 against 21 - 22 us, and ahead on a row-major one)
                                                  ((M <= 64 || N <= 64) && nb64 <= 4 * kNumCU)) && nb64 >= 4 &&
                                                     (K <= t64_k_max || t64_split ||
                                                      // enough 64x64 tiles for the chip: no need to split a long K (a few rows against a 32000 x 4096
                                                      // vocabulary: 48 us, 128x128 tiles 55) - up to K = 4096 for more than one row of tiles: beyond, the
                                                      // 128x128 kernels with K split over the chip are ahead ([512,8192]x[8192,1536]: 42 us here, 31 there;
                                                      // [768,8192]x[8192,2048]: 62 against 52; at K = 4096 these are level or ahead: 23.4 against 27.5)
                                                      // (from 80 tiles of 128x128 on, two parts of K each on the 128x128 kernels fill the chip and are
                                                      // ahead at K > 2048: [384,4096]x[4096,4096]^T 34.3 -> 28.4 us, [2048,3072]x[768,3072]^T 26.7 -> 24.8)
                                                      // (measured again with the 64x64-tile kernel's fragments read a stage ahead and the 128x128
                                                      // kernels' warming workgroups: up to 64 tiles of 128x128 at K = 3072 / 4096 this kernel is
                                                      // 6 - 20 % ahead, at 72 - 96 tiles 4 - 28 % behind; at K = 8192 ahead up to 32 tiles)
                                                      ((K <= 4096 || M <= 64 || (K <= 8192 && nb128 <= 32)) && (M <= 64 || nb128 <= 64) &&
                                                       ((nb128 < kNumCU / 2 && M >= 16 && light_b) || nb64 >= 160))));
      // The 16x16x32 form of the four-wave kernel (gemm_x16.hip) takes every product that fills the chip
      // with 256x256 tiles when K is a multiple of 128 (from 256 on): measured against the 32x32x16 forms on
      // [4096,K]x[K,16384], it is 11 % faster at K = 256 and 4 - 15 % from K = 768 on (C3: [4096,4096]x
      // [4096,11008] 306 -> 279 us, [4096,11008]x[11008,4096] 270 -> 249 us).  It also takes 129 - 191 tiles
      // (and 96 - 128 at K >= 2048) unless they make one round of 256x128 tiles: a tile's time does not
      // depend on how many CUs run one, while the 128x128 kernels need a second round of their four times
      // as many tiles ([2304,4096]x[4096,4096], 144 tiles: 104 -> 78 us; [1280,4096]x[4096,7680]: 117 -> 82).
      // Output rows that do not start on 128-byte lines (N % 64 != 0) get its whole-tile-row epilogue.
      // MI355_GEMM_TILE=x16 forces this form for any tile count (=x16mixed: with the mixed-width grid at any K), =256x256 / =mixed keep
      // the 32x32x16 form (test knobs).
      // Fewer tiles than CUs: only when the tiles are mostly output (a few rows against a wide weight make
      // 125 tiles of 256 rows that are 99 % padding: [8,4096]x[4096,32000] took 83 us here, 48 on 64x64 tiles).
      const bool well_filled = (double)M * (double)N >= 0.75 * (double)nblocks * BM * BN;
      const bool x16_ok = K % 128 == 0 && K >= 256 && !a_t && ld32;
      const bool x16_pays = nblocks > kNumCU || well_filled;  // (the planner's rule; the knobs force the kernel regardless)
      const bool x16_mixed_forced = forced_tile != nullptr && strcmp(forced_tile, "x16mixed") == 0;  // mixed widths at any K
      const bool x16 = x16_ok && (forced_tile != nullptr ? strcmp(forced_tile, "x16") == 0 || x16_mixed_forced || strcmp(forced_tile, "x16persist") == 0
                                                         : x16_pays && (nblocks > kNumCU / 2 || (nblocks >= 96 && K >= 2048)) && !mid &&
                                                               !t64 && forced_waves == nullptr);
      // Too few tiles for the chip and a long K: the same kernel with two workgroups per tile that share K
      // and meet in the workspace (plan_x16_split).  Any value of MI355_GEMM_TILE but x16split keeps it off.
      X16SplitPlan xs = plan_x16_split(M, N, K);
#ifdef MI355_GEMM_TRACE
      xs.splits = 1;  // the stamps use the workspace
#endif
      const bool x16_split = x16_ok && xs.splits > 1 && workspace != nullptr && workspace_bytes >= xs.ws_bytes &&
                             reinterpret_cast<uintptr_t>(workspace) % 16 == 0 &&
                             (forced_tile != nullptr ? strncmp(forced_tile, "x16split", 8) == 0
                                                     // (where the 256x128 form applies it goes first up to K = 3072 with CUs left for its warming
                                                     // workgroups, and below K = 3072 on 229 - 256 such tiles: there, measured on 21 shapes, the
                                                     // two forms take 40 - 44 against 47 - 52 us at K = 2048, 56 - 66 against 53 - 57 at 3072 and
                                                     // 70 - 78 against 65 - 66 at 4096)
                                                     : x16_pays && M >= 512 && forced_waves == nullptr && !(mid && (K < 3072 || tiles_mid <= 224)));  // (256 rows against 32000 x 4096: 94 us split, 85 unsplit - the planes on top of a weight that is streamed anyway)
      if (x16_split) {
        kern = gemm_x16_splitk_kernel(std::is_same<T, bf16_t>::value, !b_nt);
        form = "x16_split";
        threads = 256;
        lds_bytes = kX16Lds;
        g.ws = static_cast<float*>(workspace);
        g.sk_splits = xs.splits;
        g.sk_tiles8 = xs.tiles8;
        g.sk_epoch = next_split_epoch();
        g.sk_spin_limit = kn.x16_spin_limit;
        g.sk_flags = reinterpret_cast<unsigned long long*>(static_cast<unsigned char*>(workspace) + (int64_t)(xs.splits - 1) * nblocks * (BM * BN * 4));
        g.out_rows = N % 64 != 0 || reinterpret_cast<uintptr_t>(out) % 128 != 0;
        nblocks = (int64_t)xs.splits * xs.tiles8;
      } else if (x16) {
        kern = gemm_x16_kernel(std::is_same<T, bf16_t>::value, !b_nt);
        form = "x16";
        threads = 256;
        lds_bytes = kX16Lds;
        // More tiles than CUs, all of them whole: one workgroup per CU walks its tiles with the fill
        // requests running on across them (gemm_mfma_x16_persistent_kernel).  MI355_GEMM_TILE=x16 keeps
        // one workgroup per tile, =x16persist takes the walk for any tile count (test knobs).
        const bool persist_forced = forced_tile != nullptr && strcmp(forced_tile, "x16persist") == 0;
        // The walk pays from four rounds of tiles on, or with a long K: with a short K and one to three
        // rounds the workgroups that start late or run on a slower CU get as many tiles as the others,
        // where the dispatcher hands a tile to whichever CU is free first ([8192,768]x[768,2304], 288
        // tiles: 46.2 us against 43.4; [12544,768]x[768,3072], 588 tiles: 75.8 against 71.1; level at
        // exactly two and three rounds; 24.5 rounds at K = 768: 592 against 636).
        // M or N off the multiples of 256: the walk moves its last row / column of tiles back to the edge and
        // computes the overlap twice - for output rows on 128-byte lines, and never when c shares memory with
        // out (an element of the overlap would take beta * c twice).
        const unsigned char* c_lo = static_cast<const unsigned char*>(c);
        const unsigned char* o_lo = static_cast<const unsigned char*>(out);
        const int64_t c_span = ((M - 1) * c_rs + (N - 1) * c_cs + 1) * (int64_t)sizeof(T);  // (non-negative strides)
        const bool c_apart = c == nullptr || beta == 0.0 ||
                             (c_rs >= 0 && c_cs >= 0 && (c_lo + c_span <= o_lo || o_lo + M * N * (int64_t)sizeof(T) <= c_lo));
        const bool whole = M % BM == 0 && N % BN == 0;
        const bool edge_ok = M >= BM && N >= BN && N % 64 == 0 && reinterpret_cast<uintptr_t>(out) % 128 == 0 && c_apart;
        bool persist = (whole || edge_ok) && g.out_vec && K >= 384 &&
                       (forced_tile == nullptr ? nblocks > kNumCU && (K >= 2048 || nblocks >= 4 * kNumCU) : persist_forced);
#ifdef MI355_GEMM_TRACE
        persist = false;  // the stamps are per workgroup = per tile
#endif
        if (persist) {
          kern = gemm_x16_persistent_kernel(std::is_same<T, bf16_t>::value, !b_nt);
          form = "x16_persistent";
          if (nblocks > kNumCU) nblocks = kNumCU;
        }
        // The mixed-width grid (192-wide tiles in the last round) is built for this form too, but it does not
        // pay here: [4096,4096]x[4096,11008] takes 284.6 us with it and 285.6 us without - a last round
        // that leaves CUs idle runs at a higher clock under the power limit, and a 192-wide tile issues the
        // same fills as a 256-wide one.  Only MI355_GEMM_TILE=x16mixed selects it.
        if (nblocks > kNumCU && x16_mixed_forced) {
          const MixedPlan mp = plan_mixed(g.tiles_m, N);
          if (mp.narrow > 0) {
            g.tiles_n = mp.wide;
            g.tail_n = mp.narrow;
            nblocks = (int64_t)g.tiles_m * (mp.wide + mp.narrow);
            kern = gemm_x16_mixed_kernel(std::is_same<T, bf16_t>::value, !b_nt);
            form = "x16_mixed";
          }
        }
        // Output rows off the 128-byte lines: whole tile rows per store instruction (store_tile_rows16).
        g.out_rows = !persist && g.tail_n == 0 && (N % 64 != 0 || reinterpret_cast<uintptr_t>(out) % 128 != 0);
        if (!persist && g.tail_n == 0) warm_blocks = warm_for(nblocks, 1024);
      } else if (t64) {
        g.tiles_m = (int32_t)((M + TBM - 1) / TBM);
        g.tiles_n = (int32_t)((N + TBN - 1) / TBN);
        nblocks = nb64;
        threads = 256;
        if (t64_split) {
          nsplit = ts.nsplit;
          g.ws = static_cast<float*>(workspace);
          g.ksplit = ts.ksplit;
          g.ws_ld = (int32_t)((N + 3) / 4 * 4);
          if (ts.mode == 2) arm_insplit(nblocks, TBM);
        }
        const bool deep = nblocks * nsplit <= kNumCU;
        lds_bytes = (deep ? 8 : 4) * kTStage;
        form = deep ? "t64_ring8" : "t64_ring4";
        if (deep) warm_blocks = warm_for(nblocks, 1024);
        if (nsplit > 1 && meet_inside) {
          if (deep) kern = b_nt ? (const void*)gemm_mfma_t64_kernel<T, false, 8, 2> : (const void*)gemm_mfma_t64_kernel<T, true, 8, 2>;
          else kern = b_nt ? (const void*)gemm_mfma_t64_kernel<T, false, 4, 2> : (const void*)gemm_mfma_t64_kernel<T, true, 4, 2>;
        } else if (nsplit > 1) {
          if (deep) kern = b_nt ? (const void*)gemm_mfma_t64_kernel<T, false, 8, 1> : (const void*)gemm_mfma_t64_kernel<T, true, 8, 1>;
          else kern = b_nt ? (const void*)gemm_mfma_t64_kernel<T, false, 4, 1> : (const void*)gemm_mfma_t64_kernel<T, true, 4, 1>;
        } else {
          if (deep) kern = b_nt ? (const void*)gemm_mfma_t64_kernel<T, false, 8> : (const void*)gemm_mfma_t64_kernel<T, true, 8>;
          else kern = b_nt ? (const void*)gemm_mfma_t64_kernel<T, false, 4> : (const void*)gemm_mfma_t64_kernel<T, true, 4>;
        }
      } else if (mid) {
        g.tiles_n = (int32_t)((N + 127) / 128);
        nblocks = tiles_mid;
        kern = pick_w4(std::integral_constant<int, 2>{});
        form = "w4_256x128";
        threads = 256;
        lds_bytes = kGemmLds64;
        warm_blocks = warm_for(nblocks, 768);
        // (The 16x16x32 kernel on 256x128 tiles was measured for this slot: with half the MFMAs per fill and
        // per LDS read it is level with this form on a transposed b and 10 % behind on a row-major one.)
      } else if (!ktail && nblocks < kNumCU * 3 / 4) {  // 128x128 tiles, two workgroups per CU
        g.tiles_m = (int32_t)((M + SBM - 1) / SBM);
        g.tiles_n = (int32_t)((N + SBN - 1) / SBN);
        nblocks = (int64_t)g.tiles_m * g.tiles_n;
        const SplitPlan sp = plan_splitk(M, N, K, sizeof(T));
        const int64_t ws_ld = (N + 3) / 4 * 4;
        // Two parts of K on exactly one round of workgroups (128 tiles x 2) leave no CU for warm_operands and meet
        // while every CU is busy: with both operands K-contiguous the unsplit launch with its 32 warming workgroups
        // is ahead up to K = 2048 ([512,2048]x[4096,2048]^T 21.2 -> 19.3 us, [1024,2048]x[2048,2048]^T 20.4 -> 19.0,
        // [2048,2048]x[1024,2048]^T 21.0 -> 19.0), level at 3072 and behind from 4096 on; a row-major b is 6 % ahead
        // with the split at K = 2048 already, and so are two rows of tiles against a wide b, which is streamed
        // more than multiplied ([256,2048]x[8192,2048]^T 23.1 us split, 23.9 unsplit).
        const bool full_round_nt = b_nt && !a_t && sp.nsplit == 2 && nblocks * 2 >= kNumCU && K <= 2048 && K % 64 == 0 && M >= 512;
        const bool split = sp.nsplit > 1 && !full_round_nt && workspace != nullptr &&
                           workspace_bytes >= split_ws_bytes(sp, M, N, SBM) && reinterpret_cast<uintptr_t>(workspace) % 16 == 0;
        if (split) {
          nsplit = sp.nsplit;
          g.ws = static_cast<float*>(workspace);
          g.ksplit = sp.ksplit;
          g.ws_ld = (int32_t)ws_ld;
          if (sp.mode == 2) arm_insplit(nblocks, SBM);
        }
        // At most one workgroup per CU and whole 64-k pairs per split: the deep-ring kernel.
        const bool pairs = nblocks * nsplit <= kNumCU && K % 64 == 0 && (!split || sp.ksplit % 64 == 0);
        lds_bytes = pairs ? kSmall2Lds : kSmallLds;
        using M0 = std::integral_constant<int, 0>;
        using M1 = std::integral_constant<int, 1>;
        using M2 = std::integral_constant<int, 2>;
        if (pairs) kern = !split ? pick_small(std::true_type{}, M0{}) : meet_inside ? pick_small(std::true_type{}, M2{}) : pick_small(std::true_type{}, M1{});
        else kern = !split ? pick_small(std::false_type{}, M0{}) : meet_inside ? pick_small(std::false_type{}, M2{}) : pick_small(std::false_type{}, M1{});
        threads = pairs && !four_wave_ring ? 512 : 256;  // the deep-ring kernel: four computing waves and four loaders
        form = !pairs ? "small_128x128" : four_wave_ring ? "ring4_128x128" : "ring8_128x128";
        // CUs without a tile warm the last-level cache for the others (warm_operands): the deep-ring kernels only,
        // a K loop of 16 stages and more.  gemm_prefetch = N forces that many workgroups per part (a measurement knob).
        if (pairs) warm_blocks = warm_for(nblocks, 1024);
      } else if (ktail) {
        kern = b_nt ? (const void*)gemm_mfma_kernel<T, false, true> : (const void*)gemm_mfma_kernel<T, true, true>;
        form = "ktail_256x256";
      } else if (K % 64 == 0) {
        // Four waves of 128x128 run the steady state 3-5 % faster and pay ~2 us more per tile
        // (two-pass epilogue), which evens out near K = 2048.  MI355_GEMM_WAVES=4|8 forces one form.
        const char* forced = forced_waves;
        const bool w4 = a_t || (ld32 && (forced != nullptr ? forced[0] == '4' : K >= 2048));  // the eight-wave kernels have no M-contiguous-A form
        lds_bytes = kGemmLds64;
        if (w4) {
          kern = pick_w4(std::integral_constant<int, 4>{});
          form = "w4_256x256";
          threads = 256;
          // More than one round of tiles with a ragged last round: cut the last columns into 192-wide tiles.
          const bool plain = forced_tile != nullptr && strcmp(forced_tile, "256x256") == 0;
          const bool force_mixed = forced_tile != nullptr && strcmp(forced_tile, "mixed") == 0;  // any K (a test knob)
          if (nblocks > kNumCU && !plain && (K >= kMixedMinK || force_mixed)) {
            const MixedPlan mp = plan_mixed(g.tiles_m, N);
            if (mp.narrow > 0) {
              g.tiles_n = mp.wide;
              g.tail_n = mp.narrow;
              nblocks = (int64_t)g.tiles_m * (mp.wide + mp.narrow);
              form = "w4_mixed";
              if (a_t) kern = b_nt ? (const void*)gemm_mfma_w4_mixed_kernel<T, false, true> : (const void*)gemm_mfma_w4_mixed_kernel<T, true, true>;
              else kern = b_nt ? (const void*)gemm_mfma_w4_mixed_kernel<T, false, false> : (const void*)gemm_mfma_w4_mixed_kernel<T, true, false>;
            }
          }
        } else {
          kern = b_nt ? (const void*)gemm_mfma_dma64_kernel<T, false> : (const void*)gemm_mfma_dma64_kernel<T, true>;
          form = "dma64_256x256";
        }
      } else {
        kern = b_nt ? (const void*)gemm_mfma_dma_kernel<T, false> : (const void*)gemm_mfma_dma_kernel<T, true>;
        form = "dma32_256x256";
      }
      if (g_plan_text != nullptr)
        return describe_plan(form, g.tiles_m, g.tiles_n + g.tail_n, nblocks + warm_blocks, nsplit, threads, lds_bytes,
                             x16_split ? xs.splits : nsplit, x16_split || meet_inside ? "inside" : nsplit > 1 ? "launch" : "none", warm_blocks);
      // More than 64 KB of dynamic LDS needs the attribute once per kernel and process.
      static thread_local const void* attr_done[64] = {};
      bool seen = false;
      for (const void* k : attr_done) seen = seen || k == kern;
      if (!seen) {
        hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
        if (e != hipSuccess)
          return set_error(MI355_ERR_LAUNCH, "mi355_gemm: cannot reserve %d bytes of LDS: %s", lds_bytes, hipGetErrorString(e));
        for (const void*& k : attr_done)
          if (k == nullptr) { k = kern; break; }
      }
#ifdef MI355_GEMM_TRACE
      if (nsplit == 1) g.ws = workspace_bytes >= nblocks * 4 * 16 * 8 ? static_cast<float*>(workspace) : nullptr;
#endif
      void* params[] = {&g};
      hipError_t e = hipLaunchKernel(kern, dim3((unsigned)(nblocks + warm_blocks), (unsigned)nsplit), dim3(threads), params, lds_bytes, st);
      if (e != hipSuccess) return set_error(MI355_ERR_LAUNCH, "mi355_gemm(mfma): launch failed: %s", hipGetErrorString(e));
      const int rc = check_launch("mi355_gemm(mfma)");
      if (rc || nsplit == 1 || meet_inside) return rc;
      return finish_splitk<T>(g, nsplit, st);
    }
  }
  if constexpr (std::is_same<T, float>::value) {
    const bool a_ok = a_cs == 1 && a_rs % 4 == 0 && aligned16(a);
    const bool b_nt = b_rs == 1 && b_cs % 4 == 0 && aligned16(b);
    const bool b_nn = b_cs == 1 && b_rs % 4 == 0 && aligned16(b);
    const bool fits = M < (1 << 30) && N < (1 << 30) && K < (1 << 30);
    const bool b_nn_ok = b_nn && N % 4 == 0;
    if (a_ok && (b_nt || b_nn_ok) && K % FBK == 0 && K > 0 && fits && (M * N >= 32 * 32 || K >= 256 || M * N * K >= (int64_t(1) << 22))) {
      GemmArgs g{};
      g.a = a; g.b = b; g.c = c; g.out = out;
      g.lda = a_rs;
      g.ldb = b_nt ? b_cs : b_rs;
      g.c_rs = c_rs; g.c_cs = c_cs;
      g.out_vec = N % 4 == 0 && aligned16(out);
      g.M = (int32_t)M; g.N = (int32_t)N; g.K = (int32_t)K;
      g.alpha = (float)alpha; g.beta = (float)beta;
      const int tile = f32_tile(M, N);
      g.tiles_m = (int32_t)((M + tile - 1) / tile);
      g.tiles_n = (int32_t)((N + tile - 1) / tile);
      const int64_t nblocks = (int64_t)g.tiles_m * g.tiles_n;
      MI355_REQUIRE(nblocks < (int64_t(1) << 31), "mi355_gemm: too many tiles");
      int nsplit = 1;
      const SplitPlan sp = plan_splitk(M, N, K, 4);
      const int64_t ws_ld = (N + 3) / 4 * 4;
      if (sp.nsplit > 1 && workspace != nullptr && workspace_bytes >= (int64_t)sp.nsplit * M * ws_ld * 4 &&
          reinterpret_cast<uintptr_t>(workspace) % 16 == 0) {
        nsplit = sp.nsplit;
        g.ws = static_cast<float*>(workspace);
        g.ksplit = sp.ksplit;
        g.ws_ld = (int32_t)ws_ld;
      }
      // 64x64 tiles: eight 8 KB stages (64 KB, two workgroups per CU).  128x128 tiles: four 16 KB
      // stages, or eight when a CU gets one workgroup anyway and the deeper ring hides the fills.
      const void* kern;
      const bool deep = nblocks * nsplit <= kNumCU;
      const int lds_bytes = tile == 64 ? 8 * 8192 : deep ? 8 * kSStage : kSmallLds;
#define MI355_F32_KERNEL(S_, TILE_)                                                                              \
  (nsplit > 1 ? (b_nt ? (const void*)gemm_mfma_f32_kernel<false, true, S_, TILE_> : (const void*)gemm_mfma_f32_kernel<true, true, S_, TILE_>) \
              : (b_nt ? (const void*)gemm_mfma_f32_kernel<false, false, S_, TILE_> : (const void*)gemm_mfma_f32_kernel<true, false, S_, TILE_>))
      if (tile == 64) kern = MI355_F32_KERNEL(8, 64);
      else if (deep) kern = MI355_F32_KERNEL(8, 128);
      else kern = MI355_F32_KERNEL(kStages3, 128);
#undef MI355_F32_KERNEL
      if (g_plan_text != nullptr)
        return describe_plan(tile == 64 ? "f32_64x64" : deep ? "f32_128x128_ring8" : "f32_128x128_ring4", g.tiles_m, g.tiles_n, nblocks, nsplit,
                             256, lds_bytes, nsplit, nsplit > 1 ? "launch" : "none", 0);
      static thread_local const void* attr_done[12] = {};
      bool seen = false;
      for (const void* k : attr_done) seen = seen || k == kern;
      if (!seen) {
        hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
        if (e != hipSuccess)
          return set_error(MI355_ERR_LAUNCH, "mi355_gemm: cannot reserve %d bytes of LDS: %s", lds_bytes, hipGetErrorString(e));
        for (const void*& k : attr_done)
          if (k == nullptr) { k = kern; break; }
      }
      void* params[] = {&g};
      hipError_t e = hipLaunchKernel(kern, dim3((unsigned)nblocks, (unsigned)nsplit), dim3(256), params, lds_bytes, st);
      if (e != hipSuccess) return set_error(MI355_ERR_LAUNCH, "mi355_gemm(mfma f32): launch failed: %s", hipGetErrorString(e));
      const int rc = check_launch("mi355_gemm(mfma f32)");
      if (rc || nsplit == 1) return rc;
      return finish_splitk<float>(g, nsplit, st);
    }
  }
  if (g_plan_text != nullptr)
    return describe_plan(std::is_same<T, double>::value ? "f64_mfma" : "generic", 0, 0, 0, 1, 256, 0, 1, "none", 0);
  if constexpr (std::is_same<T, double>::value) {  // fp64: the MFMA kernel of gemm_f64.hip
    return launch_gemm_f64(static_cast<const double*>(a), a_rs, a_cs, static_cast<const double*>(b), b_rs, b_cs,
                           static_cast<const double*>(c), c_rs, c_cs, static_cast<double*>(out), M, N, K, alpha, beta, st);
  } else {
    // 128x128 tiles once they still give every CU a block, else 64x64
    const bool big = ((M + 127) / 128) * ((N + 127) / 128) >= kNumCU && K >= 64;
    const int64_t gt = big ? 128 : 64;
    const int64_t gx = (N + gt - 1) / gt, gy = (M + gt - 1) / gt;
    MI355_REQUIRE(gy < 65536 && gx < (int64_t(1) << 31), "mi355_gemm: generic path needs M < 4M rows");
    if (big)
      hipLaunchKernelGGL((gemm_generic_kernel<T, 8>), dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, st,
                         static_cast<const T*>(a), a_rs, a_cs, static_cast<const T*>(b), b_rs, b_cs,
                         static_cast<const T*>(c), c_rs, c_cs, static_cast<T*>(out), M, N, K, (float)alpha, (float)beta);
    else
      hipLaunchKernelGGL((gemm_generic_kernel<T, 4>), dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, st,
                         static_cast<const T*>(a), a_rs, a_cs, static_cast<const T*>(b), b_rs, b_cs,
                         static_cast<const T*>(c), c_rs, c_cs, static_cast<T*>(out), M, N, K, (float)alpha, (float)beta);
    return check_launch("mi355_gemm(generic)");
  }
}


// out (fp32) = alpha * ws + beta * c in place over a dense [M, N] fp32 matrix, N % 4 == 0 (mm.dtype / addmm.dtype:
// the 128x128 kernels' SPLIT form has left the raw fp32 product in `out` itself).
template <typename T>
__global__ __launch_bounds__(256) void gemm_f32out_finish_kernel(GemmArgs g) {
  const int64_t quads = (int64_t)g.M * g.N / 4;
  const int qpr = g.N / 4;
  const T* C = static_cast<const T*>(g.c);
  const bool use_c = C != nullptr && g.beta != 0.f;
  float* D = static_cast<float*>(g.out);
  for (int64_t qd = (int64_t)blockIdx.x * 256 + threadIdx.x; qd < quads; qd += (int64_t)gridDim.x * 256) {
    f32x4 v = *reinterpret_cast<const f32x4*>(D + qd * 4);
    const int64_t m = qd / qpr, n = (qd - m * qpr) * 4;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float r = g.alpha * v[e];
      if (use_c) r += g.beta * static_cast<float>(C[m * g.c_rs + (n + e) * g.c_cs]);
      v[e] = r;
    }
    *reinterpret_cast<f32x4*>(D + qd * 4) = v;
  }
}

// bf16 / f16 operands, fp32 result: the 128x128 MFMA kernels in their SPLIT form with a single split whose
// "plane" is the output itself - the fp32 accumulators go to memory as they are, never rounded to T.
template <typename T>
static int run_gemm_f32out(const void* a, int64_t a_rs, int64_t a_cs, const void* b, int64_t b_rs, int64_t b_cs, const void* c,
                           int64_t c_rs, int64_t c_cs, float* out, int64_t M, int64_t N, int64_t K, double alpha, double beta,
                           hipStream_t st) {
  const bool a_ok = a_cs == 1 && a_rs % 8 == 0 && aligned16(a);
  const bool b_nt = b_rs == 1 && b_cs % 8 == 0 && aligned16(b);
  const bool b_nn = b_cs == 1 && b_rs % 8 == 0 && aligned16(b) && N % 8 == 0;
  const bool fits = M < (1 << 30) && N < (1 << 30) && K < (1 << 30);
  if (!(a_ok && (b_nt || b_nn) && K > 0 && K % BK3 == 0 && N % 4 == 0 && aligned16(out) && fits))
    return set_error(MI355_ERR_UNSUPPORTED,
                     "mi355_gemm_f32out: layout not taken (needs K-contiguous a, b K-contiguous or row-major with N %% 8 == 0, "
                     "K %% 32 == 0, N %% 4 == 0, 16-byte aligned bases): widen the operands and call mi355_gemm in f32");
  GemmArgs g{};
  g.a = a; g.b = b; g.c = c; g.out = out;
  g.lda = a_rs;
  g.ldb = b_nt ? b_cs : b_rs;
  g.c_rs = c_rs; g.c_cs = c_cs;
  g.M = (int32_t)M; g.N = (int32_t)N; g.K = (int32_t)K;
  g.alpha = (float)alpha; g.beta = (float)beta;
  g.tiles_m = (int32_t)((M + SBM - 1) / SBM);
  g.tiles_n = (int32_t)((N + SBN - 1) / SBN);
  const int64_t nblocks = (int64_t)g.tiles_m * g.tiles_n;
  MI355_REQUIRE(nblocks < (int64_t(1) << 31), "mi355_gemm_f32out: too many tiles");
  g.ws = out;
  g.ksplit = (int32_t)K;
  g.ws_ld = (int32_t)N;
  const bool pairs = nblocks <= kNumCU && K % 64 == 0;  // at most one workgroup per CU: the deep-ring kernel
  const int lds_bytes = pairs ? kSmall2Lds : kSmallLds;
  const void* kern;
  if (pairs) kern = b_nt ? (const void*)gemm_mfma_small2_kernel<T, false, 1, false> : (const void*)gemm_mfma_small3_kernel<T, true, 1, false>;  // (loader waves for a row-major b)
  else kern = b_nt ? (const void*)gemm_mfma_small_kernel<T, false, 1, false> : (const void*)gemm_mfma_small_kernel<T, true, 1, false>;
  hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
  if (e != hipSuccess)
    return set_error(MI355_ERR_LAUNCH, "mi355_gemm_f32out: cannot reserve %d bytes of LDS: %s", lds_bytes, hipGetErrorString(e));
  void* params[] = {&g};
  e = hipLaunchKernel(kern, dim3((unsigned)nblocks, 1), dim3(pairs && !b_nt ? 512 : 256), params, lds_bytes, st);
  if (e != hipSuccess) return set_error(MI355_ERR_LAUNCH, "mi355_gemm_f32out: launch failed: %s", hipGetErrorString(e));
  int rc = check_launch("mi355_gemm_f32out");
  if (rc) return rc;
  if (alpha != 1.0 || (c != nullptr && beta != 0.0)) {
    const int grid = grid_for(M * N / 4, 256, kNumCU * 8);
    hipLaunchKernelGGL((gemm_f32out_finish_kernel<T>), dim3(grid), dim3(256), 0, st, g);
    rc = check_launch("mi355_gemm_f32out(finish)");
  }
  return rc;
}

}  // namespace mi355

using namespace mi355;

extern "C" int64_t mi355_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int dtype) {
  const int es = dtype_size(dtype);
  if (M <= 0 || N <= 0 || K <= 0 || (es != 2 && es != 4)) return 0;
  if (dtype != MI355_BF16 && dtype != MI355_F16 && dtype != MI355_F32) return 0;
  const SplitPlan p = plan_splitk(M, N, K, es);
  int64_t two_launch = split_ws_bytes(p, M, N, es == 4 ? f32_tile(M, N) : SBM);  // (either way of meeting)
  if (es == 2) {  // the 64x64-tile kernel's own split
    const int64_t t64 = split_ws_bytes(plan_t64_split(M, N, K), M, N, TBM);
    two_launch = t64 > two_launch ? t64 : two_launch;
  }
  const int64_t one_launch = es == 2 ? plan_x16_split(M, N, K).ws_bytes : 0;
  return two_launch > one_launch ? two_launch : one_launch;
}

extern "C" int mi355_gemm_tile_columns(int64_t M, int64_t N, int64_t K, int32_t* wide, int32_t* narrow) {
  MI355_REQUIRE(M > 0 && N > 0 && wide != nullptr && narrow != nullptr, "mi355_gemm_tile_columns: bad argument");
  const int64_t tiles_m = (M + BM - 1) / BM;
  MixedPlan mp{(int)((N + BN - 1) / BN), 0};
  if (tiles_m * mp.wide > kNumCU && K >= kMixedMinK) mp = plan_mixed(tiles_m, N);
  *wide = mp.wide;
  *narrow = mp.narrow;
  return MI355_OK;
}

extern "C" int mi355_gemm(const void* a, int64_t a_rs, int64_t a_cs, const void* b, int64_t b_rs, int64_t b_cs,
                          const void* c, int64_t c_rs, int64_t c_cs, void* out, int64_t M, int64_t N, int64_t K,
                          double alpha, double beta, int dtype, void* workspace, int64_t workspace_bytes,
                          void* stream) {
  MI355_REQUIRE(M >= 0 && N >= 0 && K >= 0, "mi355_gemm: negative extent");
  if (M == 0 || N == 0) return MI355_OK;
  MI355_REQUIRE(out != nullptr, "mi355_gemm: NULL out");
  MI355_REQUIRE(K == 0 || (a != nullptr && b != nullptr), "mi355_gemm: NULL operand");
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case MI355_BF16: return run_gemm<bf16_t>(a, a_rs, a_cs, b, b_rs, b_cs, c, c_rs, c_cs, out, M, N, K, alpha, beta, workspace, workspace_bytes, st);
    case MI355_F16: return run_gemm<f16_t>(a, a_rs, a_cs, b, b_rs, b_cs, c, c_rs, c_cs, out, M, N, K, alpha, beta, workspace, workspace_bytes, st);
    case MI355_F32: return run_gemm<float>(a, a_rs, a_cs, b, b_rs, b_cs, c, c_rs, c_cs, out, M, N, K, alpha, beta, workspace, workspace_bytes, st);
    case MI355_F64: return run_gemm<double>(a, a_rs, a_cs, b, b_rs, b_cs, c, c_rs, c_cs, out, M, N, K, alpha, beta, workspace, workspace_bytes, st);
    default: return set_error(MI355_ERR_UNSUPPORTED, "mi355_gemm: unsupported dtype %s", dtype_name(dtype));
  }
}

extern "C" int mi355_gemm_plan(int64_t M, int64_t N, int64_t K, int dtype, int64_t a_rs, int64_t a_cs, int64_t b_rs, int64_t b_cs,
                               int with_workspace, char* text, int64_t text_bytes) {
  MI355_REQUIRE(M > 0 && N > 0 && K >= 0 && text != nullptr && text_bytes >= 128, "mi355_gemm_plan: bad argument");
  // Operand addresses only enter the plan through their alignment: 16-byte aligned stand-ins, never dereferenced.
  void* const fake = reinterpret_cast<void*>(uintptr_t(1) << 20);
  void* const ws = with_workspace ? fake : nullptr;
  const int64_t ws_bytes = with_workspace ? (int64_t(1) << 60) : 0;
  text[0] = 0;
  g_plan_text = text;
  g_plan_cap = text_bytes;
  int rc;
  switch (dtype) {
    case MI355_BF16: rc = run_gemm<bf16_t>(fake, a_rs, a_cs, fake, b_rs, b_cs, nullptr, 0, 0, fake, M, N, K, 1.0, 0.0, ws, ws_bytes, nullptr); break;
    case MI355_F16: rc = run_gemm<f16_t>(fake, a_rs, a_cs, fake, b_rs, b_cs, nullptr, 0, 0, fake, M, N, K, 1.0, 0.0, ws, ws_bytes, nullptr); break;
    case MI355_F32: rc = run_gemm<float>(fake, a_rs, a_cs, fake, b_rs, b_cs, nullptr, 0, 0, fake, M, N, K, 1.0, 0.0, ws, ws_bytes, nullptr); break;
    case MI355_F64: rc = run_gemm<double>(fake, a_rs, a_cs, fake, b_rs, b_cs, nullptr, 0, 0, fake, M, N, K, 1.0, 0.0, ws, ws_bytes, nullptr); break;
    default: rc = set_error(MI355_ERR_UNSUPPORTED, "mi355_gemm_plan: unsupported dtype %s", dtype_name(dtype));
  }
  g_plan_text = nullptr;
  return rc;
}

extern "C" int mi355_gemm_f32out(const void* a, int64_t a_rs, int64_t a_cs, const void* b, int64_t b_rs, int64_t b_cs,
                                 const void* c, int64_t c_rs, int64_t c_cs, void* out, int64_t M, int64_t N, int64_t K,
                                 double alpha, double beta, int dtype, void* stream) {
  MI355_REQUIRE(M >= 0 && N >= 0 && K >= 0, "mi355_gemm_f32out: negative extent");
  if (M == 0 || N == 0) return MI355_OK;
  MI355_REQUIRE(out != nullptr, "mi355_gemm_f32out: NULL out");
  MI355_REQUIRE(K == 0 || (a != nullptr && b != nullptr), "mi355_gemm_f32out: NULL operand");
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case MI355_BF16: return run_gemm_f32out<bf16_t>(a, a_rs, a_cs, b, b_rs, b_cs, c, c_rs, c_cs, static_cast<float*>(out), M, N, K, alpha, beta, st);
    case MI355_F16: return run_gemm_f32out<f16_t>(a, a_rs, a_cs, b, b_rs, b_cs, c, c_rs, c_cs, static_cast<float*>(out), M, N, K, alpha, beta, st);
    default: return set_error(MI355_ERR_UNSUPPORTED, "mi355_gemm_f32out: operands must be bf16 or f16, got %s", dtype_name(dtype));
  }
}
