// Types and helpers shared by the GEMM kernel sources (gemm.hip, gemm_x16.hip): the argument
// block, the block -> tile map, the transposing LDS read and the global -> LDS fill requests.
#pragma once
#include "common.h"

namespace mi355 {

constexpr int BM = 256, BN = 256;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct alignas(sizeof(T) * 4) VecN4 {
  T v[4];
};

typedef float f32x16 __attribute__((ext_vector_type(16)));

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
  int32_t tail_n;  // gemm_mfma_w4_mixed_kernel: 192-wide tile columns behind the tiles_n 256-wide ones
  int32_t c_vec;  // c is unit-stride along n with 8-byte aligned rows: read it as vectors
  int32_t out_vec;  // out rows start on 16-byte boundaries (N a multiple of the vector width): vector stores
  // Split-K (128x128 kernels only): blockIdx.y = split, which covers k in [split * ksplit,
  // min(K, (split + 1) * ksplit)) and writes its raw fp32 tile to ws[split][M][ws_ld], ws_ld = N
  // rounded up to a multiple of 4 (rows of every plane start on 16-byte boundaries for any N).
  float* ws;
  int32_t ksplit;
  int32_t ws_ld;
  int32_t out_rows;  // gemm_mfma_x16_kernel: out rows do not start on 128-byte lines (N % 64 != 0), stage whole tile rows
  int32_t bias_vec;  // c is one unit-stride row broadcast along m (a Linear layer's bias), 8-byte aligned: any N
  // gemm_mfma_x16_splitk_kernel: sk_splits workgroups share a tile's K range and meet in the caller's
  // workspace: (sk_splits - 1) fp32 planes of 256 x 256 per tile at ws, behind them one 64-bit flag per plane
  // (sk_flags), which holds sk_epoch (a value of this launch alone) once the plane is complete.
  int32_t sk_splits;
  int32_t sk_tiles8;  // tiles rounded up to a multiple of 8: blocks [r * sk_tiles8, (r + 1) * sk_tiles8) have one role
  unsigned long long sk_epoch;
  unsigned long long* sk_flags;
  int32_t sk_spin_limit;  // polls of a flag before the summing workgroup gives up (Knobs::x16_spin_limit)
};

// Tile id for this block: blocks land on XCD (blockIdx % 8); give each XCD a contiguous
// band of tile ids, then walk the band in groups of GROUP tile-rows so A and B panels repeat
// in that XCD's L2 (32 tiles of an XCD: 8 rows x 4 columns of square tiles; 256x128 tiles take 4 rows x 8
// columns, 1024 + 1024 operand rows per XCD instead of 2048 + 512).
template <int GROUP = 8>
__device__ __forceinline__ void tile_coords(const int tiles_m, const int tiles_n, int pid, int& tm, int& tn) {
  const int nblocks = tiles_m * tiles_n;
  const int per_xcd = (nblocks + kNumXCD - 1) / kNumXCD;
  const int full = nblocks % kNumXCD;  // XCDs that own `per_xcd` tiles when not divisible
  const int xcd = pid % kNumXCD, local = pid / kNumXCD;
  if (full == 0) pid = xcd * per_xcd + local;
  else pid = (xcd < full ? xcd * per_xcd : full * per_xcd + (xcd - full) * (per_xcd - 1)) + local;
  const int in_group = GROUP * tiles_n;
  const int group = pid / in_group;
  const int first_m = group * GROUP;
  const int rows = tiles_m - first_m < GROUP ? tiles_m - first_m : GROUP;
  tm = first_m + (pid % in_group) % rows;
  tn = (pid % in_group) / rows;
}
template <int GROUP = 8>
__device__ __forceinline__ void tile_coords(const GemmArgs& g, int& tm, int& tn) {
  tile_coords<GROUP>(g.tiles_m, g.tiles_n, blockIdx.x, tm, tn);
}

// Epilogue of the MFMA kernels for output rows that start at any 2-byte offset (N % 8 != 0: a 50257-wide
// vocabulary projection).  `slab` holds `rows` result rows of SLOTS 16-byte slots (8 SLOTS elements; slot s
// of row r at s ^ ((r / 2) % 8) for 128-byte rows, at s ^ (r % SLOTS) otherwise), of which the first `cols`
// columns go to D[m_first + row][n_first ...].  A store instruction costs the memory pipeline the same
// whether its lanes carry 2 or 16 bytes, so the lanes walk the 16-byte grid of the destination, not the
// columns: SLOTS lanes per row, lane s stores the s-th whole 16-byte unit that lies inside the row segment
// (its eight elements gathered from the two LDS slots they straddle), and the up to seven elements in front
// of the first unit and behind the last one go out as single elements (they share their 16-byte units with
// the neighbouring tiles' columns).
template <typename T, int ROWS, int SLOTS = 8>
__device__ __forceinline__ void store_slab_rows_shifted(const unsigned char* slab, T* D, int64_t N, int m_first, int rows,
                                                        int n_first, int cols, int lane) {
  constexpr int RPI = 64 / SLOTS;  // rows per store instruction
  static_assert(sizeof(T) == 2 && (SLOTS == 8 || SLOTS == 32) && ROWS % RPI == 0, "two-byte elements");
  if (cols <= 0) return;
  const int s = lane % SLOTS;
  const int s1 = s + 1 < SLOTS ? s + 1 : s;
#pragma unroll 2
  for (int t = 0; t < ROWS / RPI; ++t) {
    const int row = t * RPI + lane / SLOTS;
    const int x = SLOTS == 8 ? (row >> 1) & 7 : row & (SLOTS - 1);
    const unsigned char* rp = slab + row * (SLOTS * 16);
    // Unit s = elements head + 8 s .. + 7: the upper 8 - head elements of slot s and the lower head elements of
    // slot s + 1, read whole (16-byte reads: no bank conflicts) and shifted into place - by head / 2 dwords
    // through two rounds of selects, by head % 2 halves through v_alignbit.
    const u32x4 lo = *reinterpret_cast<const u32x4*>(rp + ((s ^ x) << 4));
    const u32x4 hi = *reinterpret_cast<const u32x4*>(rp + ((s1 ^ x) << 4));
    uint16_t* dst = reinterpret_cast<uint16_t*>(D) + ((int64_t)(m_first + row) * N + n_first);
    const int to_unit = (int)((16 - (reinterpret_cast<uintptr_t>(dst) & 15)) & 15) >> 1;  // elements up to the next 16-byte boundary
    const int head = row >= rows ? 0 : to_unit < cols ? to_unit : cols;
    const int nfull = row >= rows ? 0 : (cols - head) >> 3;
    const int tail0 = row >= rows ? cols : head + 8 * nfull;
    const bool q2 = (to_unit & 4) != 0, q1 = (to_unit & 2) != 0;
    const uint32_t a0 = q2 ? lo[2] : lo[0], a1 = q2 ? lo[3] : lo[1], a2 = q2 ? hi[0] : lo[2], a3 = q2 ? hi[1] : lo[3],
                   a4 = q2 ? hi[2] : hi[0], a5 = q2 ? hi[3] : hi[1];
    const uint32_t b0 = q1 ? a1 : a0, b1 = q1 ? a2 : a1, b2 = q1 ? a3 : a2, b3 = q1 ? a4 : a3, b4 = q1 ? a5 : a4;
    const uint32_t sh = (uint32_t)(to_unit & 1) * 16u;
    if (s < nfull) {
      u32x4 v;
      v[0] = __builtin_amdgcn_alignbit(b1, b0, sh);
      v[1] = __builtin_amdgcn_alignbit(b2, b1, sh);
      v[2] = __builtin_amdgcn_alignbit(b3, b2, sh);
      v[3] = __builtin_amdgcn_alignbit(b4, b3, sh);
      *reinterpret_cast<u32x4*>(dst + head + 8 * s) = v;
    }
    // The elements in front of the first unit are the first `head` of slot 0; those behind the last unit start
    // at element tail0 = head + 8 nfull, i.e. at position `head` of slot nfull: lane s of the row takes element
    // s of either run from the slots it has (lanes 0 and nfull hold them).
    const int e_tail = tail0 + s;
    if (s < head)
      dst[s] = *reinterpret_cast<const uint16_t*>(rp + ((0 ^ x) << 4) + (s << 1));
    if (e_tail < cols)
      dst[e_tail] = *reinterpret_cast<const uint16_t*>(rp + ((((e_tail >> 3) & (SLOTS - 1)) ^ x) << 4) + ((e_tail & 7) << 1));
  }
}

// Workgroups behind a launch's tiles (blockIdx.x >= tiles_m * tiles_n; the host adds them on CUs that would
// sit idle): they read one dword of every 128-byte line of both operands' k range [kbeg, kend), early k
// first, and leave.  A 128x128 workgroup keeps at most 128 KB of fills in flight, so with one workgroup per CU
// its K loop runs at fill latency: about 0.42 us per 64 k when the lines come from the last-level cache, 0.55
// and more from HBM.  These reads pull the operands into that cache well ahead of the tiles' own fills
// ([1536,4096]x[2048,4096]^T on inputs that no cache holds: 40 us without them).
constexpr int kWarmLoads = 64;  // lines a thread of a warming workgroup touches at most
template <typename T, bool A_T, bool B_NN>
__device__ __forceinline__ void warm_operands(const GemmArgs& g, int kbeg, int kend) {
  const int first = g.tiles_m * g.tiles_n;
  const int64_t nthreads = (int64_t)(gridDim.x - first) * blockDim.x;
  const int64_t me = (int64_t)(blockIdx.x - first) * blockDim.x + threadIdx.x;
  const T* A = static_cast<const T*>(g.a);
  const T* B = static_cast<const T*>(g.b);
  // Lines of one 64-k stage: a K-contiguous operand has one per row, a row-major one (M or N / 64) per k row.
  const int ca = (g.M + 63) / 64, cb = (g.N + 63) / 64;
  const int la = A_T ? 64 * ca : g.M, lb = B_NN ? 64 * cb : g.N;
  const int per_stage = la + lb;
  const int64_t total = (int64_t)((kend - kbeg) / 64) * per_stage;
  uint32_t sink = 0;
  // Sixteen loads in flight per thread, at most kWarmLoads per thread: a launch with few of these workgroups leaves
  // the late stages to the tiles' own fills rather than outlast the tiles.
  for (int64_t base = me; base < total && base < me + (kWarmLoads / 16) * 16 * nthreads; base += 16 * nthreads) {
    uint32_t v[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      int64_t i = base + u * nthreads;
      i = i < total ? i : total - 1;
      const int s = (int)(i / per_stage);
      int j = (int)(i - (int64_t)s * per_stage);
      const int64_t k0 = kbeg + 64 * (int64_t)s;
      const T* p;
      if (j < la) {
        if constexpr (A_T) p = A + (k0 + j / ca) * g.lda + (j % ca) * 64;
        else p = A + (int64_t)j * g.lda + k0;
      } else {
        j -= la;
        if constexpr (B_NN) p = B + (k0 + j / cb) * g.ldb + (j % cb) * 64;
        else p = B + (int64_t)j * g.ldb + k0;
      }
      v[u] = *reinterpret_cast<const uint32_t*>(p);
    }
#pragma unroll
    for (int u = 0; u < 16; ++u) sink ^= v[u];
  }
  // (never true: keeps the loads alive)
  if (sink == 0x5bd1e995u && g.M < 0) *reinterpret_cast<volatile uint32_t*>(g.out) = sink;
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

// global_load_lds_dwordx4: one wave-level load moves 64 x 16 bytes from global memory straight into
// 1 KB of LDS (lane l lands at M0 + 16 l) without passing through VGPRs.  Issued from inline asm: the
// compiler's wait-count bookkeeping does not see these loads, the kernels count them (s_waitcnt vmcnt).
__device__ __forceinline__ void lds_dma16(uint32_t lds_byte_offset, const void* gptr) {
  asm volatile("s_mov_b32 m0, %0\n\t"
               "s_nop 0\n\t"
               "global_load_lds_dwordx4 %1, off" ::"s"(lds_byte_offset), "v"(gptr)
               : "memory");
}

// The same fill with the address split into a uniform 64-bit base (SGPR pair) and a 32-bit byte
// offset per lane: the offsets of a wave's requests are loop invariants (one VGPR each instead of
// a pointer pair) and a k step only moves the scalar base.
__device__ __forceinline__ void lds_dma16s(uint32_t lds_byte_offset, uint32_t lane_byte_offset, const void* base) {
  asm volatile("s_mov_b32 m0, %0\n\t"
               "s_nop 0\n\t"
               "global_load_lds_dwordx4 %1, %2" ::"s"(lds_byte_offset), "v"(lane_byte_offset), "s"(base)
               : "memory");
}

// gemm_x16.hip: the 256x256-tile kernel on v_mfma_f32_16x16x32 (bf16 / f16, K % 128 == 0, K >= 256, K-contiguous
// a; b K-contiguous or row-major), its dynamic LDS size, and the host-side kernel handle.
constexpr int kX16Lds = 5 * 32768;
const void* gemm_x16_kernel(bool is_bf16, bool b_nn);
const void* gemm_x16_persistent_kernel(bool is_bf16, bool b_nn);  // one workgroup per CU walks the tiles (whole tiles, K >= 384)
const void* gemm_x16_mixed_kernel(bool is_bf16, bool b_nn);
const void* gemm_x16_splitk_kernel(bool is_bf16, bool b_nn);  // 2 - 4 workgroups per tile split K and meet in the workspace
constexpr int kX16SplitUnit = 128;        // K shares are multiples of this
// The summing workgroup's share of `units` K units among `splits` workgroups: an even share and, from eight units
// each on, one more - a unit takes about 2.2 us, a producer's plane store 3 us (host and device agree through this).
__host__ __device__ constexpr int x16_split_summing_units(int units, int splits) {
  return (units + splits - 1) / splits + (units >= 8 * splits ? 1 : 0);
}
  // 256-wide tile columns, then 192-wide ones (GemmArgs::tail_n)

// gemm.hip: the status word of the in-launch split K of the 128x128- and 64x64-tile kernels, read into *word and
// cleared when set; a HIP error code, 0 on success.
int read_insplit_status(unsigned int* word);

// gemm_f64.hip: fp64 products on v_mfma_f64_16x16x4_f64, any strides (c may be null).
int launch_gemm_f64(const double* a, int64_t a_rs, int64_t a_cs, const double* b, int64_t b_rs, int64_t b_cs, const double* c,
                    int64_t c_rs, int64_t c_cs, double* out, int64_t M, int64_t N, int64_t K, double alpha, double beta,
                    hipStream_t st);

}  // namespace mi355
