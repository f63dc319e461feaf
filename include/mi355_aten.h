/*
 * mi355_aten.h — C ABI of libmi355_aten.so: hand-written HIP kernels (gfx950 / MI355X)
 * for the core ATen operator set of a BackendBench directory backend.
 *
 * What each entry point replaces in the reference (meta-pytorch/BackendBench):
 * the reference holds no kernels.  It holds one *slot* per operator overload — the
 * module-level callable `<folder>_kernel_impl` that
 * BackendBench/backends/directory.py:74-100 loads from
 * `<ops_dir>/<folder>/<folder>_implementation*.py` and that
 * BackendBench/eval.py:102,186,195 (or the torch dispatcher after
 * BackendBench/__init__.py:70-101) calls with the ATen overload's arguments.
 * The Python wrappers in backendbench_amd/ops fill those slots; the functions below
 * are what those wrappers bind through ctypes.  Folder names are the ones
 * BackendBench/scripts/op_map.py lists (line cited per entry point).
 *
 * Conventions (all entry points):
 *   - every `void*` data pointer is a DEVICE pointer (tensor.data_ptr());
 *   - sizes and strides are in ELEMENTS, int64;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); kernels are
 *     only enqueued on it: no allocation, no synchronisation, no stream creation;
 *   - return 0 on success, a negative mi355_status otherwise; mi355_last_error()
 *     then returns a thread-local message.  Nothing is launched on error;
 *   - zero-element outputs return 0 without launching.
 */
#ifndef MI355_ATEN_H
#define MI355_ATEN_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355_ABI_VERSION 8
#define MI355_MAX_DIMS 8

typedef enum mi355_dtype {
  MI355_F32 = 0,
  MI355_F16 = 1,
  MI355_BF16 = 2,
  MI355_F64 = 3,
  MI355_I32 = 4,
  MI355_I64 = 5,
  MI355_I16 = 6,
  MI355_I8 = 7,
  MI355_U8 = 8,
  MI355_BOOL = 9,
  MI355_DTYPE_COUNT = 10
} mi355_dtype;

typedef enum mi355_status {
  MI355_OK = 0,
  MI355_ERR_INVALID = -1,     /* bad argument (shape, stride, null pointer, alignment) */
  MI355_ERR_UNSUPPORTED = -2, /* dtype / layout combination with no kernel            */
  MI355_ERR_LAUNCH = -3       /* hipLaunchKernel reported an error                    */
} mi355_status;

/* Strided view of device memory.  ndim <= MI355_MAX_DIMS; stride 0 = broadcast. */
typedef struct mi355_tensor {
  void* data;
  int32_t dtype; /* mi355_dtype */
  int32_t ndim;
  int64_t sizes[MI355_MAX_DIMS];
  int64_t strides[MI355_MAX_DIMS];
} mi355_tensor;

int mi355_abi_version(void);
const char* mi355_last_error(void);

/* Once per process and GPU, with that GPU current, before the first kernel call (the Python
 * binding does it on the first launch on a device).  No counterpart in the reference, which
 * holds no device code.  Checks that the device is a gfx950 part with the 256 compute units
 * the launch heuristics are sized for (persistent GEMM grids, split-K grids, streaming row
 * kernels) and refuses any other with MI355_ERR_UNSUPPORTED; resolves the address of the
 * built-in scratch array of mi355_reduce_static on this device, so that a later call of it
 * makes no runtime query (a caller may be recording a HIP graph by then). */
int mi355_init(void);

/* Test and measurement knobs; no counterpart in the reference.  The planner's choice of GEMM
 * kernel can be overridden so that a test reaches every kernel form on a shape of its choosing:
 *   "gemm_tile":  "x16" | "x16persist" | "x16split" | "x16split2" .. "x16split4" | "x16mixed" | "256x256" |
 *                 "mixed" | "256x128" | "128x128" | "64x64" | "ring4" | "ring8"  (initial value: the
 *                 environment's MI355_GEMM_TILE; ring4 / ring8: the four- / eight-wave form of the 128x128
 *                 deep-ring kernel on any layout)
 *   "gemm_waves": "4" | "8"                  (initial value: MI355_GEMM_WAVES)
 *   "gemm_split": "launch2" | "inlaunch"     how the parts of a K split over several workgroups of the
 *                 128x128- and 64x64-tile kernels meet: in a summing launch, or inside the one launch
 *                 (the planner picks per shape)
 *   "gemm_prefetch": "0" .. "256"  workgroups per part of K that only read the operands ahead of the tiles, on
 *                 CUs a launch of one workgroup per CU leaves without a tile (cut down to the CUs left over;
 *                 unset: up to 32 where 16 and more are left and the K loop is long enough)
 *   "x16_spin_limit": polls of the in-launch split-K's bounded wait for a partial product
 *                 before it gives up (default 2^21, about two seconds); a test sets it to 0
 *                 to walk the give-up path while every kernel still runs to its end.
 * value NULL or "" restores the default.  The environment is read once, at the first call
 * of any entry point that looks at a knob; afterwards only this function changes them.
 * Not thread-safe against concurrent mi355_gemm calls. */
int mi355_set_knob(const char* name, const char* value);

/* ---- elementwise -------------------------------------------------------------- */

typedef enum mi355_binary_op {
  MI355_ADD = 0,
  MI355_MUL = 1,
  MI355_MAXIMUM = 2,
  MI355_MINIMUM = 3
} mi355_binary_op;

/* out = a (op) b with a, b already broadcast to out's shape (stride 0 where expanded)
 * and already of out's dtype (one exception, ATen's type promotion done in registers: for
 * MI355_ADD / MI355_MUL into fp32, one of a, b may be f16 or bf16 while the other is fp32).
 * MI355_ADD computes a + alpha*b (alpha_f for floating
 * dtypes, alpha_i for integer dtypes).  MI355_MAXIMUM / MI355_MINIMUM propagate NaN.
 * `out` may be `a` itself (in-place overloads).
 * Slots: add__Tensor (op_map.py:266), mul__Tensor (op_map.py:749),
 * maximum__default (op_map.py:706), minimum__default (op_map.py:717); with both,
 * clamp__Tensor (op_map.py:372). */
int mi355_binary(int op, const mi355_tensor* a, const mi355_tensor* b, double alpha_f,
                 int64_t alpha_i, const mi355_tensor* out, void* stream);

typedef enum mi355_unary_op { MI355_RELU = 0, MI355_CLAMP = 1 } mi355_unary_op;

/* out = relu(x) or clamp(x, lo, hi); x has out's shape and dtype.  `bounds` bit 0 = lo
 * present, bit 1 = hi present.  NaN inputs stay NaN; lo > hi yields hi everywhere.
 * `out` may be `x` itself (in-place overloads).
 * Slots: relu__default (op_map.py:877), clamp__default (op_map.py:371),
 * clamp_min__default (op_map.py:369), clamp_max__default (op_map.py:367). */
int mi355_unary(int op, const mi355_tensor* x, int bounds, double lo_f, double hi_f,
                int64_t lo_i, int64_t hi_i, const mi355_tensor* out, void* stream);

/* out = cond ? a : b, bit-exact select.  cond is MI355_BOOL or MI355_U8; a, b have out's
 * dtype; all three already broadcast to out's shape.
 * Slot: where__self (op_map.py:1132). */
int mi355_where(const mi355_tensor* cond, const mi355_tensor* a, const mi355_tensor* b,
                const mi355_tensor* out, void* stream);

/* out = min(max(x, lo), hi) with tensor bounds, one pass; NaN in any operand propagates.  x, lo,
 * hi already broadcast to out's shape and of out's dtype.  A call with one bound only is
 * mi355_binary(MI355_MAXIMUM / MI355_MINIMUM).
 * Slot: clamp__Tensor (op_map.py:372). */
int mi355_clamp_tensor(const mi355_tensor* x, const mi355_tensor* lo, const mi355_tensor* hi,
                       const mi355_tensor* out, void* stream);

/* dst = (dst dtype) src, any strides on either side, same shape (src may broadcast).
 * Host-side helper for the slots above and below: type promotion and
 * making an operand dense without calling another ATen kernel. */
int mi355_copy(const mi355_tensor* src, const mi355_tensor* dst, void* stream);

/* ---- reductions ----------------------------------------------------------------- */

typedef enum mi355_reduce_op {
  MI355_SUM = 0,
  MI355_MEAN = 1,
  MI355_AMAX = 2,
  MI355_ARGMAX = 3
} mi355_reduce_op;

/* x is dense, viewed as [outer, red, inner]; reduces the middle axis; out is dense
 * [outer, inner].  Accumulates in fp32 (f16/bf16/f32), fp64 (f64) or int64 (integers).
 * out_dtype: x's dtype or the accumulation dtype for SUM/MEAN/AMAX; MI355_I64 for
 * ARGMAX (first index among equal maxima, NaN counts as the maximum).  red == 0 is the
 * caller's business (identity fill or error), not accepted here.  Few-row, long
 * reductions are split over the chip and combined in a second pass: when
 * mi355_reduce_workspace_bytes() is non-zero the caller passes that much device scratch
 * (contents undefined before and after).
 * Slots: sum__dim_IntList (op_map.py:1063), sum__default (:1061), mean__dim (:708),
 * mean__default (:707), amax__default (:282), argmax__default (:300). */
int64_t mi355_reduce_workspace_bytes(int op, int in_dtype, int64_t outer, int64_t red,
                                     int64_t inner);
int mi355_reduce(int op, const void* x, int in_dtype, int64_t outer, int64_t red,
                 int64_t inner, void* out, int out_dtype, void* workspace,
                 int64_t workspace_bytes, void* stream);

/* mi355_reduce for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.
 * Same arguments and results as mi355_reduce minus the workspace: the partial results of a
 * split reduction go to a buffer built into the library (one per GPU, mi355_reduce_static_max_bytes()
 * = 4 MiB, held until the process ends).  Calls no allocator.  A reduction whose
 * mi355_reduce_workspace_bytes() exceeds the buffer is refused with MI355_ERR_INVALID.
 * All calls on one GPU share that GPU's buffer: calls that may overlap in time on one GPU
 * (different streams, different threads) race; calls ordered on one stream do not. */
/* Under HIP graph capture call mi355_init() beforehand: the first mi355_reduce_static on a
 * device otherwise asks the runtime for the buffer's address (hipGetSymbolAddress). */
int64_t mi355_reduce_static_max_bytes(void);
int mi355_reduce_static(int op, const void* x, int in_dtype, int64_t outer, int64_t red,
                        int64_t inner, void* out, int out_dtype, void* stream);

/* Bytes of scratch mi355_softmax (over the last dim) and mi355_layer_norm can use for `rows` rows of
 * `n` elements of `dtype` (0 = none): a handful of very long rows (fewer than 64 rows of 32768
 * elements and more) are cut into chunks over the whole chip, with one partial state per (row,
 * chunk) in the scratch between the two launches of the call. */
int64_t mi355_row_workspace_bytes(int64_t rows, int64_t n, int dtype);

/* y = softmax (log_softmax != 0: log-softmax) over the middle axis of dense x viewed as
 * [outer, dim, inner]; fp32 math.  out_dtype = in_dtype, or MI355_F32 for half_to_float.
 * workspace: device memory, 8-byte aligned, of mi355_row_workspace_bytes(outer, dim, in_dtype)
 * bytes (only used when inner == 1), or NULL / smaller: then long rows take one block each.
 * Slots: _softmax__default (op_map.py:193), _log_softmax__default (op_map.py:151). */
int mi355_softmax(const void* x, int in_dtype, void* y, int out_dtype, int64_t outer,
                  int64_t dim, int64_t inner, int log_softmax, void* workspace,
                  int64_t workspace_bytes, void* stream);

/* Layer norm over the last N elements of each of M dense rows.  weight/bias may be NULL
 * and may differ in dtype from x (w_dtype).  mean/rstd are dense [M] in stat_dtype
 * (MI355_F32 or x's dtype).  Biased variance, rstd = 1/sqrt(var + eps).
 * workspace: as for mi355_softmax, mi355_row_workspace_bytes(M, N, dtype) bytes or NULL.
 * Slots: native_layer_norm__default (op_map.py:776), native_layer_norm__out. */
int mi355_layer_norm(const void* x, int dtype, const void* weight, const void* bias,
                     int w_dtype, void* y, void* mean, void* rstd, int stat_dtype,
                     int64_t M, int64_t N, double eps, void* workspace,
                     int64_t workspace_bytes, void* stream);

/* ---- matrix multiply -------------------------------------------------------------- */

/* Bytes of scratch mi355_gemm can use for a problem of this size and dtype (0 = none).  The
 * scratch holds fp32 partial products when a problem with few output tiles and a long K is
 * split along K over the chip (by a second, summing launch, or inside one launch whose
 * workgroups meet in the scratch through flag words kept there); it only has to live until the
 * kernels of that call have run, its contents are undefined before and after, and two calls
 * that may run at the same time must not share it. */
int64_t mi355_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int dtype);

/* out[M,N] = beta * c + alpha * (a[M,K] @ b[K,N]), fp32 accumulate, out dense row-major
 * in `dtype` (bf16 / f16 / f32 via MFMA).  a, b, c carry explicit (row, col) element
 * strides so transposed operands and a broadcast bias (c_rs = 0, c_cs = 1) need no copy.
 * c may be NULL (then beta is ignored); beta == 0 never reads c.  K == 0 is accepted.
 * Fast (MFMA) layouts, all with 16-byte aligned base and row starts: a with unit column stride,
 * or for bf16 / f16 with unit row stride (a transposed view) when K % 64 == 0 and M % 8 == 0;
 * b with unit row stride (weight.t()) or unit column stride with N a multiple of 8 (fp32: 4).
 * Any other strides run on a plain FMA kernel: correct, far slower.  f64 runs on its own MFMA kernel
 * (v_mfma_f64_16x16x4_f64) for any strides.
 * workspace: device memory, 16-byte aligned, of at least mi355_gemm_workspace_bytes() bytes,
 * or NULL / smaller — then the call is not split along K (same result, slower on skinny shapes).
 * Slots: mm__default (op_map.py:739), addmm__default (op_map.py:270). */
int mi355_gemm(const void* a, int64_t a_rs, int64_t a_cs, const void* b, int64_t b_rs,
               int64_t b_cs, const void* c, int64_t c_rs, int64_t c_cs, void* out,
               int64_t M, int64_t N, int64_t K, double alpha, double beta, int dtype,
               void* workspace, int64_t workspace_bytes, void* stream);

/* out[M,N] in FP32 (dense row-major) = beta * c + alpha * (a[M,K] @ b[K,N]) for bf16 / f16 a, b, c
 * (`dtype`): the fp32 accumulators are stored as they are, never rounded to the operand type.
 * Takes the MFMA layouts only - a with unit column stride, b with unit row stride or with unit
 * column stride and N % 8 == 0, K % 32 == 0, N % 4 == 0, 16-byte aligned bases and row starts -
 * and returns MI355_ERR_UNSUPPORTED without launching anything for every other problem: the
 * caller then widens a, b, c to fp32 (mi355_copy) and calls mi355_gemm with MI355_F32, which
 * computes the same sums of exact products.  No workspace.
 * Slots: mm__dtype (op_map.py:740), addmm__dtype (op_map.py:271) and their out= forms. */
int mi355_gemm_f32out(const void* a, int64_t a_rs, int64_t a_cs, const void* b, int64_t b_rs,
                      int64_t b_cs, const void* c, int64_t c_rs, int64_t c_cs, void* out,
                      int64_t M, int64_t N, int64_t K, double alpha, double beta, int dtype,
                      void* stream);

/* Reads and clears the sticky status word of the GEMM kernels; no counterpart in the reference.
 * A split-K launch whose summing workgroup ran out of polls (see "x16_spin_limit") fills its
 * output tile with NaNs and sets the word; mi355_gemm itself has long returned MI355_OK by then.
 * Returns MI355_ERR_LAUNCH with a message if the word was set since the last call, else 0.
 * Synchronous (two small copies from / to the device): synchronise the streams that ran GEMMs
 * first, and do not call it while a stream is being captured. */
int mi355_gemm_status(void);

/* How the large-tile bf16 / f16 kernel cuts the N columns of an [M, N] output (K a multiple of 64):
 * `wide` tile columns of 256 followed by `narrow` tile columns of 192.  narrow > 0 when K >= 4096,
 * the 256 x 256 tiles make more than one round over the 256 CUs, and cutting the last columns
 * narrower shortens the ragged last round.  Host-only planning query for tests and documentation;
 * no counterpart in the reference. */
int mi355_gemm_tile_columns(int64_t M, int64_t N, int64_t K, int32_t* wide, int32_t* narrow);

/* What mi355_gemm would launch for an [M, K] x [K, N] product of `dtype` with these operand strides
 * (elements; operands and output taken as 16-byte aligned, no c), with or without a workspace of any
 * size: one line of text, e.g.
 *   "form=ring4_128x128 tiles=12x16 grid=224x1 threads=256 lds=163840 parts=1 meet=none warm=32"
 * form  = the kernel form (x16, x16_persistent, x16_split, x16_mixed, w4_256x256, w4_mixed, w4_256x128,
 *         ring4_128x128, ring8_128x128, small_128x128, t64_ring8, t64_ring4, dma64_256x256, dma32_256x256,
 *         ktail_256x256, f32_64x64, f32_128x128_ring8, f32_128x128_ring4, f64_mfma, generic);
 * tiles = rows x columns of tiles; grid = workgroups per part x parts of K; parts / meet = how many
 * workgroups share a tile's K range and where they meet ("launch": a summing launch, "inside": in the
 * one launch); warm = cache-warming workgroups appended per part.  The test knobs apply.  Nothing is
 * launched and no device is touched: a host-only planning query for tests and documentation, with no
 * counterpart in the reference.  text_bytes >= 128. */
int mi355_gemm_plan(int64_t M, int64_t N, int64_t K, int dtype, int64_t a_rs, int64_t a_cs, int64_t b_rs,
                    int64_t b_cs, int with_workspace, char* text, int64_t text_bytes);

/* Measurement only, no counterpart in the reference: the matrix-core instruction stream of the
 * large-tile mm kernel (per wave a 128 x 128 fp32 register tile, 32 v_mfma_f32_32x32x16 per 32-k
 * step) with no memory traffic in the loop.  `blocks` workgroups of four waves run `steps` (a
 * multiple of four) steps on operand fragments loaded once from a and b (16 fragments of 16 bytes per thread each:
 * blocks * 65536 bytes; the caller chooses the data), out receives blocks * 256 floats.  Work:
 * blocks * 4 * steps * 2 * 128 * 128 * 32 flop.  variant 0: the mm kernel's operand order; 1: operands
 * swapped between the two ports; 2: the other operand held across MFMAs; 3: v_mfma_f32_16x16x32;
 * 4 / 5: 32x32x16 with the MFMAs on one accumulator block in chains of four / two; 6 - 9: 16x16x32 in
 * chains (whole tile / quadrant by quadrant in chains of 1, 2, 4); 10 - 14: the 16x16x32 stream of the
 * mm kernel in exactly the written order (asm statements): chains of two back to back (10), with one
 * (11) or three (14) s_nop between the two, two blocks interleaved (12), first halves then second halves (13).
 * Its sustained rate on a given data distribution is the ceiling the power / clock envelope leaves to
 * mi355_gemm on that data.
 * dtype MI355_F64: `variant` is the number of waves per workgroup (1, 4, 8 or 16), every wave issues
 * `steps` rounds of eight independent v_mfma_f64_16x16x4_f64 on one value per lane (a, b: 256 doubles
 * each): blocks * variant * steps * 8 * 2048 flop - how the issue rate of that instruction depends on
 * the waves per SIMD. */
int mi355_calib_mfma(const void* a, const void* b, void* out, int dtype, int blocks, int steps,
                     int variant, void* stream);

/* ---- indexing --------------------------------------------------------------------- */

/* src dense [outer, n_src, inner], out dense [outer, n_idx, inner]:
 * out[o, j, :] = src[o, index[j], :].  elem_size in bytes (1, 2, 4, 8); idx_dtype
 * MI355_I32 or MI355_I64; index dense.  An index outside [0, n_src) is never
 * dereferenced: the row is zero-filled and *err_flag (an int32 the device can write: device
 * memory or pinned host memory, may be NULL) is set to 1 — the host decides when to read it.
 * Slots: index_select__default (op_map.py:571), embedding__default (op_map.py:447). */
int mi355_index_select(const void* src, int elem_size, int64_t outer, int64_t n_src,
                       int64_t inner, const void* index, int idx_dtype, int64_t n_idx,
                       void* out, int32_t* err_flag, void* stream);

/* out[...] = src[..., index[...], ...] along `dim`; out dense with index's shape, index
 * MI355_I64 (any strides), src any strides, index.size(d) <= src.size(d) for d != dim.
 * Same out-of-range convention as mi355_index_select.
 * Slot: gather__default (op_map.py:510). */
int mi355_gather(const mi355_tensor* src, int dim, const mi355_tensor* index,
                 const mi355_tensor* out, int32_t* err_flag, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MI355_ATEN_H */
