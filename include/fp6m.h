/*
 * fp6m.h -- C ABI of the MI355X (gfx950) mixed INT4 / FP6-e3m2 weight-only GEMM.
 *
 * Plain pointers and sizes only; no torch, no HIP types (a stream is passed as
 * the opaque `hipStream_t` pointer value).  Every entry point cites the
 * interface of liuchuan22/FP6-Marlin it replaces (paths relative to that
 * repository).  All functions return FP6M_OK (0) or one of the codes below and
 * never throw across the boundary.
 *
 * Matrix conventions (identical to the reference):
 *   A  [m, k] fp16 row-major, device
 *   C  [m, n] fp16 row-major, device, fully overwritten
 *   B  1-D int32, device:  INT4 words of columns [0, n-quant_cols)       (k * (n-quant_cols) / 8  words)
 *                       || FP6 "2-bit" words of the last quant_cols columns  (k * quant_cols / 16      words)
 *                       || FP6 "4-bit" words of the same columns             (k * quant_cols / 8       words)
 *      exactly what test.py:123-152 (gen_mixed_weight) concatenates.
 *   s  fp16, device: INT4 scales || FP6 scales.  Per-column scales are stored
 *      in the reference's permuted order (test.py:80-83); INT4 group scales
 *      (group_size = 128) are [k/128, n-quant_cols] in natural column order.
 */
#ifndef FP6M_H_
#define FP6M_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FP6M_OK              0
#define FP6M_ERR_PROB_SHAPE  1 /* fp6_marlin_cuda_kernel.cu:861  n or k not divisible by the tile   */
#define FP6M_ERR_KERN_SHAPE  2 /* fp6_marlin_cuda_kernel.cu:862  no kernel for (thread_k, thread_n) */
#define FP6M_ERR_RANGE       3 /* weight_quant.cpp:48-53 throws std::invalid_argument                */
#define FP6M_ERR_SHAPE       4 /* weight_quant.cpp:112, weight_prepacking.cpp:124-125,182-183, pybind.cpp:22-24,50 */
#define FP6M_ERR_ARG         5 /* null pointer, unsupported group_size / quant_cols                  */
#define FP6M_ERR_HIP         6 /* a HIP runtime call failed; fp6m_last_hip_error() has the code      */
#define FP6M_ERR_NO_GPU_CODE 7 /* the library was built without its gfx950 kernels                   */
#define FP6M_ERR_SCRATCH     8 /* partial sums do not fit fp6m_mul_static's scratch, or no room for another workspace's region */

/* Human-readable text for a return code (static storage). */
const char* fp6m_strerror(int code);
/* hipError_t of the most recent failing HIP call on this thread (0 if none). */
int fp6m_last_hip_error(void);
/* ABI version of this header: bumped on any incompatible change. */
int fp6m_abi_version(void);

/*
 * The GEMM.  Replaces
 *   int fp6_marlin_cuda(const void* A, const void* B, void* C, void* s, int prob_m, int prob_n,
 *                       int prob_k, void* workspace, int dev, cudaStream_t stream, int thread_k,
 *                       int thread_n, int sms, int max_par, int quant_cols)
 *   (fp6_marlin/fp6_marlin_cuda_kernel.cu:864-951, declared again fp6_marlin/fp6_marlin_cuda.cpp:26-42).
 *
 * Same argument order and meaning, plus `group_size` at the end:
 *   workspace   >= fp6m_workspace_elems(prob_n, max_par) 4-byte elements of device memory, all zero
 *               on entry; it is all zero again when the call's work has finished (same contract as
 *               the reference's lock array, fp6_marlin_cuda_kernel.cu:90-92).
 *   dev, stream device ordinal and hipStream_t; the call is asynchronous on `stream`.
 *   thread_k, thread_n  -1/-1 = automatic.  Otherwise validated exactly like the reference:
 *               (128,128) only for prob_m <= 16, (64,256) for any m; anything else -> ERR_KERN_SHAPE;
 *               prob_n % thread_n or prob_k % thread_k -> ERR_PROB_SHAPE.  They do not select a
 *               different kernel here (tile shapes are chosen for 256 CUs / wave64).
 *   sms         -1 = automatic; otherwise an upper bound on the number of workgroups that cooperate
 *               on one column tile's reduction (debug/testing knob, like the reference's).
 *   max_par     as in the reference: bounds how many 64-row blocks of A one launch covers.
 *   quant_cols  -1 (or 0) = all INT4; n = all FP6; otherwise the last quant_cols columns are FP6.
 *               Must be a multiple of 128, as must n - quant_cols.
 *   group_size  -1 = one INT4 scale per column (what the reference kernel supports);
 *               128 = one INT4 scale per 128 rows of k per column.  FP6 scales are always per column.
 * Zero-sized problems return FP6M_OK without launching (fp6_marlin_cuda_kernel.cu:906-907).
 */
int fp6m_mul(const void* A, const void* B, void* C, const void* s, int prob_m, int prob_n, int prob_k,
             void* workspace, int dev, void* stream, int thread_k, int thread_n, int sms, int max_par,
             int quant_cols, int group_size);

/*
 * fp6m_mul for callers that cannot allocate device memory (code under HIP-graph capture, tight serving loops,
 * harnesses that forbid it).  No counterpart in the reference.  Same arguments, results and return codes as
 * fp6m_mul, with these differences:
 *   - what column tiles shared by several workgroups are summed through (fp32 partial tiles for m > 16, 64-bit
 *     accumulate-and-count cells for m <= 16) lives in a 20 MiB array that is part of the library's device code (one
 *     copy per GPU, held until the process ends) instead of the workspace's region; the call allocates and frees
 *     nothing.  fp6m_init(dev) beforehand also keeps the one-time lookup of the device's properties and of the
 *     array's address out of the first call;
 *   - a launch of more than 16 rows whose k split needs more than the 12 MiB the array has for partial tiles returns
 *     FP6M_ERR_SCRATCH (fp6m_mul would shrink the split instead).  The need is (workgroups that share column tiles) x
 *     (32, 64 or 128 rows) x 128 columns x 4 bytes; the dispatcher sizes its own splits to the 12 MiB (it keeps 64-row
 *     tiles where a split of 128-row tiles would not fit), so this only triggers for splits forced with
 *     fp6m_tuning_set or on devices with more compute units.  Launches of up to 4 rows never fail this way (without
 *     room for their cells, n * m * 8 bytes > 8 MiB, no tile is shared); those of 5 to 16 rows only with a forced split;
 *   - every call on a GPU shares that GPU's array: calls that overlap on one GPU race, whatever their workspaces
 *     and streams.  `workspace` keeps its role (tile counters, zero on entry and on exit).
 */
int fp6m_mul_static(const void* A, const void* B, void* C, const void* s, int prob_m, int prob_n, int prob_k,
                    void* workspace, int dev, void* stream, int thread_k, int thread_n, int sms, int max_par,
                    int quant_cols, int group_size);

/*
 * The packed words in the order this GPU's kernels would choose, next to the reference's.  Same bits; what moves is
 * the 16-byte (4-bit plane, INT4 words) or 8-byte (2-bit plane) granule that one lane consumes per k-block of 16 rows:
 *   reference  [k-block][64-column group g][fragment owner t = 4 l + i]          (weight_prepacking.cpp:123-177,
 *              test.py:60-79: mma.m16n8k16 lane order, a tile's k-blocks a whole matrix row apart)
 *   gfx950     [128-column tile][k-block][MFMA lane 16 i + 8 (g & 1) + l]        (v_mfma_f32_16x16x32_f16 operand
 *              order: a tile's packed words form one sequential stream and lanes read them in lane order)
 * fp6m_repack_gfx950 converts a whole B buffer (INT4 words || FP6 2-bit plane || FP6 4-bit plane; the column mix of
 * fp6m_mul when quant_rows == 0, else the row mix of fp6m_mul_rows with quant_cols ignored) either way on the host;
 * to_gfx950 = 0 is the exact inverse.  Scales are not affected.  Column counts of each region must be multiples of 128,
 * row counts multiples of 16 -> else FP6M_ERR_SHAPE.  in and out must not overlap.
 */
#define FP6M_LAYOUT_GFX950 1
int fp6m_repack_gfx950(const int32_t* in, int32_t* out, size_t k, size_t n, int quant_cols, int quant_rows, int to_gfx950);

/*
 * The GEMM with the reordering and the additions around it folded in.  No counterpart in the reference: its
 * harness packs a weight whose FP6 columns already sit at the tail (gen_mixed_weight, test.py:123-152) and
 * leaves the matching reorder of the output columns (and, for selected input channels, of the activations) and
 * any bias / residual addition to separate kernels of the caller.
 *   A, lda    device fp16 [m, lda] row-major.  Without a_cols, lda must equal prob_k.
 *   a_cols    device int32 [prob_k] or NULL: row kk of the packed weight multiplies column a_cols[kk] of A
 *             (0 <= a_cols[kk] < lda).  With one row the decode kernel fetches A through the map itself; otherwise a
 *             pass of its own gathers the rows into a 64 MiB buffer of the call's workspace, which the first call with a_cols
 *             allocates; min(prob_m, 64 * max_par) * prob_k * 2 bytes must fit (else FP6M_ERR_ARG).
 *   c_cols    device int32 [prob_n] or NULL: packed column j (INT4 columns first, then the FP6 columns) is written
 *             to column c_cols[j] of C; must be a permutation of 0 .. prob_n-1.
 *   bias      device fp16 [prob_n] or NULL, indexed by C column.
 *   residual  device fp16 [prob_m, prob_n] or NULL, laid out like C; may be C itself (in-place accumulation).
 *   C[r, c_cols[j]] = fp16(acc[r, j] * scale[j] + bias[c_cols[j]] + residual[r, c_cols[j]]): the additions are in
 *   fp32 and the result is rounded once.  With all four NULL the result equals fp6m_mul's bit for bit.
 * Map entries out of range are clamped on the device (wrong values, no fault); validate maps once on the host.
 * Other arguments as for fp6m_mul (tile shapes are always automatic).
 *   flags     0, or FP6M_LAYOUT_GFX950 when B went through fp6m_repack_gfx950.
 */
int fp6m_mul_fused(const void* A, int lda, const void* B, void* C, const void* s, int prob_m, int prob_n, int prob_k,
                   void* workspace, int dev, void* stream, int sms, int max_par, int quant_cols, int group_size,
                   const int32_t* a_cols, const int32_t* c_cols, const void* bias, const void* residual, int flags);

/*
 * The GEMM for a weight mixed along k instead of n: the last quant_rows rows (input channels) of every column are
 * FP6 e3m2 with one scale per column, the prob_k - quant_rows rows before them INT4 with one scale per 128 rows and
 * column.  Both segments of a column tile accumulate into the same output tile inside one launch.  No counterpart
 * in the reference, which splits the columns between the two formats (fp6_marlin_cuda_kernel.cu:308-337); there the
 * same result takes two launches on the two row ranges and an addition.
 *   B   INT4 words of rows [0, prob_k - quant_rows) (fp6m_int4_pack of that [rows, n] block) || FP6 2-bit plane ||
 *       FP6 4-bit plane of the last quant_rows rows (fp6m_fp6_prepack of that [quant_rows, n] block)
 *   s   INT4 scales [(prob_k - quant_rows) / 128, n] in natural column order || FP6 scales [n] in the permuted
 *       order of fp6m_permute_scales
 * (prob_k - quant_rows) % 128, quant_rows % 64 or prob_n % 128 != 0 -> FP6M_ERR_PROB_SHAPE.
 * lda, a_cols, c_cols, bias, residual, flags as for fp6m_mul_fused (a_cols is how arbitrary input channels reach the
 * tail).
 */
int fp6m_mul_rows(const void* A, int lda, const void* B, void* C, const void* s, int prob_m, int prob_n, int prob_k,
                  void* workspace, int dev, void* stream, int sms, int max_par, int quant_rows, const int32_t* a_cols,
                  const int32_t* c_cols, const void* bias, const void* residual, int flags);

/*
 * Testing / tuning hook: overrides one of the dispatcher's per-shape choices for all later calls in this process.
 * No counterpart in the reference (whose only such knob is the `sms` argument).  knob = "ksplit" (k parts per tile),
 * "wk16" / "wk" (waves per workgroup of the m <= 16 / m > 16 kernel: 4 or 8), "mb" (16-row blocks per wave: 2, 4 or 8),
 * "pair" (paired activation fetch on/off),
 * "sk" (the one-wave decode kernel on for m <= 4 / off), "share" / "share6" (k units per chunk of its work list: both
 * regions / the FP6 region only), "cap" (the waves it aims at), "wgs" (exactly that many waves, one-unit chunks drawn
 * from the counters), "gather" (its own activation gather on / off), "cells" (0: the m <= 16 kernel sums the shared
 * tiles of up to four rows through partial tiles, like those of more rows, instead of in the accumulate-and-count cells),
 * "xcd" (the m <= 16 kernel's partial tiles of 5 to 16 rows exchanged inside one XCD: 1 wherever possible, 0 never),
 * "gen" (0: the decode kernel's chunks all of one length), "gen2" / "gen3" (per cent: the share of a SIMD that its planner
 * assumes for the waves of the second / third generation, which sets their chunk lengths), "cap2" (the most chunks per
 * tile that it gives those generations), "young" (per cent: the k slice
 * of the second wave of every SIMD in eight-wave workgroups relative to the first one's; 100 = equal slices),
 * "cls" (0: the kernels never put the INT4 tiles in two classes -- whole tiles on the first workgroups, the
 * rest in parts on later ones --, 1: wherever they can), "cus" (tests: plan for a chip of that many CUs),
 * "verbose" (print every launch's configuration to stderr); knob = NULL clears all overrides.  Unknown knob ->
 * FP6M_ERR_ARG.  Not synchronised with GEMM calls running on other threads.  The library reads no environment
 * variables on a call (FP6M_VERBOSE is looked up once at load time).
 */
int fp6m_tuning_set(const char* knob, int value);

/* Minimum workspace length in 4-byte elements: n / 128 * max_par (fp6_marlin/fp6_marlin_cuda.cpp:62-63). */
size_t fp6m_workspace_elems(int prob_n, int max_par);

/*
 * Device memory the GEMM keeps besides its operands, and what may run concurrently.
 *
 * Column tiles whose k range is shared by several workgroups are summed through fp32 partial tiles or 64-bit cells in
 * device memory (the reference sums them through C in fp16 under the locks in `workspace`,
 * fp6_marlin_cuda_kernel.cu:645-696).  That scratch belongs to the workspace: every workspace address the library has
 * seen on a device owns a 24 MiB region (plus 64 MiB for gathered activations once a call with a_cols has used it).
 * The concurrency rule is therefore the reference's, one call at a time per workspace (fp6_marlin_cuda.cpp:62-63):
 * calls with different workspaces may overlap on different streams, also when replayed from HIP graphs; two
 * overlapping calls must not share a workspace.
 * A device has FP6M_MAX_WORKSPACES regions.  The first FP6M_BUILTIN_WORKSPACES share one pool that is allocated once
 * per device (hipMalloc + hipMemset, synchronous) by the first call that may wait for it -- fp6m_init_workspace, or the
 * first GEMM call whose stream is not being captured -- after which a call with a new workspace allocates nothing and
 * never waits for the device.  A call that is being captured before the pool exists uses, for its workspace, a slot of
 * an array that is part of the library's device code (96 MiB per GPU, held until the process ends) instead: it
 * allocates nothing either and can be captured as it is, like the reference's (fp6_marlin_cuda_kernel.cu:864-880), but
 * atomics on that memory are slower (a 4096 x 4096 decode GEMM takes 6.6 instead of 5.7 us), so give a workspace its
 * region with fp6m_init_workspace, or run one call with it, before capturing where that matters.  The other regions
 * get their memory from hipMalloc + hipMemset when a fifth, sixth .. workspace turns up (not under capture), and keep
 * it for good.  A workspace the library has not seen
 * takes a region nobody owns; when there is none, the region whose workspace has gone unused longest is handed over
 * after a hipDeviceSynchronize -- so callers that make a new workspace for every call (the reference's test.py:168 and
 * bench.py:44 do) never run out, at the price of that wait from the seventeenth workspace on.  Consequences: keep at
 * most FP6M_MAX_WORKSPACES workspaces in concurrent use per device (overlapping calls on more would share scratch); a
 * graph captured with a workspace whose region has since been handed over must not be replayed while calls with the
 * new owner are running; and a call under capture whose workspace has no region yet is refused (FP6M_ERR_SCRATCH)
 * unless a region is free -- fp6m_init_workspace beforehand makes sure.  The gathered-activation buffer of
 * fp6m_mul_fused (64 MiB, once per region) is always allocated with hipMalloc.  Share one workspace between calls that
 * never overlap (all layers of a model on one stream).  fp6m_release_workspace gives a workspace's region up (call it
 * before the workspace is freed), or all of a device's with workspace = NULL; it waits for the device first, and
 * graphs captured with that workspace must not be replayed afterwards.  No counterpart in the reference.
 */
#define FP6M_MAX_WORKSPACES 16
#define FP6M_BUILTIN_WORKSPACES 4
/*
 * Looks up the device's properties (compute units, addresses of the built-in scratch) and checks, with a few launches
 * of a probe kernel, how the device deals a dispatch's workgroups to its XCDs (the m <= 16 kernel exchanges partial
 * tiles inside one XCD's L2 only where that check has passed).  Waits for the device; allocates nothing.  Optional:
 * the first GEMM call on a device does the same, unless its stream is being captured, in which case the check is left
 * to a later call.
 */
int fp6m_init(int dev);
/* Region of `workspace` now rather than in its first call; with_gather != 0 also allocates its gathered-activation
 * buffer (needed before capturing an fp6m_mul_fused call that passes a_cols with more than one row). */
int fp6m_init_workspace(int dev, const void* workspace, int with_gather);
int fp6m_release_workspace(int dev, const void* workspace);

/*
 * FP16 -> FP6 (e3m2) row quantiser.  Replaces
 *   void weight_prepacking_fp16_to_fp6(uint16_t* weight_16bit, uint8_t* weight_6bit_packed, size_t K, size_t N)
 *   (fp6_marlin/weight_quant.cpp:106-124, declared fp6_marlin/pybind.cpp:7).
 * `w`: rows x cols binary16 bit patterns, `out`: rows x cols*6/8 bytes, four codes per three bytes, MSB
 * first.  Truncating cast; values with 0 < |x| < 0.0625, |x| > 28 or NaN -> FP6M_ERR_RANGE (the reference
 * throws); cols*6 % 8 != 0 -> FP6M_ERR_SHAPE.
 */
int fp6m_fp6_quantize(const uint16_t* w, uint8_t* out, size_t rows, size_t cols);

/*
 * FP6 2+4-bit prepacker, bit-exact with
 *   void weight_matrix_prepacking(int* packed_weights, int* FP6Weights, size_t K, size_t N)
 *   (fp6_marlin/weight_prepacking.cpp:123-177, declared fp6_marlin/pybind.cpp:6).
 * `fp6`: oc rows (output channels) x ic*6/8 bytes of row-packed codes; `packed`: oc*ic*6/8 bytes, the
 * 2-bit plane followed by the 4-bit plane.  oc % 64 or ic % 64 -> FP6M_ERR_SHAPE (the reference asserts).
 */
int fp6m_fp6_prepack(int32_t* packed, const int32_t* fp6, size_t oc, size_t ic);

/*
 * FP6 -> FP16 dequantiser.  Replaces
 *   void dequantMatrix_fp6_to_fp16(half* A_16bit_h, unsigned char* A_x_bit_h, size_t M, size_t K, half* scale)
 *   (fp6_marlin/weight_prepacking.cpp:180-217, declared fp6_marlin/pybind.cpp:5).
 * out[r][c] = fp16(value(code[r][c]) * scale[r]), one rounding.
 */
int fp6m_fp6_dequant(uint16_t* out, const uint8_t* fp6, size_t rows, size_t cols, const uint16_t* scale);

/*
 * Symmetric INT4 quantiser of the reference's harness (test.py:85-101, gen_int4_weight up to the
 * fake-quantised reference).  `w`: k x n binary16, row-major.  group_size -1 (per column) or a divisor
 * of k.  Outputs: codes k x n bytes in 0..15, scales (k/group) x n binary16 in natural column order,
 * w_ref k x n binary16 = (code - 8) * scale.  Any output pointer may be NULL.
 */
int fp6m_int4_quantize(const uint16_t* w, size_t k, size_t n, int group_size, uint8_t* codes,
                       uint16_t* scales, uint16_t* w_ref);

/*
 * Marlin INT4 packer, bit-exact with the packing half of gen_int4_weight (test.py:106-113 with the
 * permutation of test.py:60-79).  codes k x n bytes in 0..15 -> packed int32 [k/16, n*2].
 * k % 16 or n % 64 -> FP6M_ERR_SHAPE.
 */
int fp6m_int4_pack(const uint8_t* codes, int32_t* packed, size_t k, size_t n);

/* Scale permutation of test.py:80-83 applied per group of 32 (test.py:49-53, 102-105). n % 32 -> ERR_SHAPE. */
int fp6m_permute_scales(const uint16_t* in, uint16_t* out, size_t n);

/*
 * Host inverse of both packers: the dequantised fp16 weight W_ref [k, n] that `B`/`s` encode -- the
 * left operand of the reference's dequantise-then-matmul check (test.py:37-38, 98, 165-167).
 */
int fp6m_unpack_to_fp16(const int32_t* B, const uint16_t* s, uint16_t* w_ref, size_t k, size_t n,
                        int quant_cols, int group_size);

/* Weight preparation on the GPU: what the reference's harness does on the host with numpy and its CPU extension
 * (gen_mixed_weight test.py:123-152 = gen_int4_weight test.py:85-121 + gen_fp6_weight test.py:13-58, i.e.
 * weight_quantization_cpu pybind.cpp:42-59 and weight_prepacking_cpu pybind.cpp:18-31, + the scale permutation
 * test.py:80-83), in one call on device memory, bit for bit.
 *   w        device fp16 [k, n] row-major
 *   B, s     device outputs in the wire format of fp6m_mul (sizes as for fp6m_unpack_to_fp16)
 *   w_ref    optional device fp16 [k, n]: the dequantised weight the GEMM multiplies by (NULL to skip)
 *   harness_layout  1 = the reference harness bit for bit (its FP6 path reads the flat [k, quant_cols] buffer as
 *            [quant_cols, k] without transposing); 0 = quantise the true transpose (what Layer.pack uses)
 * k % 64 == 0, quant_cols and n - quant_cols multiples of 64, group_size -1 or a divisor of k.
 * Enqueued on `stream`; when quant_cols > 0 the call waits for its kernels, because the FP6 range check
 * (FP6M_ERR_RANGE: a NaN weight or a zero-scale column in the harness layout) is reported by value. */
int fp6m_pack_mixed_device(const void* w, int k, int n, int quant_cols, int group_size, int harness_layout,
                           void* B, void* s, void* w_ref, int dev, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FP6M_H_ */
