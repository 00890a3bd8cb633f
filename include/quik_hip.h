/* C ABI of libquik_hip.so: the MI355X (gfx950) implementation of the forward path of
 * QUIK's MixedQLinear.  Plain pointers and sizes only; every pointer is DEVICE memory on
 * the current HIP device unless stated otherwise, every output buffer is allocated by the
 * caller, `stream` is a hipStream_t passed as void* (NULL = the default stream), and all
 * calls are asynchronous with respect to the host.  Every function returns QUIK_OK (0) or
 * a negative quik_status; quik_status_string() gives the message the Python layer raises.
 *
 * Each entry point names the interface of the reference it replaces (paths relative to
 * the reference checkout).  The reference returns freshly allocated tensors; here the
 * thin host layer (quik_amd/asymmetric.py, symmetric.py, matmul.py) allocates and this
 * library only fills.
 */
#ifndef QUIK_HIP_H_
#define QUIK_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum quik_status {
  QUIK_OK = 0,
  QUIK_ERR_BITS = -1,      /* bits argument must be either 4 or 8 (or 8/16/32 for symmetric dequantize) */
  QUIK_ERR_SHAPE = -2,     /* sizes inconsistent with each other */
  QUIK_ERR_DTYPE = -3,     /* dtype id not QUIK_F16 / QUIK_BF16, or not supported by this op */
  QUIK_ERR_ALIGN = -4,     /* K or a pointer violates the alignment the op needs */
  QUIK_ERR_NULL = -5,      /* required pointer is NULL */
  QUIK_ERR_RANGE = -6,     /* size beyond what the kernel supports */
  QUIK_ERR_LAUNCH = -7,    /* HIP reported a launch error; hipGetLastError text via quik_last_hip_error() */
  QUIK_ERR_COLMAP = -8     /* the column map does not select the streaming quantize kernel (or has no in-place
                              order) and this entry point has no other path; also: the map's flags are not known
                              to the host yet and the stream is being captured (call quik_colmap_streaming once
                              per map outside the capture).  Nothing was launched. */
} quik_status;

typedef enum quik_dtype { QUIK_F16 = 0, QUIK_BF16 = 1 } quik_dtype;

const char *quik_status_string(int status);
const char *quik_last_hip_error(void);
int quik_abi_version(void);

/* ------------------------------------------------------------------------------------
 * Column map: the outlier split of one layer in the compact form the quantize kernel
 * reads.  Built once per layer (or per call by the stateless op) from the int64 index
 * tensors the reference passes to every call (src/asymmetric/asymmetric.cu:449-453).
 * Indices outside [0, cols) are clamped into range.
 * quik_colmap_bytes: size of the workspace, 0 if the arguments are invalid. */
int64_t quik_colmap_bytes(int64_t cols, int64_t num_int, int64_t num_fp);
int quik_colmap_build(const int64_t *int_indices, int64_t num_int,
                      const int64_t *fp_indices, int64_t num_fp, int64_t cols,
                      void *colmap, void *stream);

/* quik.asymmetric.quantize(src, int_indices, fp_indices, bits) -> (dst, meta, fp_x)
 * replaces QUIK::asymmetric::quantize, src/asymmetric/asymmetric.cpp:16-25 and
 * quantizeCUDA, src/asymmetric/asymmetric.cu:492-584.
 *   x      [rows, cols] dtype, contiguous
 *   dst    [rows, num_int/2] uint8 (bits=4, low nibble = even element) or [rows, num_int] int8
 *   meta   [2*rows] dtype, interleaved (scale, zero)
 *   fp_x   [rows, num_fp] dtype
 * num_int + num_fp must equal cols and num_int must be even (asymmetric.cu:519-524).
 * `colmap` comes from quik_colmap_build for the same (cols, num_int, num_fp). */
int quik_asym_quantize(const void *x, int dtype, int64_t rows, int64_t cols,
                       const void *colmap, int64_t num_int, int64_t num_fp, int bits,
                       void *dst, void *meta, void *fp_x, void *stream);

/* quik.asymmetric.find_meta(src, bits) -> meta [2*rows]; fp16 only, all columns.
 * replaces findMaxMinMetaCUDA, src/asymmetric/asymmetric.cu:320-338. */
int quik_asym_find_meta(const void *x, int64_t rows, int64_t cols, int bits,
                        void *meta, void *stream);

/* quik.asymmetric.quantizeOld(src, meta, bits) -> dst; fp16 only, every column.
 * replaces quantizeCUDAOld, src/asymmetric/asymmetric.cu:68-117.
 * dst is [rows, ceil(cols/2)] uint8 for bits=4 (flat pairing over the whole array as the
 * reference kernel does, :25-43) or [rows, cols] int8. */
int quik_asym_quantize_old(const void *x, const void *meta, int64_t rows, int64_t cols,
                           int bits, void *dst, void *stream);

/* quik.asymmetric.dequantize(x, meta, scale_col, wReduced, y, bits) -> out
 * replaces dequantizeCUDA, src/asymmetric/asymmetric.cu:175-233 (kernel :119-173).
 *   acc [rows, cols] int32; meta [2*rows]; scale_col [cols]; w_reduced [cols];
 *   y, out [rows, cols] dtype.  fp32 arithmetic, one rounding to dtype. */
int quik_asym_dequantize(const int32_t *acc, const void *meta, const void *scale_col,
                         const void *w_reduced, const void *y, int dtype, int64_t rows,
                         int64_t cols, int bits, void *out, void *stream);

/* quik.symmetric.quantize(src, scale, bits) -> dst; fp16 only.
 * replaces int4QuantizationCUDA / int8QuantizationCUDA, src/symmetric/symmetric.cu:6-79.
 *   x [rows, cols] fp16; scale [rows] fp16; dst [rows, ceil(cols/2)] uint8 or [rows, cols] int8.
 * No clamp: int4 keeps the low four bits, int8 wraps (C conversion). */
int quik_sym_quantize(const void *x, const void *scale, int64_t rows, int64_t cols,
                      int bits, void *dst, void *stream);

/* quik.symmetric.dequantize(x, scale_row, scale_col, y, bits) -> out; fp16 chain.
 * replaces dequantizationCUDA<T>, src/symmetric/symmetric.cu:91-152;
 * x_bits selects the element type of x: 8 int8, 16 fp16, 32 int32 (symmetric.cpp:32-41). */
int quik_sym_dequantize(const void *x, int x_bits, const void *scale_row,
                        const void *scale_col, const void *y, int64_t rows, int64_t cols,
                        void *out, void *stream);

/* quik.asymmetric.int4FusedDequantize / int8FusedDequantize(A, B, scale_row, scale_col, shift_value,
 *                                                          zero_row, w_reduced, y) -> out fp16 [M, N]
 * replaces int4FusedDequantizeCUDA / int8FusedDequantizeCUDA, src/asymmetric/fused_dequantize.cu:9-119.
 *   A [M, K/2] uint8 or [M, K] int8; B [N, K/2] or [N, K]; scale_row, zero_row [M] fp16;
 *   scale_col, w_reduced [N] fp16; y [M, N] fp16.
 *   out = ((h(acc) * scale_col) * scale_row + (zero_row + h(shift) * scale_row) * w_reduced) + y
 * in fp16 arithmetic, one rounding per operation, exactly as the reference's epilogue
 * (include/asymmetric/epilogue/thread/linear_combination_dequant.h:155-162).
 * One launch: the epilogue runs on the accumulators of the GEMM tiles; no int32 matrix goes through
 * memory.  Calls with at most 32 rows (quik_fused_dequantize_workspace_bytes(M, N) > 0) run on the
 * weight-streaming kernel, which has no such epilogue: for those the exact int32 product goes to
 * acc_workspace ([M, N] int32, caller-provided) and a second launch applies the epilogue; otherwise
 * acc_workspace may be NULL. */
int64_t quik_fused_dequantize_workspace_bytes(int64_t M, int64_t N);
int quik_asym_fused_dequantize(const void *A, const void *B, const void *scale_row,
                               const void *scale_col, float shift_value, const void *zero_row,
                               const void *w_reduced, const void *y, int64_t M, int64_t N,
                               int64_t K, int bits, int32_t *acc_workspace, void *out,
                               void *stream);

/* quik.symmetric.int4FusedDequantize / int8FusedDequantize(A, B, scale_row, scale_col, y) -> out
 * replaces int4FusedDequantizeCUDA / int8FusedDequantizeCUDA, src/symmetric/fused_dequantize.cu:9-107.
 *   out = ((h(acc) * scale_row) * scale_col) + y in fp16 arithmetic
 * (include/symmetric/epilogue/thread/linear_combination_dequant.h:149-150).  Workspace as above. */
int quik_sym_fused_dequantize(const void *A, const void *B, const void *scale_row,
                              const void *scale_col, const void *y, int64_t M, int64_t N,
                              int64_t K, int bits, int32_t *acc_workspace, void *out,
                              void *stream);

/* ---- W4A4 on the 6-bit matrix-core path -------------------------------------------------------
 * No counterpart in the reference: an internal operand format between this library's own quantize
 * and GEMM kernels.  int4 levels (code + 8) are E2M3 numbers; v_mfma_f32_32x32x64_f8f6f4 multiplies
 * them exactly at twice the int8 rate, and the integer accumulator is recovered exactly from the
 * fp32 sum and the per-row / per-column level sums, so the results are those of
 * quik_mixed_linear_fwd bit for bit.  An operand buffer holds a [rows, K] int4 matrix, its [rows, F]
 * fp16/bf16 outlier columns and the per-row level sums, in the order the GEMM tiles read them.
 * Needs K % 128 == 0, K <= 74496 (the fp32 sums are exact up to there), F % 32 == 0, M > 32;
 * operand buffers aligned to 256 bytes. */

/* bytes of an operand buffer for [rows, K] int4 + [rows, F] outliers (0 if the shape is not supported) */
int64_t quik_fp6_operand_bytes(int64_t rows, int64_t K, int64_t F);

/* weights [N, K/2] nibble-packed int4 (MixedQLinear.int_weight) and [N, F] fp16/bf16
 * (MixedQLinear.fp_weight, may be NULL when F == 0) -> operand buffer; once per layer.
 * Along K the operand buffers of this path are in the column map's in-place order (position k = source
 * column k of the activation, outlier positions filled by the integer columns of the last F source
 * columns), which lets the quantize kernel write a row without moving data sideways; `colmap` is the
 * layer's column map (quik_colmap_build for cols = K + F; quik_colmap_streaming(...) must be 1), from
 * which the weights take the same order.  Buffers packed for one column map must only meet activations
 * quantized with the same one. */
int quik_fp6_pack_weight(const uint8_t *qw, const void *fp_w, int64_t N, int64_t K, int64_t F,
                         const void *colmap, void *out, void *stream);

/* 1 if the column map selects the streaming quantize kernel (ascending int_indices that, with fp_indices,
 * partition the columns; cols % 8 == 0; cols <= 32768), 0 if not, negative on error.  The first call for a map
 * copies one word from the device and synchronises the stream; the library remembers the answer per (address,
 * shape) until quik_colmap_build writes to that address again.  The entry points that need such a map
 * (quik_asym_quantize_fp6, quik_asym_quantize_tile8, quik_sym_quantize_mapped, quik_fp6_pack_weight) make the
 * same look-up themselves and return QUIK_ERR_COLMAP, launching nothing, for a map that does not qualify. */
int quik_colmap_streaming(const void *colmap, int64_t cols, int64_t num_int, int64_t num_fp, void *stream);

/* as quik_asym_quantize with bits = 4, but codes and outlier values go to an operand buffer
 * (quik_fp6_operand_bytes(rows, num_int, num_fp)); the column map must select the streaming kernel
 * (quik_colmap_streaming) */
int quik_asym_quantize_fp6(const void *x, int dtype, int64_t rows, int64_t cols, const void *colmap,
                           int64_t num_int, int64_t num_fp, void *out6, void *meta, void *stream);

/* as quik_mixed_linear_fwd (asymmetric form, bits = 4) on operand buffers; any row count (M >= 1) */
int quik_mixed_linear_fwd_fp6(const void *x6, const void *w6, const void *meta, const void *s_col,
                              const void *w_reduced, const void *bias, int dtype, int64_t M, int64_t N,
                              int64_t K, int64_t F, void *out, void *stream);

/* ---- symmetric activations in one kernel --------------------------------------------------------
 * MixedQLinear's symmetric branch (experiments/qlinear.py:97-103) computes, with torch ops and
 * symmetric.quantize: int_x = x[:, int_indices]; fp_x = x[:, fp_indices];
 * scale = fp16(max|int_x| / divisor); q = rne(fp16(int_x / scale)) kept modulo 2^bits.  This entry
 * point does the same in the streaming quantize kernel (fp16 only; the column map must select that
 * kernel: quik_colmap_streaming(...) == 1, otherwise nothing is written).  tiled == 0: dst is
 * [rows, num_int/2] uint8 (bits = 4) or [rows, num_int] int8 and fp_x [rows, num_fp]; tiled != 0:
 * dst is an operand buffer of the tile-ordered GEMMs (quik_fp6_operand_bytes for bits = 4,
 * quik_tile8_operand_bytes for bits = 8; their shape conditions apply) and fp_x is not used.
 * scale: [rows] fp16.  A row that holds a NaN gets a NaN scale and all-zero codes, as with torch.
 * The tile-ordered GEMM entry points take the symmetric form when w_reduced == NULL (meta = scale). */
int quik_sym_quantize_mapped(const void *x, int64_t rows, int64_t cols, const void *colmap, int64_t num_int,
                             int64_t num_fp, int bits, float divisor, int tiled, void *dst, void *scale,
                             void *fp_x, void *stream);

/* ---- W8A8 on tile-ordered operands -------------------------------------------------------------
 * No counterpart in the reference: the same forward as quik_asym_quantize (bits = 8) +
 * quik_mixed_linear_fwd (bits = 8, asymmetric), bit for bit for more than 32 rows (up to 32 rows
 * that entry point runs a weight-streaming kernel, which adds the fp32 terms in another order:
 * equal within rounding), with both int8 operands (and the
 * outlier columns) stored in the order the GEMM tiles copy them, so that every copy moves whole
 * cache lines exactly once per tile.  Needs K % 64 == 0, F % 32 == 0, a column map that
 * selects the streaming quantize kernel; operand buffers aligned to 256 bytes. */

/* bytes of an operand buffer for [rows, K] int8 + [rows, F] outliers (0 if the shape is not supported) */
int64_t quik_tile8_operand_bytes(int64_t rows, int64_t K, int64_t F);

/* weights [N, K] int8 (MixedQLinear.int_weight) and [N, F] fp16/bf16 (fp_weight, may be NULL when
 * F == 0) -> operand buffer; once per layer */
int quik_tile8_pack_weight(const int8_t *qw, const void *fp_w, int64_t N, int64_t K, int64_t F, void *out,
                           void *stream);

/* as quik_asym_quantize with bits = 8, codes and outlier values go to an operand buffer */
int quik_asym_quantize_tile8(const void *x, int dtype, int64_t rows, int64_t cols, const void *colmap,
                             int64_t num_int, int64_t num_fp, void *out8, void *meta, void *stream);

/* as quik_mixed_linear_fwd (asymmetric form, bits = 8) on operand buffers */
int quik_mixed_linear_fwd_tile8(const void *x8, const void *w8, const void *meta, const void *s_col,
                                const void *w_reduced, const void *bias, int dtype, int64_t M, int64_t N,
                                int64_t K, int64_t F, void *out, void *stream);

/* ---- K split for the tile-ordered GEMMs ----------------------------------------------------------
 * No counterpart in the reference.  With few token rows and few output columns the 128x128 tiles of
 * the tile-ordered GEMMs are fewer than the CUs and each walks the whole K (70B down_proj, 64 tokens:
 * 64 tiles, K = 28416).  Given a workspace, several workgroups per tile take a K range each, add
 * their exact accumulators through it, and the one that finishes last does the outlier product and
 * the epilogue: same output bits, the weights stream through all CUs.
 * quik_splitk_workspace_bytes: bytes with which the _ws entry points split this shape (0: they do
 * not; bits = 4: the 6-bit path, bits = 8: the int8 path).  The first 4096 bytes of the workspace hold
 * the arrival counters and MUST be zero when a launch starts: zero the workspace before its first use;
 * every launch that completes leaves the counters at zero again, but after a launch that failed (a
 * returned QUIK_ERR_LAUNCH, an aborted process that shared the buffer) zero them again before the next
 * call, otherwise tiles are finished on incomplete sums or never.  The workspace is 16-byte aligned and
 * must not be shared by launches that may overlap (other streams).  workspace == NULL or too small: no
 * split, as the entry points without _ws. */
int64_t quik_splitk_workspace_bytes(int64_t M, int64_t N, int64_t K, int bits);
int quik_mixed_linear_fwd_fp6_ws(const void *x6, const void *w6, const void *meta, const void *s_col,
                                 const void *w_reduced, const void *bias, int dtype, int64_t M, int64_t N,
                                 int64_t K, int64_t F, void *out, void *workspace, int64_t workspace_bytes,
                                 void *stream);
int quik_mixed_linear_fwd_tile8_ws(const void *x8, const void *w8, const void *meta, const void *s_col,
                                   const void *w_reduced, const void *bias, int dtype, int64_t M, int64_t N,
                                   int64_t K, int64_t F, void *out, void *workspace, int64_t workspace_bytes,
                                   void *stream);

/* ---- one call per layer forward -----------------------------------------------------------------------
 * replaces the op sequence of MixedQLinear.forward, experiments/qlinear.py:80-148 (quantize, integer GEMM,
 * F.linear on the outlier columns, dequantize), for callers that want one boundary crossing per layer:
 * at decode sizes the kernels take 20 us and every crossing from an interpreter costs several.
 * quik_layer describes the layer's buffers once (all device pointers; the same buffers MixedQLinear
 * registers, qlinear.py:53-78); a forward picks the kernels as MixedQLinear does here: up to
 * tiled_min_rows - 1 rows the row-major quantize + quik_mixed_linear_fwd (weight-streaming kernel up to 32
 * rows), from tiled_min_rows rows the tile-ordered paths when tiled_weight is given and the shape allows.
 *   struct_bytes    sizeof(quik_layer), checked
 *   bits 4 | 8; dtype QUIK_F16 | QUIK_BF16; symmetric 0 | 1 (fp16 and a streaming column map only)
 *   colmap          quik_colmap_build(...) for (in_features, num_int, num_fp); colmap_streams: what
 *                   quik_colmap_streaming returned for it
 *   int_weight [out, num_int/2] u8 or [out, num_int] i8; weights_scales [out]; reduced_w [out] (NULL when
 *   symmetric); fp_weight [out, num_fp] (NULL when num_fp == 0); bias [out] or NULL
 *   tiled_weight    quik_fp6_pack_weight (bits 4) / quik_tile8_pack_weight (bits 8) buffer, or NULL
 *   tiled_min_rows  33 is what MixedQLinear uses.  With 1 every call takes the tile-ordered path and reads
 *                   only tiled_weight: int_weight and fp_weight may then be NULL, i.e. the layer can live
 *                   with ONE copy of its weights (0.75 byte per int4 weight, 1 per int8 weight) at the price
 *                   of slower calls of at most 32 rows (the weight-streaming kernel reads the packed nibbles)
 * workspace: quik_layer_workspace_bytes(layer, rows) bytes, 256-byte aligned, holds the quantized activation
 * between the two launches; splitk_workspace as for the _ws entry points (may be NULL).
 * mid_event: NULL, or a hipEvent_t that is recorded on the stream between the quantize launch and the
 * GEMM launch (profiling hook: lets a caller time the two kernels of a one-call forward).
 * x [rows, in_features] dtype, out [rows, out_features] dtype. */
typedef struct quik_layer {
  int32_t struct_bytes, bits, dtype, symmetric;
  int64_t in_features, num_int, num_fp, out_features;
  float sym_divisor;
  int32_t colmap_streams, tiled_min_rows, reserved;
  const void *colmap, *int_weight, *weights_scales, *reduced_w, *fp_weight, *bias, *tiled_weight;
} quik_layer;
int64_t quik_layer_workspace_bytes(const quik_layer *layer, int64_t rows);
int quik_layer_forward(const quik_layer *layer, const void *x, int64_t rows, void *workspace,
                       int64_t workspace_bytes, void *splitk_workspace, int64_t splitk_bytes, void *out,
                       void *mid_event, void *stream);
/* Calls of one or two token rows (a column map that streams; symmetric activations: fp16) take ONE launch: the
 * weight-streaming kernel quantises the rows itself, with the arithmetic of quik_asym_quantize /
 * quik_sym_quantize_mapped, and the workspace
 * stays untouched; mid_event is then recorded behind that launch.  quik_layer_set_one_launch(0) switches this off
 * for the process (the two-launch form; same output bits), 1 switches it on again (the default).  No counterpart in
 * the reference. */
void quik_layer_set_one_launch(int on);

/* ---- the reference's simulated (fake-quant) activation path ---------------------------------------
 * replaces the tensor-op sequence of ActQuantWrapper.forward, experiments/quant_sim.py:227-256
 * (ActQuantizer.find_params :167-188, asymmetric_quantize :5-7), which the reference uses for its
 * accuracy experiments: per row, over the columns whose bit in outlier_mask is clear,
 *   xmin = min(min x, 0), xmax = max(max x, 0) (both zero -> -1, +1), scale = (xmax - xmin) / (2^bits - 1),
 *   zero = round(-xmin / scale), out = scale * (clamp(round(x / scale) + zero, 0, 2^bits - 1) - zero);
 * columns whose bit is set are copied.  fp32 arithmetic, one rounding to dtype.
 *   x, out [rows, cols] dtype; outlier_mask [ceil(cols / 32)] uint32, bit c % 32 of word c / 32 = column c;
 *   bits 2 .. 8. */
int quik_sim_act_fake_quant(const void *x, int dtype, int64_t rows, int64_t cols, const uint32_t *outlier_mask,
                            int bits, void *out, void *stream);

/* ---- one entry point that allocates nothing ---------------------------------------------------------
 * No counterpart in the reference.  For callers that cannot allocate device memory around the call and
 * have no workspace to hand in: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  It is quik_mixed_linear_fwd_tile8_ws with the K-split workspace (arrival counters
 * and partial accumulators) in a device array that lives inside the library: 4 KB + 256 x 64 KB = 16 MB
 * + 4 KB per GPU, held from the first use of the library on that GPU until the process ends.  Same
 * arguments, same checks and the same output bits as quik_mixed_linear_fwd_tile8_ws with a workspace of
 * quik_splitk_workspace_bytes(M, N, K, 8) bytes; a shape whose K split would need more than the array
 * holds returns QUIK_ERR_RANGE.  The call makes no hipMalloc / hipFree: it looks up the array's address
 * once per device (on the first call there, which should therefore happen outside a graph capture),
 * clears the counters with a small kernel and launches the GEMM.  All calls on one GPU share the array:
 * calls that may overlap on that GPU (different streams) race on it and must be serialised by the caller. */
int quik_mixed_linear_fwd_tile8_noalloc(const void *x8, const void *w8, const void *meta, const void *s_col,
                                        const void *w_reduced, const void *bias, int dtype, int64_t M,
                                        int64_t N, int64_t K, int64_t F, void *out, void *stream);

/* quik.matmul.int4Matmul(A, B) -> C int32 [M, N]
 * replaces int4MatmulCUDA, src/matmul/matmul.cu:17-55.
 *   A [M, K/2], B [N, K/2] uint8 nibble-packed, K = number of int4 elements per row.
 * K % 32 == 0 (the reference's 128-bit operand alignment); K < 131072. */
int quik_int4_matmul(const uint8_t *A, const uint8_t *B, int32_t *C, int64_t M, int64_t N,
                     int64_t K, void *stream);

/* quik.matmul.int8Matmul(A, B) -> C int32 [M, N]
 * replaces int8MatmulCUDA, src/matmul/matmul.cu:98-136.  K % 16 == 0. */
int quik_int8_matmul(const int8_t *A, const int8_t *B, int32_t *C, int64_t M, int64_t N,
                     int64_t K, void *stream);

/* One-launch replacement for the tail of MixedQLinear.forward
 * (experiments/qlinear.py:122-145): outlier GEMM (+bias), integer GEMM and dequantize.
 *   out[m,n] = dtype( f32(acc[m,n]) * (s_row[m]*s_col[n])
 *                     + (zero[m] + 2^(bits-1) * s_row[m]) * w_reduced[n]
 *                     + sum_f fp_x[m,f]*fp_w[n,f] + bias[n] )
 *   qx      [M, K/2] uint8 (bits=4) or [M, K] int8 (bits=8)     (quantize output)
 *   qw      [N, K/2] uint8 or [N, K] int8                       (MixedQLinear.int_weight)
 *   meta    [2*M] dtype (scale, zero) pairs; for the symmetric variant pass
 *           w_reduced = NULL and meta = per-row scales [M] (no zero-point term)
 *   s_col   [N] dtype (weights_scales), w_reduced [N] dtype or NULL
 *   fp_x    [M, F] dtype, fp_w [N, F] dtype, F % 8 == 0 (F may be 0 with NULL pointers)
 *   bias    [N] dtype or NULL
 * The integer accumulators are exact; the rest is fp32 with one rounding to dtype. */
int quik_mixed_linear_fwd(const void *qx, const void *qw, const void *meta,
                          const void *s_col, const void *w_reduced, const void *fp_x,
                          const void *fp_w, const void *bias, int dtype, int64_t M,
                          int64_t N, int64_t K, int64_t F, int bits, void *out,
                          void *stream);

#ifdef __cplusplus
}
#endif
#endif /* QUIK_HIP_H_ */
