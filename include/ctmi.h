/*
 * ctmi.h — C ABI of libctmi.so, the MI355X (gfx950) implementation of the
 * compressed-tensors weight compress/decompress hot path.
 *
 * Conventions shared by every entry point
 *   - All tensor pointers are DEVICE pointers owned and pre-allocated by the
 *     caller; tensors are dense, row-major ("contiguous") unless a stride is
 *     passed explicitly.  Nothing is allocated, freed or retained.
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream).  Work
 *     is enqueued on it; no entry point synchronises.
 *   - Return value: CTMI_OK (0) or a negative CTMI_ERR_* code.  Arguments are
 *     validated BEFORE the first HIP call, so every error path can be exercised
 *     on a host without a GPU.  ctmi_last_error() returns a thread-local,
 *     human-readable message for the most recent failure on this thread.
 *   - The reference implementation is pure Python (torch op chains); each entry
 *     point names the reference function (file:line under
 *     src/compressed_tensors/) whose arithmetic it reproduces bit-for-bit.
 */
#ifndef CTMI_H_
#define CTMI_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- return codes (the Python layer maps them to the reference's exception
 *      classes: ValueError / NotImplementedError / AssertionError / RuntimeError) */
#define CTMI_OK 0
#define CTMI_ERR_VALUE (-1)        /* bad argument            -> ValueError          */
#define CTMI_ERR_UNSUPPORTED (-2)  /* valid but not built     -> NotImplementedError */
#define CTMI_ERR_ASSERT (-3)       /* reference `assert` site -> AssertionError      */
#define CTMI_ERR_HIP (-4)          /* HIP runtime failure     -> RuntimeError        */

/* ---- element types */
#define CTMI_F32 0
#define CTMI_F16 1
#define CTMI_BF16 2
#define CTMI_F8E4M3 3 /* torch.float8_e4m3fn */
#define CTMI_I8 4
#define CTMI_I16 5
#define CTMI_I32 6
#define CTMI_I64 7
#define CTMI_U8 8
#define CTMI_BOOL 9

/* ---- quantized number formats (QuantizationType + num_bits, quant_args.py:85-91) */
#define CTMI_QTYPE_INT 0
#define CTMI_QTYPE_FLOAT 1

/* Quantization parameters of one tensor viewed as a 2-D [rows, cols] matrix.
 *
 * Scale element (i, j) of a logical [s_rows, s_cols] grid covers the elements
 *   i == (r / blk_rows) % s_rows     and     j == c / blk_cols
 * (or j == col_group[c] when col_group is given).  That one rule expresses every
 * strategy of quantization/lifecycle/forward.py:193-353:
 *   tensor   s=[1,1]     blk=[rows, cols]        channel  s=[R,1]   blk=[1, cols]
 *   group    s=[R,C/g]   blk=[1, g]              token    s=[T,1]   blk=[1, cols]
 *   block    s=[R/bh,C/bw] blk=[bh,bw]           attn_head s=[H,1]  blk=[S, cols]
 * zero_point (optional) has the same grid.  global_scale (optional) points to
 * one fp32 on the device: the effective scale is fp32(scale)/global_scale
 * (forward.py:468-469, 501-502).
 */
typedef struct ctmi_qparams {
  const void* scale;
  const void* zero_point;     /* NULL = reference called with zero_point=None */
  const float* global_scale;  /* NULL = none */
  const int32_t* col_group;   /* NULL = column order; else int32[cols] (act-order g_idx) */
  int64_t s_rows, s_cols;
  int64_t blk_rows, blk_cols;
  int32_t scale_dtype;        /* CTMI_F32 / F16 / BF16 / F8E4M3 */
  int32_t zp_dtype;           /* any CTMI_* numeric type */
  int32_t qtype;              /* CTMI_QTYPE_* */
  int32_t num_bits;           /* INT: 1..32, FLOAT: 4 (e2m1) or 8 (e4m3fn) */
} ctmi_qparams;

const char* ctmi_last_error(void);
int ctmi_version(void);

/* A5-A8.  quantize / dequantize / fake_quantize
 * (quantization/lifecycle/forward.py:45-189, _quantize :455-487, _dequantize
 * :491-514, round_to_quantized_type quant_args.py:384-408).
 * do_quantize / do_dequantize select among the three reference functions.
 * x is [rows, cols] of x_dtype; out is [rows, cols] of out_dtype.  The
 * arithmetic dtype is derived exactly as torch type promotion would derive it
 * from (x_dtype, scale_dtype, global_scale). */
int ctmi_qdq(const void* x, int32_t x_dtype, void* out, int32_t out_dtype, int64_t rows,
             int64_t cols, const ctmi_qparams* qp, int32_t do_quantize, int32_t do_dequantize,
             void* stream);

/* A8 on its own.  round_to_quantized_type (quantization/quant_args.py:384-408): every
 * element of a float16 / bfloat16 / float32 tensor of n elements rounded to the nearest
 * value of the quantized type and kept in the tensor's dtype: INT torch.round (ties to
 * even), FLOAT with 8 bits through float8_e4m3fn and back, FLOAT with 4 bits
 * FP4_E2M1_DATA.cast_to_fp4 (:55-68).  No scale, no clamp; out may be x.
 * Other bit widths of FLOAT: CTMI_ERR_UNSUPPORTED, as the reference's NotImplementedError. */
int ctmi_round_to_quantized_type(const void* x, void* out, int32_t dtype, int64_t n,
                                 int32_t qtype, int32_t num_bits, void* stream);

/* One tensor of a state dict for ctmi_qdq_many. */
typedef struct ctmi_qdq_job {
  const void* x;
  void* out;
  int64_t rows, cols;
  int32_t x_dtype, out_dtype;
  ctmi_qparams qp;
} ctmi_qdq_job;

/* A27 for the naive / int / float-quantized formats: the per-weight loop of
 * BaseQuantizationCompressor.compress / decompress_from_state_dict
 * (compressors/quantized_compressors/base.py:91-125, 213-230) around quantize /
 * dequantize, n tensors from one call.  Every job is validated before anything
 * is enqueued; tensors that share a kernel instance are chained into common
 * launches.  Same results as n calls of ctmi_qdq. */
int ctmi_qdq_many(const ctmi_qdq_job* jobs, int64_t n, int32_t do_quantize, int32_t do_dequantize,
                  void* stream);

/* A9.  pack_to_int32 (compressors/quantized_compressors/pack_quantized.py:186-246).
 * in: int8 [rows, cols]; out: int32 [rows, ceil(cols/pf)] (packed_dim=1) or
 * int32 [ceil(rows/pf), cols] (packed_dim=0), pf = 32/num_bits. */
int ctmi_pack_to_int32(const int8_t* in, int32_t* out, int64_t rows, int64_t cols,
                       int32_t num_bits, int32_t packed_dim, void* stream);

/* A10.  unpack_from_int32 (pack_quantized.py:249-309).  rows/cols are the
 * ORIGINAL (unpacked) shape; `in` has the packed shape described above. */
int ctmi_unpack_from_int32(const int32_t* in, int8_t* out, int64_t rows, int64_t cols,
                           int32_t num_bits, int32_t packed_dim, void* stream);

/* A11 fused.  PackedQuantizationCompressor.compress_weight
 * (pack_quantized.py:88-145): quantize(dtype=int8) + pack_to_int32 in one pass.
 * out: int32 [rows, ceil(cols/pf)]. */
int ctmi_pack_quantized_compress(const void* x, int32_t x_dtype, int32_t* out, int64_t rows,
                                 int64_t cols, const ctmi_qparams* qp, void* stream);

/* A11 fused.  PackedQuantizationCompressor.decompress_weight
 * (pack_quantized.py:147-183): unpack_from_int32 + dequantize in one pass.
 * zero_point in qp is the UNPACKED int8 zero point (or NULL). */
int ctmi_pack_quantized_decompress(const int32_t* packed, void* out, int32_t out_dtype,
                                   int64_t rows, int64_t cols, const ctmi_qparams* qp,
                                   void* stream);

/* One weight of a state dict.  src/dst: for compress, dense weight -> packed
 * words; for decompress, packed words -> dense weight.  dense_dtype is the
 * dtype of the dense side. */
typedef struct ctmi_weight_job {
  const void* src;
  void* dst;
  int64_t rows, cols;
  int32_t dense_dtype;
  int32_t reserved;
  ctmi_qparams qp;
} ctmi_weight_job;

/* A27.  The per-weight loop of BaseQuantizationCompressor.compress /
 * decompress_from_state_dict (compressors/quantized_compressors/base.py:91-125,
 * 213-230) for the pack-quantized format: n fused launches from one call.
 * Every job is validated before anything is enqueued; weights that share a
 * dtype / bit-width combination are chained into common launches, 8 per launch;
 * activation-ordered weights (qp.col_group set) likewise, among themselves. */
int ctmi_pack_quantized_compress_many(const ctmi_weight_job* jobs, int64_t n, void* stream);
int ctmi_pack_quantized_decompress_many(const ctmi_weight_job* jobs, int64_t n, void* stream);
/* Number of kernel launches the call above (compress != 0) or its inverse
 * (compress == 0) would enqueue for this job list, without enqueueing any:
 * what a profiler divides a pass's time by.  Negative = error code. */
int64_t ctmi_pack_quantized_launches(const ctmi_weight_job* jobs, int64_t n, int32_t compress);

/* A13.  pack_fp4_to_uint8 (compressors/quantized_compressors/fp4_quantized.py:135-178).
 * x: [rows, cols] float type; out: uint8 [rows, cols/2]. */
int ctmi_pack_fp4_to_uint8(const void* x, int32_t x_dtype, uint8_t* out, int64_t rows,
                           int64_t cols, void* stream);

/* A14.  unpack_fp4_from_uint8 (fp4_quantized.py:187-221).  rows/cols = unpacked shape. */
int ctmi_unpack_fp4_from_uint8(const uint8_t* in, void* out, int32_t out_dtype, int64_t rows,
                               int64_t cols, void* stream);

/* A15 fused.  NVFP4PackedCompressor.compress_weight (fp4_quantized.py:84-106):
 * quantize (fp4, global scale) + pack_fp4_to_uint8.  out: uint8 [rows, cols/2]. */
int ctmi_nvfp4_compress(const void* x, int32_t x_dtype, uint8_t* out, int64_t rows, int64_t cols,
                        const ctmi_qparams* qp, void* stream);

/* A15 fused.  NVFP4PackedCompressor.decompress_weight (fp4_quantized.py:108-123):
 * unpack_fp4_from_uint8 (to bf16) + dequantize.  out: [rows, cols] out_dtype. */
int ctmi_nvfp4_decompress(const uint8_t* packed, void* out, int32_t out_dtype, int64_t rows,
                          int64_t cols, const ctmi_qparams* qp, void* stream);

/* A27 for the nvfp4 format: the per-weight loop of BaseQuantizationCompressor.compress /
 * decompress_from_state_dict (compressors/quantized_compressors/base.py:91-125, 213-230)
 * in one call.  src/dst as in ctmi_weight_job (dense weight -> packed bytes, or back);
 * qp carries the fp8 group scales and the weight's global scale.  Every job is
 * validated before anything is enqueued; weights of one dense dtype are chained
 * into common launches, 8 per launch. */
int ctmi_nvfp4_compress_many(const ctmi_weight_job* jobs, int64_t n, void* stream);
int ctmi_nvfp4_decompress_many(const ctmi_weight_job* jobs, int64_t n, void* stream);

/* A19.  pack_bitmasks / unpack_bitmasks (utils/helpers.py:302-339):
 * numpy.packbits(axis=-1, bitorder="little").  mask: bool/uint8 [rows, cols];
 * packed: uint8 [rows, ceil(cols/8)]. */
int ctmi_pack_bitmasks(const uint8_t* mask, uint8_t* packed, int64_t rows, int64_t cols,
                       void* stream);
int ctmi_unpack_bitmasks(const uint8_t* packed, uint8_t* mask, int64_t rows, int64_t cols,
                         void* stream);

/* A17.  bitmask_compress (compressors/sparse_compressors/sparse_bitmask.py:131-149)
 * in two calls, because the size of `values` is data dependent:
 *   ctmi_bitmask_count    writes bitmask [rows, ceil(cols/8)], row_offsets int64 [rows]
 *                         (exclusive prefix sum of per-row non-zero counts) and
 *                         *total_nnz (int64, device);
 *   ctmi_bitmask_compact  writes values[total_nnz] (row-major order of the non-zeros).
 * elem_size is the element width in bytes (1, 2 or 4); `x != 0` is evaluated on
 * the value of a floating type (so -0.0 is dropped, NaN kept) when
 * is_float != 0, on the raw integer otherwise.  fp8 tensors are passed as
 * floats with elem_size 1 (sparse_bitmask.py:141-145 views them as int8 only to
 * index them; the mask itself comes from `tensor != 0`).
 * tmp: device scratch of ctmi_bitmask_tmp_bytes(rows, cols) bytes, 8-byte aligned. */
int64_t ctmi_bitmask_tmp_bytes(int64_t rows, int64_t cols);
int ctmi_bitmask_count(const void* x, int32_t elem_size, int32_t is_float, uint8_t* bitmask,
                       int64_t* row_offsets, int64_t* total_nnz, void* tmp, int64_t rows,
                       int64_t cols, void* stream);
int ctmi_bitmask_compact(const void* x, int32_t elem_size, const uint8_t* bitmask,
                         const int64_t* row_offsets, void* values, int64_t rows, int64_t cols,
                         void* stream);

/* A18.  bitmask_decompress (sparse_bitmask.py:152-169): scatter `values`
 * (nvalues elements, consumed in row-major order of the set bits; set bits
 * beyond nvalues read as zero) into a zero-filled [rows, cols].
 * With tmp (ctmi_bitmask_tmp_bytes(rows, cols) bytes) the positions come from
 * the bitmask alone, as in the reference, and row_offsets may be NULL.  Without
 * tmp, row_offsets is required and trusted. */
int ctmi_bitmask_decompress(const void* values, int64_t nvalues, int32_t elem_size,
                            const uint8_t* bitmask,
                            const int64_t* row_offsets, void* out, void* tmp, int64_t rows,
                            int64_t cols, void* stream);

/* ctmi_bitmask_decompress without a scratch argument.  No counterpart in the
 * reference: it exists for callers that cannot allocate device memory (code under
 * HIP graph capture, serving loops and harnesses that forbid hipMalloc).  The
 * scratch of the scatter kernels lives in a device array inside the library,
 * ctmi_bitmask_decompress_static_max_bytes() bytes (4 MiB) per GPU, held until the
 * process ends; a shape with ctmi_bitmask_tmp_bytes(rows, cols) above that is
 * refused with CTMI_ERR_VALUE.  The entry point calls no allocating routine.
 * Positions come from the bitmask alone (the `tmp` mode of
 * ctmi_bitmask_decompress); same bits.  All calls on one GPU share that GPU's
 * array: calls that overlap on one GPU (two streams, two threads) race; calls
 * enqueued on one stream do not, and nothing needs clearing between them.  The first
 * call on a GPU looks up the array's device address (hipGetSymbolAddress): it must be
 * made outside stream capture; later calls may be captured. */
int64_t ctmi_bitmask_decompress_static_max_bytes(void);
int ctmi_bitmask_decompress_static(const void* values, int64_t nvalues, int32_t elem_size,
                                   const uint8_t* bitmask, void* out, int64_t rows, int64_t cols,
                                   void* stream);

/* A22.  sparse24_bitmask_decompress (sparse_24_bitmask.py:206-224): the same
 * scatter, `out[mask] = values`, for any bitmask.  A bitmask that keeps exactly 2
 * of every 4 columns (what the format holds) needs no prefix sums and is
 * expanded in one streaming pass.  Every workgroup checks the groups it
 * expands; a small kernel enqueued behind reads one word and, only if some group
 * did not keep exactly 2 (a bitmask no 2:4 compressor wrote), redoes the tensor
 * as a general scatter.  Other shapes (values that are not half the elements,
 * rows that are not whole bitmask bytes) take the path of ctmi_bitmask_decompress
 * and use tmp: ctmi_sparse24_tmp_bytes(rows, cols, elem_size) bytes of device
 * scratch; it needs no initialisation.
 * The word the streaming workgroups report to is one of 256 pairs of words in device
 * memory of the library; each stream is given a pair of its own when it is first seen
 * (streams beyond 256 share).  A captured graph keeps the pair of its capture stream. */
int64_t ctmi_sparse24_tmp_bytes(int64_t rows, int64_t cols, int32_t elem_size);
int ctmi_sparse24_decompress(const void* values, int64_t nvalues, int32_t elem_size,
                             const uint8_t* bitmask, void* out, void* tmp, int64_t rows,
                             int64_t cols, void* stream);

/* ctmi_sparse24_compress / ctmi_sparse24_decompress for several tensors of one dtype
 * from one call, 8 per launch.  Every tensor must have rows of whole bitmask bytes
 * (cols % 8 == 0), a whole number of work items (rows * cols a multiple of 16 for
 * 1-byte elements, of 8 otherwise) and 16-byte aligned
 * buffers; for decompression also nvalues * 2 == rows * cols.  A job that does not
 * is refused with CTMI_ERR_UNSUPPORTED before anything is enqueued: give it a call
 * of its own.  `dense` is read by compress_many and written by decompress_many;
 * nvalues is ignored by compress_many. */
typedef struct ctmi_sparse24_job {
  void* dense;      /* [rows, cols] */
  void* values;     /* [rows, cols / 2] */
  uint8_t* bitmask; /* [rows, cols / 8] */
  int64_t nvalues;
  int64_t rows, cols;
} ctmi_sparse24_job;
int ctmi_sparse24_compress_many(const ctmi_sparse24_job* jobs, int64_t n_jobs, int32_t x_dtype,
                                void* stream);
int ctmi_sparse24_decompress_many(const ctmi_sparse24_job* jobs, int64_t n_jobs,
                                  int32_t elem_size, void* stream);

/* A20.  get_24_bytemasks (sparse_24_bitmask.py:227-260): top-2-of-4 by
 * |value| with torch.topk's tie order.  x_dtype: a float type (ranked on the
 * value), or CTMI_I8 / CTMI_F8E4M3, which are ranked as the reference ranks
 * its int8 view of fp8 data: abs() computed in int8, so abs(-128) == -128.
 * numel must be a multiple of 4.  mask: bool [numel]. */
int ctmi_get_24_bytemasks(const void* x, int32_t x_dtype, uint8_t* mask, int64_t numel,
                          void* stream);

/* A21.  sparse24_bitmask_compress (sparse_24_bitmask.py:162-203): values
 * [rows, cols/2] + packed bitmask [rows, ceil(cols/8)] in one pass. */
int ctmi_sparse24_compress(const void* x, int32_t x_dtype, void* values, uint8_t* bitmask,
                           int64_t rows, int64_t cols, void* stream);

/* A12 + A21 in one pass: the stacked case of ModelCompressor.compress
 * (model_compressors/model_compressor.py:638-667), a weight that is quantized to
 * fp8 / int8 codes (naive_quantized.py:79-114) and whose codes are then compressed
 * as 2:4 (sparse_24_bitmask.py:162-203), without the dense code tensor in between.
 * values: [rows, cols / 2] codes (float8_e4m3fn or int8); bitmask as in
 * ctmi_sparse24_compress.  Same bits as ctmi_qdq followed by ctmi_sparse24_compress.
 * _supported(): cols % 8 == 0, scales in x's dtype on a tensor / channel / group
 * grid, zero point (if any) in the codes' dtype, codes of 8 bits or fewer. */
int ctmi_quantize_sparse24_compress_supported(int32_t x_dtype, int64_t rows, int64_t cols,
                                              const ctmi_qparams* qp);
int ctmi_quantize_sparse24_compress(const void* x, int32_t x_dtype, void* values, uint8_t* bitmask,
                                    int64_t rows, int64_t cols, const ctmi_qparams* qp,
                                    void* stream);

/* A22 + A13 in one pass: the stacked case of ModelCompressor.decompress
 * (model_compressors/model_compressor.py:572-604, :694-760): the 2:4 values and bitmask of a
 * quantized weight are expanded (sparse_24_bitmask.py:206-224) and the codes
 * dequantized (naive_quantized.py:116-140) without the dense code tensor in between.
 * values: [rows, cols / 2] codes (float8_e4m3fn or int8), nvalues of them; out:
 * [rows, cols] of out_dtype, the dtype of the scales.  Same bits as
 * ctmi_sparse24_decompress followed by ctmi_qdq, also for a bitmask that is not 2:4
 * (set bits are then filled from `values` in order, as in ctmi_bitmask_decompress).
 * The codes are decoded by values_dtype (CTMI_I8 or CTMI_F8E4M3), whatever qp's type
 * says: dequantize() infers its arguments from the scale's shape alone.
 * _supported(): as for ctmi_quantize_sparse24_compress.  tmp is no longer used (what the
 * check for a bitmask that is not 2:4 needs lives inside the library, as for
 * ctmi_sparse24_decompress) and may be NULL; ctmi_sparse24_dequantize_tmp_bytes() is 0. */
int ctmi_sparse24_decompress_dequantize_supported(int32_t values_dtype, int32_t out_dtype,
                                                  int64_t rows, int64_t cols,
                                                  const ctmi_qparams* qp);
int64_t ctmi_sparse24_dequantize_tmp_bytes(int64_t rows, int64_t cols);
int ctmi_sparse24_decompress_dequantize(const void* values, int64_t nvalues, int32_t values_dtype,
                                        const uint8_t* bitmask, void* out, int32_t out_dtype,
                                        void* tmp, int64_t rows, int64_t cols,
                                        const ctmi_qparams* qp, void* stream);

/* One weight for the many-weight forms of the two entry points above.  dense: the dense
 * weight (read by compress, written by decompress), dense_dtype its dtype; values: the codes
 * that survive, [rows, cols/2] of values_dtype (CTMI_I8 or CTMI_F8E4M3; compress derives it
 * from qp and ignores the member); bitmask: uint8 [rows, cols/8]. */
typedef struct ctmi_stacked24_job {
  void* dense;
  void* values;
  uint8_t* bitmask;
  int64_t rows, cols;
  int32_t dense_dtype;
  int32_t values_dtype;
  ctmi_qparams qp;
} ctmi_stacked24_job;

/* ModelCompressor.compress / decompress over the weights of a model that are both quantized
 * to int8 / fp8 codes and 2:4 compressed (model_compressor.py:638-667, :572-604): n weights
 * from one call, same results as n calls of ctmi_quantize_sparse24_compress /
 * ctmi_sparse24_decompress_dequantize.  Every job is validated before anything is enqueued
 * (a layout without a fused kernel: CTMI_ERR_UNSUPPORTED, nothing enqueued); weights that
 * share a kernel instance are chained into common launches, 8 per launch. */
int ctmi_quantize_sparse24_compress_many(const ctmi_stacked24_job* jobs, int64_t n, void* stream);
int ctmi_sparse24_decompress_dequantize_many(const ctmi_stacked24_job* jobs, int64_t n, void* stream);

/* A1.  calculate_qparams (quantization/utils/helpers.py:67-146), elementwise
 * over n (min, max) pairs of dtype mm_dtype.  mm_is_0d != 0 when the reference
 * would see 0-d min/max tensors (their zero-point subtraction then promotes to
 * fp32).  scale_dtype must be mm_dtype, or CTMI_F8E4M3 for fp4 with a global
 * scale; zero_point may be NULL. */
int ctmi_calculate_qparams(const void* min_vals, const void* max_vals, int32_t mm_dtype,
                           int32_t mm_is_0d, int64_t n, int32_t qtype, int32_t num_bits,
                           int32_t symmetric, const float* global_scale, void* scale,
                           int32_t scale_dtype, void* zero_point, int32_t zp_dtype, void* stream);

/* A16.  generate_gparam (helpers.py:414-434): out[i] = fp32(448*6 / max|min,max|),
 * evaluated as torch evaluates `float / tensor`: reciprocal, then the product, each
 * rounded to the dtype of min / max. */
int ctmi_generate_gparam(const void* min_vals, const void* max_vals, int32_t mm_dtype, int64_t n,
                         float* out, void* stream);

/* A2 / A3.  amin / amax over cells of blk_rows x blk_cols elements of a
 * [rows, cols] tensor (observer reduction: tests/mock_observer.py:38-56,
 * helpers.py:199-203).  Outputs have x_dtype and shape
 * [ceil(rows/blk_rows), ceil(cols/blk_cols)].  tmp: ctmi_minmax_tmp_bytes()
 * bytes of device scratch, only needed when blk_rows > 1. */
int64_t ctmi_minmax_tmp_bytes(int64_t rows, int64_t cols, int64_t blk_rows, int64_t blk_cols,
                              int32_t x_dtype);
int ctmi_minmax(const void* x, int32_t x_dtype, int64_t rows, int64_t cols, int64_t blk_rows,
                int64_t blk_cols, void* min_out, void* max_out, void* tmp, void* stream);

/* A2 + A1 fused for cells one row tall (group / channel / token): min-max
 * reduction and calculate_qparams in one pass over x.  scale / zero_point:
 * [rows, ceil(cols/blk_cols)]; min_out / max_out optional (x_dtype). */
int ctmi_observe_qparams(const void* x, int32_t x_dtype, int64_t rows, int64_t cols,
                         int64_t blk_cols, int32_t qtype, int32_t num_bits, int32_t symmetric,
                         const float* global_scale, void* scale, int32_t scale_dtype,
                         void* zero_point, int32_t zp_dtype, void* min_out, void* max_out,
                         void* stream);

/* A2 + A1 + A5 + A9 fused: min-max observer (tests/mock_observer.py:38-113),
 * calculate_qparams (quantization/utils/helpers.py:67-146), quantize
 * (quantization/lifecycle/forward.py:45-81, 455-487) and pack_to_int32
 * (compressors/quantized_compressors/pack_quantized.py:186-246) in one pass over
 * a weight x[rows, cols], for cells of 1 x blk_cols elements (group: blk_cols =
 * group_size, channel: blk_cols = cols) and 4- or 8-bit integer codes: what
 * PackedQuantizationCompressor.compress_weight (pack_quantized.py:88-146)
 * returns for scales a min-max observer has just produced, with the weight read
 * once.  packed: int32 [rows, cols * num_bits / 32].  scale: [rows, cols /
 * blk_cols] in x_dtype.  zero_point: optional int8 [rows, cols / blk_cols]
 * (unpacked; asymmetric schemes pack it with ctmi_pack_to_int32, packed_dim 0).
 * ctmi_observe_pack_quantized_supported() says whether the layout has a kernel
 * (groups of 8, 16, ... 512 elements that tile the rows, or one cell per row of
 * up to 16384 elements, a multiple of 8). */
typedef struct ctmi_observe_pack_job {
  const void* x;
  int32_t* packed;
  void* scale;
  int8_t* zero_point; /* optional */
  int64_t rows, cols, blk_cols;
  int32_t x_dtype, num_bits, symmetric;
} ctmi_observe_pack_job;
int ctmi_observe_pack_quantized_supported(int32_t x_dtype, int64_t rows, int64_t cols,
                                          int64_t blk_cols, int32_t num_bits);
/* every weight of a state dict in one call: the group layouts share launches,
 * eight weights at a time */
int ctmi_observe_pack_quantized_many(const ctmi_observe_pack_job* jobs, int64_t n, void* stream);
int ctmi_observe_pack_quantized(const void* x, int32_t x_dtype, int64_t rows, int64_t cols,
                                int64_t blk_cols, int32_t num_bits, int32_t symmetric,
                                int32_t* packed, void* scale, int8_t* zero_point, void* stream);

/* The same pass for weights whose groups are not runs of neighbouring columns of a
 * power-of-two length: activation ordering (quantization/lifecycle/forward.py:286-303: the
 * columns are sorted by g_idx and the sorted order is cut into groups, so the observer
 * (tests/mock_observer.py:38-113 on the sorted columns) takes min / max over the columns of a
 * group wherever they sit) and column-ordered groups of any size that divides cols.
 * col_group: int32 [cols], the group of every column (ctmi_column_groups turns a g_idx into
 * it), or NULL for column / blk_cols.  scale: [rows, cols / blk_cols] in x_dtype; zero_point:
 * optional int8 of the same shape; packed: int32 [rows, cols * num_bits / 32].  Same bits as
 * the min-max observer on the weight with its columns sorted by col_group, followed by
 * ctmi_pack_quantized_compress with qp.col_group set.
 * _supported(): cols a multiple of 8 and of blk_cols, at most 16384; at most 256 groups a row;
 * 4- or 8-bit codes. */
int ctmi_observe_pack_quantized_gidx_supported(int32_t x_dtype, int64_t rows, int64_t cols,
                                               int64_t blk_cols, int32_t num_bits);
int ctmi_observe_pack_quantized_gidx(const void* x, int32_t x_dtype, int64_t rows, int64_t cols,
                                     int64_t blk_cols, int32_t num_bits, int32_t symmetric,
                                     const int32_t* col_group, int32_t* packed, void* scale,
                                     int8_t* zero_point, void* stream);

/* The same for the nvfp4 format with a known global scale: group-16 scales of the
 * observer (tests/mock_observer.py:38-113, helpers.py:101-120: fp8 e4m3, zeros
 * replaced by 0.125) and NVFP4PackedCompressor.compress_weight
 * (fp4_quantized.py:84-107) with those scales and their zero points (all zero),
 * the weight read once.  packed: uint8 [rows, cols/2]; scale: fp8 [rows, cols/16]. */
int ctmi_observe_nvfp4_compress(const void* x, int32_t x_dtype, int64_t rows, int64_t cols,
                                const float* global_scale, uint8_t* packed, uint8_t* scale,
                                void* stream);

/* every weight of a state dict in one call: weights of one dtype share launches, eight at
 * a time */
typedef struct ctmi_observe_nvfp4_job {
  const void* x;
  const float* global_scale;
  uint8_t* packed;
  uint8_t* scale;
  int64_t rows, cols;
  int32_t x_dtype, reserved;
} ctmi_observe_nvfp4_job;
int ctmi_observe_nvfp4_compress_many(const ctmi_observe_nvfp4_job* jobs, int64_t n, void* stream);

/* One tensor for ctmi_observe_qparams_many: x [rows, cols] of x_dtype, cells of 1 x blk_cols
 * elements; scale / zero_point [rows, ceil(cols / blk_cols)] (zero_point optional);
 * global_scale: the fp32 scalar of a tensor_group (nvfp4) scheme, else NULL. */
typedef struct ctmi_observe_job {
  const void* x;
  void* scale;
  void* zero_point;
  const float* global_scale;
  int64_t rows, cols, blk_cols;
  int32_t x_dtype;
  int32_t reserved;
} ctmi_observe_job;

/* A2 + A1 for the weights of a model in one call: what a calibration pass with the min-max
 * observer does module by module (tests/mock_observer.py:38-113 followed by calculate_qparams,
 * quantization/utils/helpers.py:67-146).  Same results as n calls of ctmi_observe_qparams
 * without min_out / max_out; tensors that share a dtype and a kernel are chained into common
 * launches, 8 per launch.  scale_dtype < 0: the dtype the reference produces for each tensor
 * (its own, or float8_e4m3fn for fp4 with a global scale).  Every job is validated before
 * anything is enqueued. */
int ctmi_observe_qparams_many(const ctmi_observe_job* jobs, int64_t n, int32_t qtype, int32_t num_bits,
                              int32_t symmetric, int32_t scale_dtype, int32_t zp_dtype, void* stream);

/* A26.  Dynamic activation quantization in one pass (forward_quantize with
 * args.dynamic, quantization/lifecycle/forward.py:414-451): the scales of
 * compute_dynamic_scales_and_zp (quantization/utils/helpers.py:149-205, via
 * calculate_qparams :67-146) for cells of 1 x blk_cols elements of x[rows, cols]
 * (token: blk_cols = cols; group / tensor_group: blk_cols = group_size), then
 * fake_quantize (forward.py:150-189) of x with them: out has x's dtype and
 * shape.  The tensor is read once.  scale_out / zp_out are optional
 * [rows, cols / blk_cols] outputs with the dtypes ctmi_observe_qparams documents.
 * global_scale: the fp32 scalar of a tensor_group (nvfp4) scheme, else NULL.
 * ctmi_dynamic_qdq_supported() says whether a layout has a fused kernel (int
 * <= 8 bits and fp8: cells of up to 16384 elements in multiples of 8; fp4 with
 * a global scale: cells of 16); CTMI_ERR_UNSUPPORTED otherwise,
 * and the caller runs ctmi_observe_qparams + ctmi_qdq. */
int ctmi_dynamic_qdq_supported(int32_t x_dtype, int64_t rows, int64_t cols, int64_t blk_cols,
                               int32_t qtype, int32_t num_bits, int32_t has_global_scale);
int ctmi_dynamic_qdq(const void* x, int32_t x_dtype, void* out, int64_t rows, int64_t cols,
                     int64_t blk_cols, int32_t qtype, int32_t num_bits, int32_t symmetric,
                     const float* global_scale, void* scale_out, int32_t scale_dtype,
                     void* zp_out, int32_t zp_dtype, void* stream);

/* N1 for the naive-quantized formats: one-shot compression of a weight that has no
 * scales yet.  The min-max observer (tests/mock_observer.py:38-113), calculate_qparams
 * (quantization/utils/helpers.py:67-146) and NaiveQuantizationCompressor.compress_weight
 * (naive_quantized.py:79-114: quantize with dtype = args.pytorch_dtype()) for cells of
 * 1 x blk_cols elements (channel: blk_cols = cols; group: blk_cols = group_size) from
 * one pass over x.  codes: int8 (integer grids of up to 8 bits) or float8_e4m3fn
 * [rows, cols]; scale_out [rows, cols / blk_cols] in scale_dtype; zp_out optional.
 * Same bits as ctmi_observe_qparams followed by ctmi_qdq.  _supported() as for
 * ctmi_dynamic_qdq. */
int ctmi_observe_quantize_supported(int32_t x_dtype, int64_t rows, int64_t cols, int64_t blk_cols,
                                    int32_t qtype, int32_t num_bits);
int ctmi_observe_quantize(const void* x, int32_t x_dtype, void* codes, int64_t rows, int64_t cols,
                          int64_t blk_cols, int32_t qtype, int32_t num_bits, int32_t symmetric,
                          void* scale_out, int32_t scale_dtype, void* zp_out, int32_t zp_dtype,
                          void* stream);

/* The same for the block strategy (cells of blk_rows x blk_cols elements, the observer's
 * reshape in tests/mock_observer.py:95-113; e.g. 128 x 128 fp8 blocks): one workgroup holds
 * a block in registers, so the weight is still read once.  scale_out / zp_out:
 * [rows / blk_rows, cols / blk_cols].  Blocks must tile the tensor, be a multiple of 8
 * wide and hold at most 16384 elements.  Same bits as ctmi_minmax + ctmi_calculate_qparams
 * + ctmi_qdq. */
int ctmi_observe_quantize_blocks_supported(int32_t x_dtype, int64_t rows, int64_t cols,
                                           int64_t blk_rows, int64_t blk_cols, int32_t qtype,
                                           int32_t num_bits);
int ctmi_observe_quantize_blocks(const void* x, int32_t x_dtype, void* codes, int64_t rows,
                                 int64_t cols, int64_t blk_rows, int64_t blk_cols, int32_t qtype,
                                 int32_t num_bits, int32_t symmetric, void* scale_out,
                                 int32_t scale_dtype, void* zp_out, int32_t zp_dtype, void* stream);

/* every weight of a state dict in one call: rows of one length class share launches,
 * eight weights at a time; scale_dtype < 0: every weight's scales in its own dtype */
typedef struct ctmi_observe_quantize_job {
  const void* x;
  void* codes;
  void* scale;
  void* zero_point; /* optional */
  int64_t rows, cols, blk_cols;
  int32_t x_dtype, reserved;
} ctmi_observe_quantize_job;
int ctmi_observe_quantize_many(const ctmi_observe_quantize_job* jobs, int64_t n, int32_t qtype,
                               int32_t num_bits, int32_t symmetric, int32_t scale_dtype,
                               int32_t zp_dtype, void* stream);

/* ctmi_observe_quantize_blocks for every weight of a state dict in one call (blocks of one
 * size class share launches, eight weights at a time).  Every job must be one that
 * ctmi_observe_quantize_blocks_supported accepts; the whole list is checked before anything
 * is enqueued.  scale_dtype < 0: every weight's scales in its own dtype. */
typedef struct ctmi_observe_quantize_blocks_job {
  const void* x;
  void* codes;
  void* scale;      /* [rows / blk_rows, cols / blk_cols] */
  void* zero_point; /* optional */
  int64_t rows, cols, blk_rows, blk_cols;
  int32_t x_dtype, reserved;
} ctmi_observe_quantize_blocks_job;
int ctmi_observe_quantize_blocks_many(const ctmi_observe_quantize_blocks_job* jobs, int64_t n,
                                      int32_t qtype, int32_t num_bits, int32_t symmetric,
                                      int32_t scale_dtype, int32_t zp_dtype, void* stream);

/* MXFP4 group scales (quantization/utils/mxfp4_utils.py): powers of two held as
 * uint8 exponents.  x / out of the first two are bfloat16 group maxima, n values.
 *   ctmi_mxfp4_round_to_power_2   :41-73  (x + 32) & 0xFF80 on the bf16 bits
 *   ctmi_mxfp4_generate_scales    :76-97  127 + floor(log2(round_to_power_2(x))) - 2,
 *                                         clamped to [0, 255]
 *   ctmi_mxfp4_convert_exp_scale  :24-38  2 ** (e - 127) in out_dtype (f32 / f16 / bf16) */
int ctmi_mxfp4_round_to_power_2(const void* x, void* out, int64_t n, void* stream);
int ctmi_mxfp4_generate_scales(const void* x, uint8_t* out, int64_t n, void* stream);
int ctmi_mxfp4_convert_exp_scale(const uint8_t* exps, void* out, int32_t out_dtype, int64_t n,
                                 void* stream);

/* Activation ordering (quantization/lifecycle/forward.py:286-303): the reference
 * sorts the columns of a weight by g_idx and cuts the sorted order into runs of
 * group_size.  col_group[c] = (place of column c in a stable sort by g_idx) /
 * group_size is that rule as a per-column group index, the form ctmi_qparams
 * takes; a g_idx that holds a -1 is unset and gives column order (c / group_size).
 * g_idx may hold any int32 values (they are ordered as signed integers, like
 * torch.argsort orders them); cols < 65536.  No scratch, no host sync. */
int ctmi_column_groups(const int32_t* g_idx, int64_t cols, int64_t group_size,
                       int32_t* col_group, void* stream);

/* A24 / A25.  Hadamard transform apply (transform/utils/matrix.py:65-171,
 * transform/factory/hadamard.py:104-121) for a matrix given in factored form
 *     W = diag(sign_in) * (Ma (x) Mb) * diag(sign_out),      n = a_dim * b_dim:
 * every run of n consecutive elements x of the tensor (numel % n == 0) becomes
 *     x * W / sqrt(n)
 * rounded to io_dtype.  ma_t / mb_t: Ma^T [a,a] and Mb^T [b,b] as bf16 (entries
 * must be exact in bf16, e.g. +-1); ma_t is ignored when a_dim == 1.  sign_in /
 * sign_out: fp32 [n] or NULL.  Runs on bf16 MFMA; ctmi_hadamard_supported says
 * which (a_dim, b_dim, dtype) combinations are built. */
int ctmi_hadamard_supported(int32_t a_dim, int32_t b_dim, int32_t io_dtype);
/* mb_t == NULL (with a_dim > 1) stands for Mb = Sylvester's matrix of order b_dim, the form of
 * the reference's Hadamard matrices of size K * 2^m (transform/utils/hadamard.py:132-163: a
 * known K x K block times butterflies).  Then only the product with Ma runs on the matrix
 * cores (16-bit inputs: exact in one product) and Mb is butterfly stages on its fp32 result:
 * b_dim 4, 8, 16, 32 or 64 with a_dim up to 256 (above 224: two launches, out must not be x), or
 * b_dim 128 with a_dim up to 224 (any block; the reference takes the largest
 * block of its table, so the sizes met are 192 x 16 = 3072, 224 x 16 = 3584, 160 x 32 = 5120,
 * 224 x 32 = 7168, 224 x 64 = 14336, 224 x 128 = 28672 ...), bfloat16 or float16 tensors,
 * signs on one side
 * (ctmi_hadamard_sylvester_inner_supported).
 * mb_t == NULL with a_dim == 1, b_dim == 128 and bfloat16 tensors: Sylvester's matrix of 128
 * (what the reference uses at this size) from a kernel that keeps no matrix in memory; same
 * bits as with the matrix passed.  Tensors and sign vectors 16-byte aligned. */
int ctmi_hadamard_sylvester_inner_supported(int32_t a_dim, int32_t b_dim, int32_t io_dtype);
int ctmi_hadamard_apply(const void* x, void* out, int32_t io_dtype, int64_t numel, int32_t a_dim,
                        int32_t b_dim, const void* ma_t, const void* mb_t, const float* sign_in,
                        const float* sign_out, void* stream);

/* The same transform on several tensors (the weights of a model that share a
 * rotation, transform/factory/hadamard.py:46-67 hands one matrix to every module of
 * a scheme) from one call: tensors share launches, 8 at a time, so that the set-up
 * of the matrix is paid once per launch and not once per tensor. */
typedef struct ctmi_hadamard_job {
  const void* x;
  void* out;
  int64_t numel;
} ctmi_hadamard_job;
int ctmi_hadamard_apply_many(const ctmi_hadamard_job* jobs, int64_t n_jobs, int32_t io_dtype,
                             int32_t a_dim, int32_t b_dim, const void* ma_t, const void* mb_t,
                             const float* sign_in, const float* sign_out, void* stream);

/* A24 / A25 + A2 + A1 + A11 in one pass, for bf16 tensors, block size b_dim (32,
 * 64 or 128) equal to the quantization group size, symmetric 4-bit integers:
 * the rotation of ctmi_hadamard_apply (a_dim == 1) followed, per rotated block,
 * by the min-max observer, calculate_qparams and the quantize + pack_to_int32 of
 * ctmi_pack_quantized_compress.  Same bits as those calls in sequence.
 * packed: int32 [numel / 8]; scale: bf16 [numel / b_dim] (the group scales, row
 * major); rotated: optional bf16 [numel] copy of the rotated tensor, or NULL.
 * mb_t == NULL with b_dim == 128 stands for Sylvester's matrix of that order (what
 * deterministic_hadamard_matrix and random_hadamard_matrix build at this size,
 * transform/utils/hadamard.py:38-100): no matrix is read, and workgroups stream through
 * the tensor without a set-up phase; the sign vectors must then be 16-byte aligned.  A
 * rotated output that is exactly zero carries the sign of its sign_out entry there (-0
 * where the kernel with a matrix gives +0); codes and scales do not depend on it. */
int ctmi_hadamard_quant_pack(const void* x, int32_t io_dtype, int64_t numel, int32_t b_dim,
                             const void* mb_t, const float* sign_in, const float* sign_out,
                             int32_t num_bits, int32_t symmetric, int32_t* packed, void* scale,
                             void* rotated, void* stream);

/* ctmi_hadamard_quant_pack for several tensors from one call, 8 per launch. */
typedef struct ctmi_hadamard_pack_job {
  const void* x;
  int32_t* packed;
  void* scale;
  void* rotated; /* or NULL */
  int64_t numel;
} ctmi_hadamard_pack_job;
int ctmi_hadamard_quant_pack_many(const ctmi_hadamard_pack_job* jobs, int64_t n_jobs,
                                  int32_t io_dtype, int32_t b_dim, const void* mb_t,
                                  const float* sign_in, const float* sign_out, int32_t num_bits,
                                  int32_t symmetric, void* stream);

/* The same pipeline for transforms of size a_dim * b_dim = 32 x 64 or 64 x 64 (2048, 4096)
 * with group size 128: ctmi_hadamard_apply (factored form, ma_t / mb_t as there), the
 * symmetric int4 min-max observer over groups of 128 and ctmi_pack_quantized_compress in
 * one pass; same bits as those calls in sequence.  packed: int32 [numel / 8]; scale: bf16
 * [numel / 128]; rotated optional. */
int ctmi_hadamard_kron_quant_pack_many(const ctmi_hadamard_pack_job* jobs, int64_t n_jobs,
                                       int32_t io_dtype, int32_t a_dim, int32_t b_dim,
                                       const void* ma_t, const void* mb_t, const float* sign_in,
                                       const float* sign_out, int32_t group_size, int32_t num_bits,
                                       int32_t symmetric, void* stream);

/* A23 / A24 for the reference's own matrices of a power-of-two size n = 1024, 2048, 4096 or
 * 8192: Sylvester's H_n (deterministic_hadamard_matrix, transform/utils/hadamard.py:33-62)
 * and diag(signs) * H_n (random_hadamard_matrix, :65-89, whose table of known blocks holds
 * Sylvester's matrices for these sizes).  Every run of n elements x becomes
 *     x * diag(sign_in) * H_n * diag(sign_out) / sqrt(n)
 * (transform/factory/hadamard.py:104-121) rounded to io_dtype (bf16 / f16 / f32), computed
 * as log2(n) butterfly stages in fp32 registers: no matrix is read and nothing is rounded
 * before the end.  sign_in / sign_out: fp32 [n] or NULL, 16-byte aligned like the tensors.
 * Several tensors share a launch, 8 at a time. */
int ctmi_sylvester_supported(int32_t n, int32_t io_dtype);
int ctmi_sylvester_apply_many(const ctmi_hadamard_job* jobs, int64_t n_jobs, int32_t io_dtype,
                              int32_t n, const float* sign_in, const float* sign_out, void* stream);

/* ... followed in the same pass by the W4A16 pipeline of ctmi_hadamard_kron_quant_pack_many
 * (bf16 tensors, symmetric int4, group size 128): same bits as ctmi_sylvester_apply_many and
 * ctmi_observe_pack_quantized in sequence.  packed: int32 [numel / 8]; scale: bf16
 * [numel / 128]; rotated optional. */
int ctmi_sylvester_quant_pack_many(const ctmi_hadamard_pack_job* jobs, int64_t n_jobs,
                                   int32_t io_dtype, int32_t n, const float* sign_in,
                                   const float* sign_out, int32_t group_size, int32_t num_bits,
                                   int32_t symmetric, void* stream);

/* A23 / A24 for matrices with an explicit factor (transform/utils/matrix.py:137-171 for
 * a small explicit matrix; transform/utils/hadamard.py:102-163 for the reference's
 * Hadamard matrices of size K * 2^m built from its table of known K x K matrices,
 * diag(Q) * (H_K^T (x) Sylvester(2^m)), e.g. 14336 = 224 * 64).  Every run of h * b
 * consecutive elements x, viewed as X[h, b] after the optional sign_in, becomes
 *     vec(w^T X S_b) * sign_out * scale        (sylvester != 0, S_b = Sylvester(b))
 *     vec(w^T X)     * sign_out * scale        (sylvester == 0)
 * i.e. x * diag(sign_in) * (w (x) S_b) * diag(sign_out) * scale, rounded once to
 * io_dtype (scale = 1 / sqrt(h * b) makes a Hadamard rotation orthonormal).  w: fp32
 * [h, h] row-major (any values); sign_in / sign_out: fp32 [h * b] or NULL; b a power of
 * two up to 256 and h * b * 4 bytes within 159 KB; for b = 1, 64 runs share a workgroup
 * and h may be at most 313; for h = 1 with the Sylvester factor b may be 512 (the
 * butterflies stay in a wavefront's registers) or 1024, 2048, 4096, 8192 (the kernel of
 * ctmi_sylvester_apply_many; tensors and sign vectors 16-byte aligned);
 * ctmi_kron_matmul_supported tells.  fp32 accumulation on the vector ALUs. */
int ctmi_kron_matmul_supported(int32_t h, int32_t b, int32_t io_dtype);
int ctmi_kron_matmul(const void* x, void* out, int32_t io_dtype, int64_t numel, int32_t h,
                     int32_t b, const float* w, const float* sign_in, const float* sign_out,
                     int32_t sylvester, float scale, void* stream);

/* A24 for an arbitrary explicit fp32 matrix w [h,h] (h up to 313; matrices that are not
 * +-1 included): every run of h consecutive elements x becomes x * w / sqrt(h).  The case
 * b = 1, scale = 1 / sqrt(h) of ctmi_kron_matmul. */
int ctmi_block_matmul(const void* x, void* out, int32_t io_dtype, int64_t numel, int32_t h,
                      const float* w, void* stream);

/* Diagnostics, not part of the path: a plain device-to-device copy of `bytes` bytes (a
 * multiple of 16), the known quantity against which hardware byte counters are calibrated
 * when profiling (bench.py --calib-copies).  Nothing in the library or its host mirror
 * calls it.  No counterpart in the reference. */
int ctmi_calib_copy(const void* src, void* dst, int64_t bytes, void* stream);

/* The 4096-entry keep table used by the 2:4 kernels (host copy, for tests). */
void ctmi_topk24_lut(uint8_t* out4096);

#ifdef __cplusplus
}
#endif
#endif /* CTMI_H_ */
