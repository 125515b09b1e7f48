// Dynamic activation quantization in one pass: the scales come from the tensor
// itself, which is then fake-quantized with them while still in registers.
//
//   forward_quantize, args.dynamic            quantization/lifecycle/forward.py:414-451
//     compute_dynamic_scales_and_zp           quantization/utils/helpers.py:149-205
//     calculate_qparams                       helpers.py:67-146
//     fake_quantize                           forward.py:150-189
//
// The reference runs these one after the other (the tensor is read for the
// min / max, read again and written by fake_quantize); the arithmetic here is the
// same, step for step, on data that is read once: 4 bytes per bf16 element
// instead of 6.
//
// The same kernels with codes for output (int8 or fp8 instead of the fake-quantized
// tensor) are the one-shot form of the naive-quantized compressors: min-max
// observer (tests/mock_observer.py:38-113), calculate_qparams and
// NaiveQuantizationCompressor.compress_weight (naive_quantized.py:79-114) over a
// weight that is read once.
#include <type_traits>

#include "ctmi_device.h"
#include "ctmi_host.h"
#include "minmax.h"
#include "qdq_core.h"
#include "qparams.h"
#include "quant_core.h"
#include "quant_fast.h"

namespace ctmi {

int fill_qpcfg(QpCfg* c, int qtype, int num_bits, int symmetric, int mt, int mm_is_0d,
               bool has_gscale, int scale_dtype, int zp_dtype);
bool nvfp4_dynamic_try(const void* x, int x_dtype, void* out, int64_t rows, int64_t cols,
                       int64_t blk_cols, const float* gscale, void* scale_out, void* zp_out,
                       const QpCfg& c, hipStream_t st);

struct DynOut {
  void* scale;  // optional
  void* zp;     // optional
};

// scale and zero point of a cell from its min / max (float path) -- the caller has
// folded NaNs into has_nan
template <typename FT, int QK, bool SYM>
__device__ __forceinline__ void cell_qparams(float lo, float hi, bool has_nan, float qmin,
                                             float qmax, float* sv, float* zv) {
  if constexpr (SYM) {
    *sv = symmetric_scale<FT>(__builtin_fmaxf(__builtin_fmaxf(-lo, hi), 0.0f), has_nan,
                              (qmax - qmin) * 0.5f);
    *zv = 0.0f;  // zeros whatever the data holds
  } else {
    asymmetric_qparams<FT, QK>(lo, hi, has_nan, qmin, qmax, sv, zv);
  }
}

__device__ __forceinline__ void store_cell(const DynOut& o, int64_t cell, float sv, float zv,
                                           int scale_dtype, int zp_dtype) {
  if (o.scale) store_from_f32(o.scale, scale_dtype, cell, sv);
  if (o.zp) store_from_f32(o.zp, zp_dtype, cell, zv);
}

// Item `v` of the output: the fake-quantized values, or (CODES) the int8 / fp8 codes
// that quantize(dtype=args.pytorch_dtype()) returns
template <typename FT, int QK, bool CODES>
__device__ __forceinline__ void store_result(void* out_any, int64_t v, bool keep,
                                             const Vec<typename FT::raw, 8>& a, float sv, float zv,
                                             const QpCfg& c) {
  using FR = typename FT::raw;
  Vec<FR, 8> of;
  Vec<uint8_t, 8> oc;
  if constexpr (CODES) {
    constexpr int kOut = QK == 0 ? kKindI8 : kKindF8;
    qdq_vec8<FT, kKindFloat, kOut, QK, true>(a, oc, sv, zv, c.bit_min, c.bit_max, &of, &oc);
    if (keep) stg_nt<uint8_t, 8>(static_cast<uint8_t*>(out_any) + v * 8, oc);
  } else {
    qdq_vec8<FT, kKindFloat, kKindFloat, QK, true>(a, oc, sv, zv, c.bit_min, c.bit_max, &of, &oc);
    if (keep) stg_nt<FR, 8>(static_cast<FR*>(out_any) + v * 8, of);
  }
}

// One workgroup of 256 threads per row-long segment (token / channel) of up to
// 256 * U vectors of 8 elements: every vector is loaded before anything is looked
// at; the four wavefronts meet once, over a few words in LDS.
// Where the vectors of a cell lie.  A row-long segment is one run of vectors; a block of
// the block strategy (observer reshape of tests/mock_observer.py:95-113: cells of
// block_height x block_width elements) is `ipr` vectors in each of its rows.
struct CellLayout {
  int ipr;          // vectors per row of the cell (0: the cell is one run of vectors)
  int row_pitch;    // vectors per row of the tensor
  int cells_per_row;
  int cell_rows;
};

template <bool BLOCK>
__device__ __forceinline__ int64_t cell_vector(const CellLayout& g, int64_t s, int items, int i) {
  if constexpr (!BLOCK) {
    return s * (int64_t)items + i;
  } else {
    const int64_t br = s / g.cells_per_row, bc = s - br * g.cells_per_row;
    const int r = i / g.ipr, ci = i - r * g.ipr;
    return (br * g.cell_rows + r) * (int64_t)g.row_pitch + bc * g.ipr + ci;
  }
}

template <typename FT, int QK, bool SYM, int U, bool CODES, bool BLOCK = false>
__device__ __forceinline__ void rows_segment(const typename FT::raw* __restrict__ x,
                                             void* __restrict__ out_any, const DynOut& o, int items,
                                             int64_t s, const QpCfg& c,
                                             const CellLayout& g = CellLayout{0, 0, 0, 0}) {
  using FR = typename FT::raw;
  __shared__ float part_lo[4], part_hi[4];
  __shared__ int part_word[4];
  Vec<FR, 8> a[U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int i = k * 256 + threadIdx.x;
    // past the end: re-reads do not change min / max
    a[k] = ldg_nt<FR, 8>(x + cell_vector<BLOCK>(g, s, items, i < items ? i : items - 1) * 8);
  }
  float sv, zv;
  if constexpr (SYM && sizeof(FR) == 2) {
    uint32_t m = 0;
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const uint32_t mk = absmax8_bits<FT>(a[k]);
      m = mk > m ? mk : m;
    }
    m = group_umax(64, m);
    if ((threadIdx.x & 63) == 0) part_word[threadIdx.x >> 6] = (int)m;
    __syncthreads();
    const uint32_t m01 = max((uint32_t)part_word[0], (uint32_t)part_word[1]);
    const uint32_t m23 = max((uint32_t)part_word[2], (uint32_t)part_word[3]);
    m = max(m01, m23);
    constexpr uint32_t kInf = FT::id == CTMI_BF16 ? 0x7f80u : 0x7c00u;
    sv = symmetric_scale<FT>(FT::to_f32((FR)m), m > kInf, (c.bit_max - c.bit_min) * 0.5f);
    zv = 0.0f;
  } else {
    float lo = __builtin_inff(), hi = -__builtin_inff();
    bool unordered = false;
#pragma unroll
    for (int k = 0; k < U; ++k) vec_minmax<FT>(a[k], &lo, &hi, &unordered);
    group_minmax(64, &lo, &hi);
    unordered = group_any(64, unordered);
    if ((threadIdx.x & 63) == 0) {
      part_lo[threadIdx.x >> 6] = lo;
      part_hi[threadIdx.x >> 6] = hi;
      part_word[threadIdx.x >> 6] = unordered;
    }
    __syncthreads();
    lo = __builtin_fminf(__builtin_fminf(part_lo[0], part_lo[1]), __builtin_fminf(part_lo[2], part_lo[3]));
    hi = __builtin_fmaxf(__builtin_fmaxf(part_hi[0], part_hi[1]), __builtin_fmaxf(part_hi[2], part_hi[3]));
    unordered = (part_word[0] | part_word[1] | part_word[2] | part_word[3]) != 0;
    cell_qparams<FT, QK, SYM>(lo, hi, unordered, c.bit_min, c.bit_max, &sv, &zv);
  }
  if (threadIdx.x == 0) store_cell(o, s, sv, zv, c.scale_dtype, c.zp_dtype);
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int i = k * 256 + threadIdx.x;
    store_result<FT, QK, CODES>(out_any, cell_vector<BLOCK>(g, s, items, i < items ? i : 0), i < items,
                                a[k], sv, zv, c);
  }
}

// one workgroup per block of the block strategy, the whole block in registers
template <typename FT, int QK, bool SYM, int U>
__global__ void __launch_bounds__(256)
observe_quantize_blocks_kernel(const typename FT::raw* __restrict__ x, void* __restrict__ codes,
                               DynOut o, int items, CellLayout g, QpCfg c) {
  rows_segment<FT, QK, SYM, U, true, true>(x, codes, o, items, blockIdx.x, c, g);
}

template <typename FT, int QK, bool SYM, int U, bool CODES>
__global__ void __launch_bounds__(256)
dynamic_rows_kernel(const typename FT::raw* __restrict__ x, void* __restrict__ out_any,
                    DynOut o, int items, QpCfg c) {
  rows_segment<FT, QK, SYM, U, CODES>(x, out_any, o, items, blockIdx.x, c);
}

// The same for up to kDynMaxJobs tensors per launch: a workgroup finds its tensor by the
// running totals of segments (all wave-uniform).
constexpr int kDynMaxJobs = 8;
struct DynJobs {
  const void* x[kDynMaxJobs];
  void* out[kDynMaxJobs];
  DynOut o[kDynMaxJobs];
  int64_t end[kDynMaxJobs];  // running total of segments, job 0 .. j (unused: INT64_MAX)
  int items[kDynMaxJobs];
};

template <typename FT, int QK, bool SYM, int U, bool CODES>
__global__ void __launch_bounds__(256) dynamic_rows_many_kernel(DynJobs t, QpCfg c) {
  const int64_t s = blockIdx.x;
  int j = 0;
  int64_t first = 0;
#pragma unroll
  for (int i = 0; i < kDynMaxJobs - 1; ++i) {
    const bool past = s >= t.end[i];
    j = past ? i + 1 : j;
    first = past ? t.end[i] : first;
  }
  rows_segment<FT, QK, SYM, U, CODES>(static_cast<const typename FT::raw*>(t.x[j]), t.out[j], t.o[j],
                                      t.items[j], s - first, c);
}

// Blocks of up to kDynMaxJobs tensors per launch (one workgroup per block, as above)
struct DynBlockJobs {
  const void* x[kDynMaxJobs];
  void* out[kDynMaxJobs];
  DynOut o[kDynMaxJobs];
  int64_t end[kDynMaxJobs];  // running total of blocks, job 0 .. j (unused: INT64_MAX)
  int items[kDynMaxJobs];
  CellLayout g[kDynMaxJobs];
};

template <typename FT, int QK, bool SYM, int U>
__global__ void __launch_bounds__(256) observe_quantize_blocks_many_kernel(DynBlockJobs t, QpCfg c) {
  const int64_t s = blockIdx.x;
  int j = 0;
  int64_t first = 0;
#pragma unroll
  for (int i = 0; i < kDynMaxJobs - 1; ++i) {
    const bool past = s >= t.end[i];
    j = past ? i + 1 : j;
    first = past ? t.end[i] : first;
  }
  rows_segment<FT, QK, SYM, U, true, true>(static_cast<const typename FT::raw*>(t.x[j]), t.out[j], t.o[j],
                                           t.items[j], s - first, c, t.g[j]);
}

// Segments of L vectors, L a power of two <= 64 (group strategies): L neighbouring
// lanes own a segment; memory is one run of vectors numbered like the segments.
template <typename FT, int QK, bool SYM, bool CODES>
__global__ void __launch_bounds__(256)
dynamic_flat_kernel(const typename FT::raw* __restrict__ x, void* __restrict__ out_any,
                    DynOut o, int64_t nvec, int L, QpCfg c) {
  using FR = typename FT::raw;
  constexpr int U = 2;
  const int64_t v0 = (int64_t)blockIdx.x * (256 * U) + threadIdx.x;
  Vec<FR, 8> a[U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t v = v0 + k * 256;
    a[k] = ldg_nt<FR, 8>(x + (v < nvec ? v : nvec - 1) * 8);
  }
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t v = v0 + k * 256;
    float sv, zv;
    if constexpr (SYM && sizeof(FR) == 2) {
      const uint32_t m = group_umax(L, absmax8_bits<FT>(a[k]));
      constexpr uint32_t kInf = FT::id == CTMI_BF16 ? 0x7f80u : 0x7c00u;
      sv = symmetric_scale<FT>(FT::to_f32((FR)m), m > kInf, (c.bit_max - c.bit_min) * 0.5f);
      zv = 0.0f;
    } else {
      float lo = __builtin_inff(), hi = -__builtin_inff();
      bool unordered = false;
      vec_minmax<FT>(a[k], &lo, &hi, &unordered);
      group_minmax(L, &lo, &hi);
      cell_qparams<FT, QK, SYM>(lo, hi, group_any(L, unordered), c.bit_min, c.bit_max, &sv, &zv);
    }
    if (v < nvec && (threadIdx.x & (L - 1)) == 0) store_cell(o, v / L, sv, zv, c.scale_dtype, c.zp_dtype);
    store_result<FT, QK, CODES>(out_any, v, v < nvec, a[k], sv, zv, c);
  }
}

template <typename FT, int QK, bool SYM, bool CODES>
static bool launch_dynamic(const void* x, void* out, const DynOut& o, int64_t rows, int64_t cols,
                           int64_t blk_cols, const QpCfg& c, hipStream_t st) {
  using FR = typename FT::raw;
  const int64_t seg = blk_cols < cols ? blk_cols : cols;
  if (seg % 8 || cols % seg) return false;
  const int64_t items = seg / 8, nvec = rows * cols / 8, n_segments = rows * (cols / seg);
  if (items <= 64 && (items & (items - 1)) == 0) {
    const int64_t blocks = cdiv(nvec, 256 * 2);
    if (blocks >= (1ll << 31)) return false;
    hipLaunchKernelGGL((dynamic_flat_kernel<FT, QK, SYM, CODES>), (unsigned)blocks, 256, 0, st,
                       (const FR*)x, out, o, nvec, (int)items, c);
    return true;
  }
  if (n_segments >= (1ll << 31)) return false;
#define CTMI_DYN(UU)                                                                    \
  hipLaunchKernelGGL((dynamic_rows_kernel<FT, QK, SYM, UU, CODES>), (unsigned)n_segments, 256, 0, st, \
                     (const FR*)x, out, o, (int)items, c)
  if (items <= 256) CTMI_DYN(1);
  else if (items <= 256 * 2) CTMI_DYN(2);
  else if (items <= 256 * 4) CTMI_DYN(4);
  else if (items <= 256 * 8) CTMI_DYN(8);
  else return false;
#undef CTMI_DYN
  return true;
}

}  // namespace ctmi

using namespace ctmi;

extern "C" int ctmi_dynamic_qdq_supported(int32_t x_dtype, int64_t rows, int64_t cols,
                                          int64_t blk_cols, int32_t qtype, int32_t num_bits,
                                          int32_t has_global_scale) {
  if (x_dtype != CTMI_BF16 && x_dtype != CTMI_F16 && x_dtype != CTMI_F32) return 0;
  if (rows < 1 || cols < 1 || blk_cols < 1) return 0;
  const int64_t seg = blk_cols < cols ? blk_cols : cols;
  if (seg % 8 || cols % seg) return 0;
  const int64_t items = seg / 8;
  if (qtype == CTMI_QTYPE_FLOAT && num_bits == 4)
    return has_global_scale && items == 2;  // nvfp4: groups of 16
  if (has_global_scale) return 0;
  if (!((qtype == CTMI_QTYPE_INT && num_bits <= 8) || (qtype == CTMI_QTYPE_FLOAT && num_bits == 8)))
    return 0;
  return items <= 2048;
}

extern "C" int ctmi_dynamic_qdq(const void* x, int32_t x_dtype, void* out, int64_t rows,
                                int64_t cols, int64_t blk_cols, int32_t qtype, int32_t num_bits,
                                int32_t symmetric, const float* global_scale, void* scale_out,
                                int32_t scale_dtype, void* zp_out, int32_t zp_dtype, void* stream) {
  CTMI_REQUIRE(rows >= 1 && cols >= 1, CTMI_ERR_VALUE, "cannot observe an empty tensor");
  CTMI_REQUIRE(blk_cols >= 1, CTMI_ERR_VALUE, "empty cell");
  QpCfg c;
  int rc = fill_qpcfg(&c, qtype, num_bits, symmetric, x_dtype, 0, global_scale != nullptr,
                      scale_dtype, zp_dtype);
  if (rc) return rc;
  CTMI_REQUIRE(x && out, CTMI_ERR_VALUE, "NULL tensor pointer");
  CTMI_REQUIRE(ctmi_dynamic_qdq_supported(x_dtype, rows, cols, blk_cols, qtype, num_bits,
                                          global_scale != nullptr),
               CTMI_ERR_UNSUPPORTED,
               "no fused kernel for this layout: compute the scales and fake-quantize separately");
  const int bytes = 8 * dtype_size(x_dtype);
  CTMI_REQUIRE((uintptr_t)x % bytes == 0 && (uintptr_t)out % bytes == 0, CTMI_ERR_VALUE,
               "tensors must be aligned to 8 elements");
  hipStream_t st = (hipStream_t)stream;
  const DynOut o{scale_out, zp_out};
  bool ok;
  if (qtype == CTMI_QTYPE_FLOAT && num_bits == 4) {
    ok = nvfp4_dynamic_try(x, x_dtype, out, rows, cols, blk_cols, global_scale, scale_out, zp_out,
                           c, st);
  } else {
    const int qk = qtype == CTMI_QTYPE_INT ? 0 : 1;
#define CTMI_DYN_SYM(FT, QK)                                                               \
  (symmetric ? launch_dynamic<FT, QK, true, false>(x, out, o, rows, cols, blk_cols, c, st) \
             : launch_dynamic<FT, QK, false, false>(x, out, o, rows, cols, blk_cols, c, st))
#define CTMI_DYN_FT(FT) (qk == 0 ? CTMI_DYN_SYM(FT, 0) : CTMI_DYN_SYM(FT, 1))
    ok = x_dtype == CTMI_BF16 ? CTMI_DYN_FT(BF16)
                              : (x_dtype == CTMI_F16 ? CTMI_DYN_FT(F16) : CTMI_DYN_FT(F32));
#undef CTMI_DYN_SYM
#undef CTMI_DYN_FT
  }
  CTMI_REQUIRE(ok, CTMI_ERR_UNSUPPORTED, "no fused kernel for this layout");
  return check_launch("ctmi_dynamic_qdq");
}

extern "C" int ctmi_observe_quantize_supported(int32_t x_dtype, int64_t rows, int64_t cols,
                                               int64_t blk_cols, int32_t qtype, int32_t num_bits) {
  if (qtype == CTMI_QTYPE_FLOAT && num_bits != 8) return 0;
  return ctmi_dynamic_qdq_supported(x_dtype, rows, cols, blk_cols, qtype, num_bits, 0);
}

extern "C" int ctmi_observe_quantize(const void* x, int32_t x_dtype, void* codes, int64_t rows,
                                     int64_t cols, int64_t blk_cols, int32_t qtype,
                                     int32_t num_bits, int32_t symmetric, void* scale_out,
                                     int32_t scale_dtype, void* zp_out, int32_t zp_dtype,
                                     void* stream) {
  CTMI_REQUIRE(rows >= 1 && cols >= 1, CTMI_ERR_VALUE, "cannot observe an empty tensor");
  CTMI_REQUIRE(blk_cols >= 1, CTMI_ERR_VALUE, "empty cell");
  QpCfg c;
  int rc = fill_qpcfg(&c, qtype, num_bits, symmetric, x_dtype, 0, false, scale_dtype, zp_dtype);
  if (rc) return rc;
  CTMI_REQUIRE(x && codes && scale_out, CTMI_ERR_VALUE, "NULL tensor pointer");
  CTMI_REQUIRE(ctmi_observe_quantize_supported(x_dtype, rows, cols, blk_cols, qtype, num_bits),
               CTMI_ERR_UNSUPPORTED,
               "no fused kernel for this layout: compute the scales and quantize separately");
  CTMI_REQUIRE((uintptr_t)x % (8 * dtype_size(x_dtype)) == 0 && (uintptr_t)codes % 8 == 0,
               CTMI_ERR_VALUE, "tensors must be aligned to 8 elements");
  hipStream_t st = (hipStream_t)stream;
  const DynOut o{scale_out, zp_out};
  const int qk = qtype == CTMI_QTYPE_INT ? 0 : 1;
#define CTMI_OQ_SYM(FT, QK)                                                                  \
  (symmetric ? launch_dynamic<FT, QK, true, true>(x, codes, o, rows, cols, blk_cols, c, st)  \
             : launch_dynamic<FT, QK, false, true>(x, codes, o, rows, cols, blk_cols, c, st))
#define CTMI_OQ_FT(FT) (qk == 0 ? CTMI_OQ_SYM(FT, 0) : CTMI_OQ_SYM(FT, 1))
  const bool ok = x_dtype == CTMI_BF16 ? CTMI_OQ_FT(BF16)
                                       : (x_dtype == CTMI_F16 ? CTMI_OQ_FT(F16) : CTMI_OQ_FT(F32));
#undef CTMI_OQ_SYM
#undef CTMI_OQ_FT
  CTMI_REQUIRE(ok, CTMI_ERR_UNSUPPORTED, "no fused kernel for this layout");
  return check_launch("ctmi_observe_quantize");
}

extern "C" int ctmi_observe_quantize_blocks_supported(int32_t x_dtype, int64_t rows, int64_t cols,
                                                      int64_t blk_rows, int64_t blk_cols,
                                                      int32_t qtype, int32_t num_bits) {
  if (x_dtype != CTMI_BF16 && x_dtype != CTMI_F16 && x_dtype != CTMI_F32) return 0;
  if (rows < 1 || cols < 1 || blk_rows < 1 || blk_cols < 1) return 0;
  if (!((qtype == CTMI_QTYPE_INT && num_bits <= 8) || (qtype == CTMI_QTYPE_FLOAT && num_bits == 8)))
    return 0;
  if (rows % blk_rows || cols % blk_cols || blk_cols % 8) return 0;
  if (cols / 8 >= (1ll << 31) || (rows / blk_rows) * (cols / blk_cols) >= (1ll << 31)) return 0;
  return blk_rows * blk_cols / 8 <= 2048;  // a block lives in the registers of one workgroup
}

extern "C" int ctmi_observe_quantize_blocks(const void* x, int32_t x_dtype, void* codes, int64_t rows,
                                            int64_t cols, int64_t blk_rows, int64_t blk_cols,
                                            int32_t qtype, int32_t num_bits, int32_t symmetric,
                                            void* scale_out, int32_t scale_dtype, void* zp_out,
                                            int32_t zp_dtype, void* stream) {
  CTMI_REQUIRE(rows >= 1 && cols >= 1, CTMI_ERR_VALUE, "cannot observe an empty tensor");
  CTMI_REQUIRE(blk_rows >= 1 && blk_cols >= 1, CTMI_ERR_VALUE, "empty cell");
  QpCfg c;
  // min / max of a block are not 0-d tensors: the zero-point arithmetic stays in x's dtype
  int rc = fill_qpcfg(&c, qtype, num_bits, symmetric, x_dtype, 0, false, scale_dtype, zp_dtype);
  if (rc) return rc;
  CTMI_REQUIRE(x && codes && scale_out, CTMI_ERR_VALUE, "NULL tensor pointer");
  CTMI_REQUIRE(ctmi_observe_quantize_blocks_supported(x_dtype, rows, cols, blk_rows, blk_cols, qtype,
                                                      num_bits),
               CTMI_ERR_UNSUPPORTED,
               "no fused kernel for this layout (blocks must tile the tensor, be a multiple of 8 "
               "wide and hold at most 16384 elements): compute the scales and quantize separately");
  CTMI_REQUIRE((uintptr_t)x % (8 * dtype_size(x_dtype)) == 0 && (uintptr_t)codes % 8 == 0,
               CTMI_ERR_VALUE, "tensors must be aligned to 8 elements");
  hipStream_t st = (hipStream_t)stream;
  const DynOut o{scale_out, zp_out};
  const int items = (int)(blk_rows * blk_cols / 8);
  const CellLayout g{(int)(blk_cols / 8), (int)(cols / 8), (int)(cols / blk_cols), (int)blk_rows};
  const unsigned grid = (unsigned)((rows / blk_rows) * (cols / blk_cols));
#define CTMI_OQB_U(FT, QK, SYM, UU)                                                               \
  hipLaunchKernelGGL((observe_quantize_blocks_kernel<FT, QK, SYM, UU>), grid, 256, 0, st,         \
                     (const typename FT::raw*)x, codes, o, items, g, c)
#define CTMI_OQB(FT, QK, SYM)                    \
  if (items <= 256) CTMI_OQB_U(FT, QK, SYM, 1);  \
  else if (items <= 512) CTMI_OQB_U(FT, QK, SYM, 2);  \
  else if (items <= 1024) CTMI_OQB_U(FT, QK, SYM, 4); \
  else CTMI_OQB_U(FT, QK, SYM, 8)
#define CTMI_OQB_SYM(FT, QK) \
  if (symmetric) { CTMI_OQB(FT, QK, true); } else { CTMI_OQB(FT, QK, false); }
#define CTMI_OQB_FT(FT) \
  if (qtype == CTMI_QTYPE_INT) { CTMI_OQB_SYM(FT, 0) } else { CTMI_OQB_SYM(FT, 1) }
  if (x_dtype == CTMI_BF16) { CTMI_OQB_FT(BF16) }
  else if (x_dtype == CTMI_F16) { CTMI_OQB_FT(F16) }
  else { CTMI_OQB_FT(F32) }
#undef CTMI_OQB_U
#undef CTMI_OQB
#undef CTMI_OQB_SYM
#undef CTMI_OQB_FT
  return check_launch("ctmi_observe_quantize_blocks");
}

// rows-per-workgroup class of a job (0: not a row-kernel layout)
static int rows_class(int64_t cols, int64_t blk_cols) {
  const int64_t seg = blk_cols < cols ? blk_cols : cols;
  if (seg % 8 || cols % seg) return 0;
  const int64_t items = seg / 8;
  if (items <= 64 && (items & (items - 1)) == 0) return 0;  // the flat kernel's layouts
  if (items <= 256) return 1;
  if (items <= 512) return 2;
  if (items <= 1024) return 4;
  if (items <= 2048) return 8;
  return 0;
}

template <typename FT, int QK, bool SYM>
static void launch_rows_many(const DynJobs& t, int filled, int u, const QpCfg& c, hipStream_t st) {
  const unsigned grid = (unsigned)t.end[filled - 1];
#define CTMI_DM(UU) \
  hipLaunchKernelGGL((dynamic_rows_many_kernel<FT, QK, SYM, UU, true>), grid, 256, 0, st, t, c)
  if (u == 1) CTMI_DM(1);
  else if (u == 2) CTMI_DM(2);
  else if (u == 4) CTMI_DM(4);
  else CTMI_DM(8);
#undef CTMI_DM
}

extern "C" int ctmi_observe_quantize_many(const ctmi_observe_quantize_job* jobs, int64_t n,
                                          int32_t qtype, int32_t num_bits, int32_t symmetric,
                                          int32_t scale_dtype, int32_t zp_dtype, void* stream) {
  CTMI_REQUIRE(n >= 0 && (jobs || n == 0), CTMI_ERR_VALUE, "bad job list");
  if (n == 0) return CTMI_OK;
  // validate everything before anything is enqueued
  for (int64_t i = 0; i < n; ++i) {
    const ctmi_observe_quantize_job& j = jobs[i];
    CTMI_REQUIRE(j.rows >= 1 && j.cols >= 1 && j.blk_cols >= 1, CTMI_ERR_VALUE,
                 "job %lld: cannot observe an empty tensor", (long long)i);
    QpCfg c;
    int rc = fill_qpcfg(&c, qtype, num_bits, symmetric, j.x_dtype, 0, false,
                        scale_dtype < 0 ? j.x_dtype : scale_dtype, zp_dtype);
    if (rc) return rc;
    CTMI_REQUIRE(j.x && j.codes && j.scale, CTMI_ERR_VALUE, "job %lld: NULL tensor pointer", (long long)i);
    CTMI_REQUIRE(ctmi_observe_quantize_supported(j.x_dtype, j.rows, j.cols, j.blk_cols, qtype, num_bits),
                 CTMI_ERR_UNSUPPORTED,
                 "job %lld: no fused kernel for this layout: compute the scales and quantize separately",
                 (long long)i);
    CTMI_REQUIRE((uintptr_t)j.x % (8 * dtype_size(j.x_dtype)) == 0 && (uintptr_t)j.codes % 8 == 0,
                 CTMI_ERR_VALUE, "tensors must be aligned to 8 elements");
  }
  hipStream_t st = (hipStream_t)stream;
  const int qk = qtype == CTMI_QTYPE_INT ? 0 : 1;
  // rows of one length class and dtype share launches, kDynMaxJobs tensors at a time
  const int dts[3] = {CTMI_BF16, CTMI_F16, CTMI_F32};
  const int classes[4] = {1, 2, 4, 8};
  for (int d = 0; d < 3; ++d) {
    QpCfg c;
    fill_qpcfg(&c, qtype, num_bits, symmetric, dts[d], 0, false,
               scale_dtype < 0 ? dts[d] : scale_dtype, zp_dtype);
    for (int k = 0; k < 4; ++k) {
      DynJobs t;
      int filled = 0;
      auto reset = [&]() {
        filled = 0;
        for (int q = 0; q < kDynMaxJobs; ++q) {
          t.x[q] = nullptr;
          t.out[q] = nullptr;
          t.o[q] = DynOut{nullptr, nullptr};
          t.end[q] = INT64_MAX;
          t.items[q] = 1;
        }
      };
      auto flush = [&]() {
        if (!filled) return;
#define CTMI_DM_SYM(FT, QK)                                                  \
  (symmetric ? launch_rows_many<FT, QK, true>(t, filled, classes[k], c, st)  \
             : launch_rows_many<FT, QK, false>(t, filled, classes[k], c, st))
#define CTMI_DM_FT(FT) (qk == 0 ? CTMI_DM_SYM(FT, 0) : CTMI_DM_SYM(FT, 1))
        if (dts[d] == CTMI_BF16) CTMI_DM_FT(BF16);
        else if (dts[d] == CTMI_F16) CTMI_DM_FT(F16);
        else CTMI_DM_FT(F32);
#undef CTMI_DM_SYM
#undef CTMI_DM_FT
        reset();
      };
      reset();
      for (int64_t i = 0; i < n; ++i) {
        const ctmi_observe_quantize_job& j = jobs[i];
        if (j.x_dtype != dts[d] || rows_class(j.cols, j.blk_cols) != classes[k]) continue;
        const int64_t seg = j.blk_cols < j.cols ? j.blk_cols : j.cols;
        const int64_t segments = j.rows * (j.cols / seg);
        const int64_t before = filled ? t.end[filled - 1] : 0;
        if (filled == kDynMaxJobs || before + segments >= (1ll << 31)) flush();
        if (segments >= (1ll << 31)) continue;  // taken by the single call below
        t.x[filled] = j.x;
        t.out[filled] = j.codes;
        t.o[filled] = DynOut{j.scale, j.zero_point};
        t.items[filled] = (int)(seg / 8);
        t.end[filled] = (filled ? t.end[filled - 1] : 0) + segments;
        ++filled;
      }
      flush();
    }
  }
  int rc = check_launch("ctmi_observe_quantize_many");
  if (rc) return rc;
  for (int64_t i = 0; i < n; ++i) {
    const ctmi_observe_quantize_job& j = jobs[i];
    const int64_t seg = j.blk_cols < j.cols ? j.blk_cols : j.cols;
    if (rows_class(j.cols, j.blk_cols) != 0 && j.rows * (j.cols / seg) < (1ll << 31)) continue;
    rc = ctmi_observe_quantize(j.x, j.x_dtype, j.codes, j.rows, j.cols, j.blk_cols, qtype, num_bits,
                               symmetric, j.scale, scale_dtype < 0 ? j.x_dtype : scale_dtype,
                               j.zero_point, zp_dtype, stream);
    if (rc) return rc;
  }
  return CTMI_OK;
}

// vectors-per-thread class of a block (items = vectors of 8 elements in a block)
static int block_class(int64_t items) { return items <= 256 ? 1 : items <= 512 ? 2 : items <= 1024 ? 4 : 8; }

template <typename FT, int QK, bool SYM>
static void launch_blocks_many(const DynBlockJobs& t, int filled, int u, const QpCfg& c, hipStream_t st) {
  const unsigned grid = (unsigned)t.end[filled - 1];
#define CTMI_BM(UU) \
  hipLaunchKernelGGL((observe_quantize_blocks_many_kernel<FT, QK, SYM, UU>), grid, 256, 0, st, t, c)
  if (u == 1) CTMI_BM(1);
  else if (u == 2) CTMI_BM(2);
  else if (u == 4) CTMI_BM(4);
  else CTMI_BM(8);
#undef CTMI_BM
}

extern "C" int ctmi_observe_quantize_blocks_many(const ctmi_observe_quantize_blocks_job* jobs, int64_t n,
                                                 int32_t qtype, int32_t num_bits, int32_t symmetric,
                                                 int32_t scale_dtype, int32_t zp_dtype, void* stream) {
  CTMI_REQUIRE(n >= 0 && (jobs || n == 0), CTMI_ERR_VALUE, "bad job list");
  if (n == 0) return CTMI_OK;
  for (int64_t i = 0; i < n; ++i) {  // everything is looked at before anything is enqueued
    const ctmi_observe_quantize_blocks_job& j = jobs[i];
    CTMI_REQUIRE(j.rows >= 1 && j.cols >= 1, CTMI_ERR_VALUE, "job %lld: cannot observe an empty tensor",
                 (long long)i);
    CTMI_REQUIRE(j.blk_rows >= 1 && j.blk_cols >= 1, CTMI_ERR_VALUE, "job %lld: empty cell", (long long)i);
    QpCfg c;
    int rc = fill_qpcfg(&c, qtype, num_bits, symmetric, j.x_dtype, 0, false,
                        scale_dtype < 0 ? j.x_dtype : scale_dtype, zp_dtype);
    if (rc) return rc;
    CTMI_REQUIRE(j.x && j.codes && j.scale, CTMI_ERR_VALUE, "job %lld: NULL tensor pointer", (long long)i);
    CTMI_REQUIRE(ctmi_observe_quantize_blocks_supported(j.x_dtype, j.rows, j.cols, j.blk_rows, j.blk_cols,
                                                        qtype, num_bits),
                 CTMI_ERR_UNSUPPORTED,
                 "job %lld: no fused kernel for this layout (blocks must tile the tensor, be a multiple "
                 "of 8 wide and hold at most 16384 elements)", (long long)i);
    CTMI_REQUIRE((uintptr_t)j.x % (8 * dtype_size(j.x_dtype)) == 0 && (uintptr_t)j.codes % 8 == 0,
                 CTMI_ERR_VALUE, "job %lld: tensors must be aligned to 8 elements", (long long)i);
  }
  hipStream_t st = (hipStream_t)stream;
  const int qk = qtype == CTMI_QTYPE_INT ? 0 : 1;
  // blocks of one size class and dtype share launches, kDynMaxJobs tensors at a time
  const int dts[3] = {CTMI_BF16, CTMI_F16, CTMI_F32};
  const int classes[4] = {1, 2, 4, 8};
  for (int d = 0; d < 3; ++d) {
    QpCfg c;
    fill_qpcfg(&c, qtype, num_bits, symmetric, dts[d], 0, false, scale_dtype < 0 ? dts[d] : scale_dtype,
               zp_dtype);
    for (int k = 0; k < 4; ++k) {
      DynBlockJobs t;
      int filled = 0;
      auto reset = [&]() {
        filled = 0;
        for (int q = 0; q < kDynMaxJobs; ++q) {
          t.x[q] = nullptr;
          t.out[q] = nullptr;
          t.o[q] = DynOut{nullptr, nullptr};
          t.end[q] = INT64_MAX;
          t.items[q] = 1;
          t.g[q] = CellLayout{1, 1, 1, 1};
        }
      };
      auto flush = [&]() {
        if (!filled) return;
#define CTMI_BM_SYM(FT, QK)                                                    \
  (symmetric ? launch_blocks_many<FT, QK, true>(t, filled, classes[k], c, st)  \
             : launch_blocks_many<FT, QK, false>(t, filled, classes[k], c, st))
#define CTMI_BM_FT(FT) (qk == 0 ? CTMI_BM_SYM(FT, 0) : CTMI_BM_SYM(FT, 1))
        if (dts[d] == CTMI_BF16) CTMI_BM_FT(BF16);
        else if (dts[d] == CTMI_F16) CTMI_BM_FT(F16);
        else CTMI_BM_FT(F32);
#undef CTMI_BM_SYM
#undef CTMI_BM_FT
        reset();
      };
      reset();
      for (int64_t i = 0; i < n; ++i) {
        const ctmi_observe_quantize_blocks_job& j = jobs[i];
        const int64_t items = j.blk_rows * j.blk_cols / 8;
        if (j.x_dtype != dts[d] || block_class(items) != classes[k]) continue;
        const int64_t blocks = (j.rows / j.blk_rows) * (j.cols / j.blk_cols);  // < 2^31 (checked above)
        const int64_t before = filled ? t.end[filled - 1] : 0;
        if (filled == kDynMaxJobs || before + blocks >= (1ll << 31)) flush();
        t.x[filled] = j.x;
        t.out[filled] = j.codes;
        t.o[filled] = DynOut{j.scale, j.zero_point};
        t.items[filled] = (int)items;
        t.g[filled] = CellLayout{(int)(j.blk_cols / 8), (int)(j.cols / 8), (int)(j.cols / j.blk_cols),
                                 (int)j.blk_rows};
        t.end[filled] = (filled ? t.end[filled - 1] : 0) + blocks;
        ++filled;
      }
      flush();
    }
  }
  return check_launch("ctmi_observe_quantize_blocks_many");
}
