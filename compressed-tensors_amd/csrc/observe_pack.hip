// Observer, calculate_qparams, quantize and pack_to_int32 in one pass over a weight:
// what a one-shot (round-to-nearest) compression of a pack-quantized model runs per
// weight, with the tensor read once.
//
//   min / max per group or channel          tests/mock_observer.py:38-113
//   calculate_qparams                       quantization/utils/helpers.py:67-146
//   quantize                                quantization/lifecycle/forward.py:45-81, 455-487
//   pack_to_int32                           compressors/quantized_compressors/pack_quantized.py:186-246
//
// Traffic per element of a bf16 weight: 2 bytes in, num_bits / 8 out (+ scales),
// against 2 in for the observer and 2 in again for the compressor.
#include <type_traits>

#include "ctmi_device.h"
#include "ctmi_host.h"
#include "minmax.h"
#include "qparams.h"
#include "quant_core.h"
#include "quant_fast.h"

namespace ctmi {

int fill_qpcfg(QpCfg* c, int qtype, int num_bits, int symmetric, int mt, int mm_is_0d,
               bool has_gscale, int scale_dtype, int zp_dtype);

struct ObservePackOut {
  int32_t* packed;
  void* scale;
  int8_t* zp;  // optional, unpacked
};

template <typename XT, int BITS>
__device__ __forceinline__ Vec<int32_t, BITS / 4> observe_pack_codes(
    const Vec<typename XT::raw, 8>& a, float sv, float zv, const QpCfg& c) {
  // a symmetric scheme's zero point is 0: adding it changes no code
  if (c.symmetric) return quant_pack8<XT, XT, BITS, false>(a, sv, 0.0f, c.bit_min, c.bit_max);
  return quant_pack8<XT, XT, BITS, true>(a, sv, zv, c.bit_min, c.bit_max);
}

// Groups of L vectors of 8 elements, L a power of two <= 64: L neighbouring lanes
// own a group; vectors, words and groups are all numbered row-major.
template <typename XT, int BITS, int U>
__global__ void __launch_bounds__(256)
observe_pack_flat_kernel(const typename XT::raw* __restrict__ x, ObservePackOut o, int64_t nvec,
                         int L, QpCfg c) {
  using XR = typename XT::raw;
  constexpr int W = BITS / 4;
  const int64_t v0 = (int64_t)blockIdx.x * (256 * U) + threadIdx.x;
  Vec<XR, 8> a[U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t v = v0 + k * 256;
    a[k] = ldg_nt<XR, 8>(x + (v < nvec ? v : nvec - 1) * 8);
  }
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t v = v0 + k * 256;
    float lo = __builtin_inff(), hi = -__builtin_inff();
    bool unordered = false;
    vec_minmax<XT>(a[k], &lo, &hi, &unordered);
    group_minmax(L, &lo, &hi);
    if (group_any(L, unordered)) lo = hi = __builtin_nanf("");
    float sv, zv;
    qparams_value<XT::id>(lo, hi, 1.0f, c, &sv, &zv);
    zv = stored_zero_point(zv, c);
    if (v < nvec && (threadIdx.x & (L - 1)) == 0) {
      ((XR*)o.scale)[v / L] = XT::from_f32(sv);
      if (o.zp) o.zp[v / L] = (int8_t)f32_to_int(zv);
    }
    const Vec<int32_t, W> w = observe_pack_codes<XT, BITS>(a[k], sv, zv, c);
    if (v < nvec) stg_nt<int32_t, W>(o.packed + v * W, w);
  }
}

// One workgroup of 256 threads per row-long group (channel strategy) of up to
// 256 * U vectors.
template <typename XT, int BITS, int U>
__global__ void __launch_bounds__(256)
observe_pack_rows_kernel(const typename XT::raw* __restrict__ x, ObservePackOut o, int items,
                         QpCfg c) {
  using XR = typename XT::raw;
  constexpr int W = BITS / 4;
  __shared__ float part_lo[4], part_hi[4];
  __shared__ int part_nan[4];
  const int64_t s = blockIdx.x;
  const XR* p = x + s * (int64_t)items * 8;
  Vec<XR, 8> a[U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int i = k * 256 + threadIdx.x;
    a[k] = ldg_nt<XR, 8>(p + (int64_t)(i < items ? i : items - 1) * 8);
  }
  float lo = __builtin_inff(), hi = -__builtin_inff();
  bool unordered = false;
#pragma unroll
  for (int k = 0; k < U; ++k) vec_minmax<XT>(a[k], &lo, &hi, &unordered);
  group_minmax(64, &lo, &hi);
  unordered = group_any(64, unordered);
  if ((threadIdx.x & 63) == 0) {
    part_lo[threadIdx.x >> 6] = lo;
    part_hi[threadIdx.x >> 6] = hi;
    part_nan[threadIdx.x >> 6] = unordered;
  }
  __syncthreads();
  lo = __builtin_fminf(__builtin_fminf(part_lo[0], part_lo[1]), __builtin_fminf(part_lo[2], part_lo[3]));
  hi = __builtin_fmaxf(__builtin_fmaxf(part_hi[0], part_hi[1]), __builtin_fmaxf(part_hi[2], part_hi[3]));
  if (part_nan[0] | part_nan[1] | part_nan[2] | part_nan[3]) lo = hi = __builtin_nanf("");
  float sv, zv;
  qparams_value<XT::id>(lo, hi, 1.0f, c, &sv, &zv);
  zv = stored_zero_point(zv, c);
  if (threadIdx.x == 0) {
    ((XR*)o.scale)[s] = XT::from_f32(sv);
    if (o.zp) o.zp[s] = (int8_t)f32_to_int(zv);
  }
  int32_t* q = o.packed + s * (int64_t)items * W;
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int i = k * 256 + threadIdx.x;
    const Vec<int32_t, W> w = observe_pack_codes<XT, BITS>(a[k], sv, zv, c);
    if (i < items) stg_nt<int32_t, W>(q + (int64_t)i * W, w);
  }
}

constexpr int kObservePackMaxItems = 256 * 8;

template <typename XT, int BITS>
static bool launch_observe_pack(const void* x, const ObservePackOut& o, int64_t rows, int64_t cols,
                                int64_t seg, const QpCfg& c, hipStream_t st) {
  using XR = typename XT::raw;
  const int64_t items = seg / 8, nvec = rows * cols / 8, n_segments = rows * (cols / seg);
  if (items <= 64 && (items & (items - 1)) == 0) {
    constexpr int U = 2;
    const int64_t blocks = cdiv(nvec, 256 * U);
    if (blocks >= (1ll << 31)) return false;
    hipLaunchKernelGGL((observe_pack_flat_kernel<XT, BITS, U>), (unsigned)blocks, 256, 0, st,
                       (const XR*)x, o, nvec, (int)items, c);
    return true;
  }
  if (n_segments >= (1ll << 31) || items > kObservePackMaxItems) return false;
#define CTMI_OP(UU)                                                                          \
  hipLaunchKernelGGL((observe_pack_rows_kernel<XT, BITS, UU>), (unsigned)n_segments, 256, 0, st, \
                     (const XR*)x, o, (int)items, c)
  if (items <= 256) CTMI_OP(1);
  else if (items <= 256 * 2) CTMI_OP(2);
  else if (items <= 256 * 4) CTMI_OP(4);
  else CTMI_OP(8);
#undef CTMI_OP
  return true;
}

}  // namespace ctmi

using namespace ctmi;

extern "C" int ctmi_observe_pack_quantized_supported(int32_t x_dtype, int64_t rows, int64_t cols,
                                                     int64_t blk_cols, int32_t num_bits) {
  if (x_dtype != CTMI_BF16 && x_dtype != CTMI_F16 && x_dtype != CTMI_F32) return 0;
  if (num_bits != 4 && num_bits != 8) return 0;
  if (rows < 1 || cols < 1 || blk_cols < 1) return 0;
  const int64_t seg = blk_cols < cols ? blk_cols : cols;
  if (seg % 8 || cols % seg) return 0;
  return seg / 8 <= kObservePackMaxItems;
}

extern "C" int ctmi_observe_pack_quantized(const void* x, int32_t x_dtype, int64_t rows,
                                           int64_t cols, int64_t blk_cols, int32_t num_bits,
                                           int32_t symmetric, int32_t* packed, void* scale,
                                           int8_t* zero_point, void* stream) {
  CTMI_REQUIRE(rows >= 1 && cols >= 1, CTMI_ERR_VALUE, "cannot observe an empty tensor");
  CTMI_REQUIRE(blk_cols >= 1, CTMI_ERR_VALUE, "empty cell");
  QpCfg c;
  int rc = fill_qpcfg(&c, CTMI_QTYPE_INT, num_bits, symmetric, x_dtype, 0, false, x_dtype, CTMI_I8);
  if (rc) return rc;
  CTMI_REQUIRE(x && packed && scale, CTMI_ERR_VALUE, "NULL tensor pointer");
  CTMI_REQUIRE(ctmi_observe_pack_quantized_supported(x_dtype, rows, cols, blk_cols, num_bits),
               CTMI_ERR_UNSUPPORTED,
               "no fused kernel for this layout: run the observer and the compressor separately");
  CTMI_REQUIRE((uintptr_t)x % (8 * dtype_size(x_dtype)) == 0 && (uintptr_t)packed % (4 * (num_bits / 4)) == 0,
               CTMI_ERR_VALUE, "tensors must be aligned to 8 elements");
  const int64_t seg = blk_cols < cols ? blk_cols : cols;
  const ObservePackOut o{packed, scale, zero_point};
  hipStream_t st = (hipStream_t)stream;
  bool ok;
#define CTMI_OP_XT(XT)                                                          \
  (num_bits == 4 ? launch_observe_pack<XT, 4>(x, o, rows, cols, seg, c, st)     \
                 : launch_observe_pack<XT, 8>(x, o, rows, cols, seg, c, st))
  ok = x_dtype == CTMI_BF16 ? CTMI_OP_XT(BF16)
                            : (x_dtype == CTMI_F16 ? CTMI_OP_XT(F16) : CTMI_OP_XT(F32));
#undef CTMI_OP_XT
  CTMI_REQUIRE(ok, CTMI_ERR_UNSUPPORTED, "no fused kernel for this layout");
  return check_launch("ctmi_observe_pack_quantized");
}
