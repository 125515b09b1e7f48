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
#include <cstring>
#include <type_traits>
#include <vector>

#include "ctmi_device.h"
#include "ctmi_host.h"
#include "job_table.h"
#include "minmax.h"
#include "qdq_core.h"
#include "qparams.h"
#include "quant_core.h"
#include "quant_fast.h"

namespace ctmi {

// ------------------------------------------------------------------ groups within a row
#ifndef CTMI_OP_TUNING
#define CTMI_OP_TUNING 512, 4
#endif
constexpr int kOpTuning[2] = {CTMI_OP_TUNING};
constexpr int kOpBlock = kOpTuning[0], kOpUnroll = kOpTuning[1];

// One item = 8 neighbouring elements; L = 2^job.shift neighbouring lanes own a
// group.  Items, words and groups are numbered row-major, so a chunk of
// kOpBlock * kOpUnroll items never splits a group.  job.scale / job.zp are outputs.
template <typename XT, int BITS, bool SYM>
__global__ void __launch_bounds__(kOpBlock) observe_pack_groups_kernel(const ChainTable t) {
  using XR = typename XT::raw;
  constexpr int W = BITS / 4;
  constexpr int B = kOpBlock, U = kOpUnroll;
  uint32_t chunk, nvec;
  const ChainJob job = find_job(t, blockIdx.x, &chunk, &nvec);
  const auto* __restrict__ x = (const XR*)job.src;
  int32_t* __restrict__ out = (int32_t*)job.dst;
  XR* __restrict__ scale = (XR*)const_cast<void*>(job.scale);
  int8_t* __restrict__ zp = const_cast<int8_t*>(job.zp);
  const int L = 1 << job.shift;
  const uint32_t v0 = chunk * (B * U) + threadIdx.x;
  const bool full = (chunk + 1) * (uint32_t)(B * U) <= nvec;
  auto body = [&](auto guard) {
    constexpr bool GUARD = decltype(guard)::value;
    Vec<XR, 8> a[U];
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const uint32_t v = v0 + k * B;
      // past the end: read the last item again, it changes no group it belongs to
      a[k] = ldg_nt<XR, 8>(x + (size_t)(GUARD && v >= nvec ? nvec - 1 : v) * 8);
    }
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const uint32_t v = v0 + k * B;
      float sv, zv = 0.0f;
      if constexpr (SYM && sizeof(XR) == 2) {
        const uint32_t m = group_umax(L, absmax8_bits<XT>(a[k]));
        constexpr uint32_t kInf = XT::id == CTMI_BF16 ? 0x7f80u : 0x7c00u;
        sv = symmetric_scale<XT>(XT::to_f32((XR)m), m > kInf, (t.qmax - t.qmin) * 0.5f);
      } else {
        float lo = __builtin_inff(), hi = -__builtin_inff();
        bool unordered = false;
        vec_minmax<XT>(a[k], &lo, &hi, &unordered);
        group_minmax(L, &lo, &hi);
        unordered = group_any(L, unordered);
        if constexpr (SYM) {
          const float m = __builtin_fmaxf(__builtin_fmaxf(-lo, hi), 0.0f);
          sv = symmetric_scale<XT>(m, unordered, (t.qmax - t.qmin) * 0.5f);
        } else {
          asymmetric_qparams<XT, 0>(lo, hi, unordered, t.qmin, t.qmax, &sv, &zv);
        }
      }
      if ((!GUARD || v < nvec) && (threadIdx.x & (L - 1)) == 0) {
        scale[v >> job.shift] = XT::from_f32(sv);
        if (zp) zp[v >> job.shift] = SYM ? (int8_t)0 : (int8_t)f32_to_int(zv);
      }
      // a symmetric scheme's zero point is 0: adding it changes no code
      const Vec<int32_t, W> w = quant_pack8<XT, XT, BITS, !SYM>(a[k], sv, zv, t.qmin, t.qmax);
      if (!GUARD || v < nvec) stg_nt<int32_t, W>(out + (size_t)v * W, w);
    }
  };
  if (full) body(std::false_type{});
  else body(std::true_type{});
}

// ------------------------------------------------------------------ one group per row
// One workgroup of 256 threads per row (channel strategy) of up to 256 * U items.
template <typename XT, int BITS, bool SYM, int U>
__global__ void __launch_bounds__(256)
observe_pack_rows_kernel(const typename XT::raw* __restrict__ x, int32_t* __restrict__ packed,
                         typename XT::raw* __restrict__ scale, int8_t* __restrict__ zp, int items,
                         float qmin, float qmax) {
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
  unordered = (part_nan[0] | part_nan[1] | part_nan[2] | part_nan[3]) != 0;
  float sv, zv = 0.0f;
  if constexpr (SYM) {
    sv = symmetric_scale<XT>(__builtin_fmaxf(__builtin_fmaxf(-lo, hi), 0.0f), unordered,
                             (qmax - qmin) * 0.5f);
  } else {
    asymmetric_qparams<XT, 0>(lo, hi, unordered, qmin, qmax, &sv, &zv);
  }
  if (threadIdx.x == 0) {
    scale[s] = XT::from_f32(sv);
    if (zp) zp[s] = SYM ? (int8_t)0 : (int8_t)f32_to_int(zv);
  }
  int32_t* q = packed + s * (int64_t)items * W;
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int i = k * 256 + threadIdx.x;
    const Vec<int32_t, W> w = quant_pack8<XT, XT, BITS, !SYM>(a[k], sv, zv, qmin, qmax);
    if (i < items) stg_nt<int32_t, W>(q + (int64_t)i * W, w);
  }
}

constexpr int kObservePackMaxItems = 256 * 8;

// ------------------------------------------------------------------ host side
struct OpKey {
  int x_dtype, bits, symmetric;
  bool operator==(const OpKey& o) const {
    return x_dtype == o.x_dtype && bits == o.bits && symmetric == o.symmetric;
  }
};

struct OpPlan {
  OpKey key;
  bool grouped;  // groups within a row (chained launches) or one group per row
  const void* x;
  int32_t* packed;
  void* scale;
  int8_t* zp;
  int64_t rows, items;  // items per group
  uint32_t nvec, shift;
};

template <typename XT, int BITS>
static void launch_groups_sym(const OpKey& k, const ChainTable& t, unsigned grid, hipStream_t st) {
  if (k.symmetric) hipLaunchKernelGGL((observe_pack_groups_kernel<XT, BITS, true>), grid, kOpBlock, 0, st, t);
  else hipLaunchKernelGGL((observe_pack_groups_kernel<XT, BITS, false>), grid, kOpBlock, 0, st, t);
}

template <typename XT>
static void launch_groups_bits(const OpKey& k, const ChainTable& t, unsigned grid, hipStream_t st) {
  if (k.bits == 4) launch_groups_sym<XT, 4>(k, t, grid, st);
  else launch_groups_sym<XT, 8>(k, t, grid, st);
}

static void launch_groups(const OpKey& k, const ChainTable& t, unsigned grid, hipStream_t st) {
  if (k.x_dtype == CTMI_BF16) launch_groups_bits<BF16>(k, t, grid, st);
  else if (k.x_dtype == CTMI_F16) launch_groups_bits<F16>(k, t, grid, st);
  else launch_groups_bits<F32>(k, t, grid, st);
}

template <typename XT, int BITS, bool SYM>
static void launch_rows_u(const OpPlan& p, float qmin, float qmax, hipStream_t st) {
  using XR = typename XT::raw;
#define CTMI_OP(UU)                                                                            \
  hipLaunchKernelGGL((observe_pack_rows_kernel<XT, BITS, SYM, UU>), (unsigned)p.rows, 256, 0, st, \
                     (const XR*)p.x, p.packed, (XR*)p.scale, p.zp, (int)p.items, qmin, qmax)
  if (p.items <= 256) CTMI_OP(1);
  else if (p.items <= 256 * 2) CTMI_OP(2);
  else if (p.items <= 256 * 4) CTMI_OP(4);
  else CTMI_OP(8);
#undef CTMI_OP
}

template <typename XT>
static void launch_rows_xt(const OpPlan& p, float qmin, float qmax, hipStream_t st) {
  if (p.key.bits == 4) {
    if (p.key.symmetric) launch_rows_u<XT, 4, true>(p, qmin, qmax, st);
    else launch_rows_u<XT, 4, false>(p, qmin, qmax, st);
  } else {
    if (p.key.symmetric) launch_rows_u<XT, 8, true>(p, qmin, qmax, st);
    else launch_rows_u<XT, 8, false>(p, qmin, qmax, st);
  }
}

static void launch_rows(const OpPlan& p, float qmin, float qmax, hipStream_t st) {
  if (p.key.x_dtype == CTMI_BF16) launch_rows_xt<BF16>(p, qmin, qmax, st);
  else if (p.key.x_dtype == CTMI_F16) launch_rows_xt<F16>(p, qmin, qmax, st);
  else launch_rows_xt<F32>(p, qmin, qmax, st);
}

static bool op_supported(int x_dtype, int64_t rows, int64_t cols, int64_t blk_cols, int num_bits) {
  if (x_dtype != CTMI_BF16 && x_dtype != CTMI_F16 && x_dtype != CTMI_F32) return false;
  if (num_bits != 4 && num_bits != 8) return false;
  if (rows < 1 || cols < 1 || blk_cols < 1) return false;
  const int64_t seg = blk_cols < cols ? blk_cols : cols;
  if (seg % 8 || cols % seg) return false;
  const int64_t items = seg / 8;
  if (rows * cols / 8 >= (1ll << 31)) return false;
  if (items <= 64 && (items & (items - 1)) == 0) return true;  // groups of neighbouring lanes
  return seg == cols && items <= kObservePackMaxItems;         // one workgroup per row
}

static int plan_observe_pack(const ctmi_observe_pack_job& j, OpPlan* p) {
  CTMI_REQUIRE(j.rows >= 1 && j.cols >= 1, CTMI_ERR_VALUE, "cannot observe an empty tensor");
  CTMI_REQUIRE(j.blk_cols >= 1, CTMI_ERR_VALUE, "empty cell");
  float qmin, qmax;
  int rc = quant_range(CTMI_QTYPE_INT, j.num_bits, &qmin, &qmax);
  if (rc) return rc;
  CTMI_REQUIRE(j.x_dtype == CTMI_F32 || j.x_dtype == CTMI_F16 || j.x_dtype == CTMI_BF16,
               CTMI_ERR_UNSUPPORTED, "weights must be float16/bfloat16/float32");
  CTMI_REQUIRE(j.x && j.packed && j.scale, CTMI_ERR_VALUE, "NULL tensor pointer");
  CTMI_REQUIRE(op_supported(j.x_dtype, j.rows, j.cols, j.blk_cols, j.num_bits), CTMI_ERR_UNSUPPORTED,
               "no fused kernel for this layout: run the observer and the compressor separately");
  CTMI_REQUIRE((uintptr_t)j.x % (8 * dtype_size(j.x_dtype)) == 0 &&
                   (uintptr_t)j.packed % (4 * (j.num_bits / 4)) == 0 &&
                   (uintptr_t)j.scale % dtype_size(j.x_dtype) == 0,
               CTMI_ERR_VALUE, "tensors must be aligned to 8 elements");
  const int64_t seg = j.blk_cols < j.cols ? j.blk_cols : j.cols;
  p->key = OpKey{j.x_dtype, j.num_bits, j.symmetric ? 1 : 0};
  p->x = j.x;
  p->packed = j.packed;
  p->scale = j.scale;
  p->zp = j.zero_point;
  p->rows = j.rows;
  p->items = seg / 8;
  p->nvec = (uint32_t)(j.rows * j.cols / 8);
  p->grouped = p->items <= 64 && (p->items & (p->items - 1)) == 0;
  p->shift = 0;
  while ((1ll << p->shift) < p->items) ++p->shift;
  return CTMI_OK;
}

static int run_observe_pack(const OpPlan* plans, int64_t n, hipStream_t st, const char* what) {
  std::vector<char> done((size_t)n, 0);
  const int per_block = kOpBlock * kOpUnroll;
  for (int64_t i = 0; i < n; ++i) {
    if (done[i]) continue;
    const OpKey key = plans[i].key;
    float qmin, qmax;
    quant_range(CTMI_QTYPE_INT, key.bits, &qmin, &qmax);
    if (!plans[i].grouped) {
      launch_rows(plans[i], qmin, qmax, st);
      done[i] = 1;
      continue;
    }
    ChainTable t;
    std::memset(&t, 0, sizeof(t));
    t.qmin = qmin;
    t.qmax = qmax;
    uint64_t chunks = 0;
    auto reset = [&]() {
      t.n = 0;
      chunks = 0;
      for (int k = 0; k < kMaxJobs; ++k) t.chunk_end[k] = 0xFFFFFFFFu;
    };
    reset();
    auto flush = [&]() {
      if (t.n == 0) return;
      launch_groups(key, t, (unsigned)chunks, st);
      reset();
    };
    for (int64_t j = i; j < n; ++j) {
      if (done[j] || !plans[j].grouped || !(plans[j].key == key)) continue;
      const uint64_t c = (uint64_t)cdiv(plans[j].nvec, per_block);
      if (t.n == kMaxJobs || chunks + c >= (1ull << 31)) flush();
      ChainJob cj;
      std::memset(&cj, 0, sizeof(cj));
      cj.src = plans[j].x;
      cj.dst = plans[j].packed;
      cj.scale = plans[j].scale;
      cj.zp = plans[j].zp;
      cj.shift = plans[j].shift;
      t.job[t.n] = cj;
      t.nvec[t.n] = plans[j].nvec;
      chunks += c;
      t.chunk_end[t.n] = (uint32_t)chunks;
      ++t.n;
      done[j] = 1;
    }
    flush();
  }
  return check_launch(what);
}

}  // namespace ctmi

using namespace ctmi;

extern "C" int ctmi_observe_pack_quantized_supported(int32_t x_dtype, int64_t rows, int64_t cols,
                                                     int64_t blk_cols, int32_t num_bits) {
  return op_supported(x_dtype, rows, cols, blk_cols, num_bits) ? 1 : 0;
}

extern "C" int ctmi_observe_pack_quantized_many(const ctmi_observe_pack_job* jobs, int64_t n,
                                                void* stream) {
  CTMI_REQUIRE(n >= 0 && (jobs || n == 0), CTMI_ERR_VALUE, "bad job list");
  std::vector<OpPlan> plans((size_t)n);
  for (int64_t i = 0; i < n; ++i) {  // every job is validated before anything is enqueued
    int rc = plan_observe_pack(jobs[i], &plans[i]);
    if (rc) return rc;
  }
  return run_observe_pack(plans.data(), n, (hipStream_t)stream, "ctmi_observe_pack_quantized_many");
}

extern "C" int ctmi_observe_pack_quantized(const void* x, int32_t x_dtype, int64_t rows,
                                           int64_t cols, int64_t blk_cols, int32_t num_bits,
                                           int32_t symmetric, int32_t* packed, void* scale,
                                           int8_t* zero_point, void* stream) {
  const ctmi_observe_pack_job j{x, packed, scale, zero_point, rows, cols, blk_cols, x_dtype,
                                num_bits, symmetric};
  OpPlan p;
  int rc = plan_observe_pack(j, &p);
  if (rc) return rc;
  return run_observe_pack(&p, 1, (hipStream_t)stream, "ctmi_observe_pack_quantized");
}
