// Scale / zero-point derivation: min-max reduction and calculate_qparams.
//
//   calculate_qparams              quantization/utils/helpers.py:67-146
//   compute_dynamic_scales_and_zp  helpers.py:149-205
//   generate_gparam                helpers.py:414-434
//   min-max observer               tests/mock_observer.py:38-56 (amin / amax per slice)
//
// calculate_qparams is evaluated in the dtype of the min/max tensors (each op
// rounded to it), except where the reference's operands promote to fp32.
#include <cstring>
#include <vector>

#include "ctmi_device.h"
#include "ctmi_host.h"
#include "job_table.h"
#include "qparams.h"
#include "minmax.h"

namespace ctmi {

// fp4.hip: group-16 fp8 scales of a 16-bit tensor; false = not its case, nothing launched
bool nvfp4_observe_try(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t blk_cols,
                       const float* gscale, void* scale_out, void* zp_out, const QpCfg& c,
                       hipStream_t st);


__global__ void __launch_bounds__(256)
qparams_kernel(const void* __restrict__ mn, const void* __restrict__ mx, const float* gscale,
               void* __restrict__ scale, void* __restrict__ zp, int64_t n, QpCfg c) {
  const float gs = gscale ? gscale[0] : 1.0f;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    float s, z;
    qparams_value(load_f32(mn, c.mt, i), load_f32(mx, c.mt, i), gs, c, &s, &z);
    store_from_f32(scale, c.scale_dtype, i, s);
    if (zp) store_from_f32(zp, c.zp_dtype, i, z);
  }
}

__global__ void __launch_bounds__(256)
gparam_kernel(const void* __restrict__ mn, const void* __restrict__ mx, int mt,
              float* __restrict__ out, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const float a = nan_min(load_f32(mn, mt, i), 0.0f);
    const float b = nan_max(load_f32(mx, mt, i), 0.0f);
    const float m = nan_max(fabsf(a), fabsf(b));
    // `448 * 6 / max_val_pos` with a Python float on the left runs as
    // max_val_pos.reciprocal() * 2688 (Tensor.__rtruediv__): two roundings in the
    // min / max dtype, then the cast to fp32
    out[i] = round_to(round_to(1.0f / m, mt) * 2688.0f, mt);
  }
}

// ------------------------------------------------------------------ min/max reduction
// Cell = blk_rows x blk_cols patch of a [rows, cols] tensor.  Stage 1 reduces
// every (row, cell column) segment; L lanes cooperate on one segment with
// 16-byte loads and finish with xor-shuffles.  Stage 2 (only when
// blk_rows > 1) folds the rows of a cell.
template <typename XT>
__device__ __forceinline__ void segment_minmax(const typename XT::raw* __restrict__ p, int64_t n,
                                               int lane_in_seg, int L, bool vec, float* mn,
                                               float* mx) {
  float lo = __builtin_inff(), hi = -__builtin_inff();
  if (vec) {
    for (int64_t v = lane_in_seg; v < n / 8; v += L) {
      Vec<typename XT::raw, 8> a = ldg<typename XT::raw, 8>(p + v * 8);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float f = XT::to_f32(a.v[j]);
        lo = nan_min(f, lo);
        hi = nan_max(f, hi);
      }
    }
  } else {
    for (int64_t i = lane_in_seg; i < n; i += L) {
      const float f = XT::to_f32(p[i]);
      lo = nan_min(f, lo);
      hi = nan_max(f, hi);
    }
  }
  for (int d = L / 2; d > 0; d >>= 1) {
    lo = nan_min(__shfl_xor(lo, d, kWave), lo);
    hi = nan_max(__shfl_xor(hi, d, kWave), hi);
  }
  *mn = lo;
  *mx = hi;
}

struct SegGeom {
  int64_t rows, cols, seg_cols /* blk_cols */, n_seg /* segments per row */;
  int L;        // lanes per segment (power of two <= 64)
  int vec;      // 16-byte loads allowed
};

template <typename XT>
__global__ void __launch_bounds__(256)
minmax_rows_kernel(const typename XT::raw* __restrict__ x, typename XT::raw* __restrict__ mn,
                   typename XT::raw* __restrict__ mx, SegGeom g) {
  const int segs_per_block = 256 / g.L;
  const int seg_in_block = threadIdx.x / g.L;
  const int lane_in_seg = threadIdx.x % g.L;
  const int64_t total = g.rows * g.n_seg;
  // uniform trip count per workgroup so the shuffles always see full segments
  for (int64_t base = (int64_t)blockIdx.x * segs_per_block; base < total;
       base += (int64_t)gridDim.x * segs_per_block) {
    const int64_t s = base + seg_in_block;
    float lo = 0.0f, hi = 0.0f;
    const bool live = s < total;
    const int64_t r = live ? s / g.n_seg : 0;
    const int64_t j = live ? s - r * g.n_seg : 0;
    int64_t n = g.cols - j * g.seg_cols;
    if (n > g.seg_cols) n = g.seg_cols;
    if (!live) n = 0;
    segment_minmax<XT>(x + r * g.cols + j * g.seg_cols, n, lane_in_seg, g.L, g.vec != 0, &lo, &hi);
    if (live && lane_in_seg == 0) {
      mn[s] = XT::from_f32(lo);
      mx[s] = XT::from_f32(hi);
    }
  }
}

// fused: stage 1 + calculate_qparams, for cells that are one row tall
template <typename XT>
__global__ void __launch_bounds__(256)
observe_rows_kernel(const typename XT::raw* __restrict__ x, const float* gscale,
                    void* __restrict__ scale, void* __restrict__ zp,
                    typename XT::raw* __restrict__ mn_out, typename XT::raw* __restrict__ mx_out,
                    SegGeom g, QpCfg c) {
  const float gs = gscale ? gscale[0] : 1.0f;
  const int segs_per_block = 256 / g.L;
  const int seg_in_block = threadIdx.x / g.L;
  const int lane_in_seg = threadIdx.x % g.L;
  const int64_t total = g.rows * g.n_seg;
  for (int64_t base = (int64_t)blockIdx.x * segs_per_block; base < total;
       base += (int64_t)gridDim.x * segs_per_block) {
    const int64_t s = base + seg_in_block;
    float lo = 0.0f, hi = 0.0f;
    const bool live = s < total;
    const int64_t r = live ? s / g.n_seg : 0;
    const int64_t j = live ? s - r * g.n_seg : 0;
    int64_t n = g.cols - j * g.seg_cols;
    if (n > g.seg_cols) n = g.seg_cols;
    if (!live) n = 0;
    segment_minmax<XT>(x + r * g.cols + j * g.seg_cols, n, lane_in_seg, g.L, g.vec != 0, &lo, &hi);
    if (live && lane_in_seg == 0) {
      float sv, zv;
      qparams_value(lo, hi, gs, c, &sv, &zv);
      store_from_f32(scale, c.scale_dtype, s, sv);
      if (zp) store_from_f32(zp, c.zp_dtype, s, zv);
      if (mn_out) mn_out[s] = XT::from_f32(lo);
      if (mx_out) mx_out[s] = XT::from_f32(hi);
    }
  }
}

// ---- streaming forms of stage 1 (+ calculate_qparams) for 16-byte-aligned tensors whose
// segments are whole numbers of 8-element vectors and tile the rows exactly.
// Memory is then one run of vectors, numbered like the segments.  Both kernels
// issue every load of a workgroup's share before looking at any value, one
// workgroup per share (no grid-stride loop).
struct ObserveOut {
  void* scale;   // NULL: min/max only
  void* zp;
  void* mn;
  void* mx;
};

template <typename XT>
__device__ __forceinline__ void emit_segment(const ObserveOut& o, int64_t s, float lo, float hi,
                                             float gs, const QpCfg& c) {
  if (o.scale) {
    float sv, zv;
    qparams_value(lo, hi, gs, c, &sv, &zv);
    store_from_f32(o.scale, c.scale_dtype, s, sv);
    if (o.zp) store_from_f32(o.zp, c.zp_dtype, s, zv);
  }
  if (o.mn) ((typename XT::raw*)o.mn)[s] = XT::from_f32(lo);
  if (o.mx) ((typename XT::raw*)o.mx)[s] = XT::from_f32(hi);
}

constexpr int kObsUnroll = 4;

// L vectors per segment, L a power of two <= 64: L neighbouring lanes own a segment
template <typename XT>
__global__ void __launch_bounds__(256)
observe_flat_kernel(const typename XT::raw* __restrict__ x, const float* gscale, ObserveOut o,
                    int64_t nvec, int L, QpCfg c) {
  constexpr int U = kObsUnroll;
  const float gs = gscale ? gscale[0] : 1.0f;
  const int64_t v0 = (int64_t)blockIdx.x * (256 * U) + threadIdx.x;
  Vec<typename XT::raw, 8> a[U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    // past the end: re-read the last vector (nothing is emitted for it)
    const int64_t v = v0 + k * 256;
    a[k] = ldg_nt<typename XT::raw, 8>(x + (v < nvec ? v : nvec - 1) * 8);  // read once
  }
  // The segments' results go through LDS so that the scale arithmetic and the
  // stores run on full wavefronts, one segment per lane, instead of on one lane
  // in L.  A workgroup covers 256 * U vectors = 256 * U / L whole segments.
  __shared__ float seg_lo[256 * U], seg_hi[256 * U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    float lo = __builtin_inff(), hi = -__builtin_inff();
    bool unordered = false;
    vec_minmax<XT>(a[k], &lo, &hi, &unordered);
    group_minmax(L, &lo, &hi);
    if (group_any(L, unordered)) lo = hi = __builtin_nanf("");
    if ((threadIdx.x & (L - 1)) == 0) {
      const int slot = (k * 256 + threadIdx.x) / L;
      seg_lo[slot] = lo;
      seg_hi[slot] = hi;
    }
  }
  __syncthreads();
  const int per_wg = 256 * U / L;
  const int64_t first = (int64_t)blockIdx.x * per_wg, n_seg = nvec / L;
  for (int i = threadIdx.x; i < per_wg && first + i < n_seg; i += 256)
    emit_segment<XT>(o, first + i, seg_lo[i], seg_hi[i], gs, c);
}

// more than 64 vectors per segment: one wavefront per segment
template <typename XT>
__global__ void __launch_bounds__(256)
observe_wide_kernel(const typename XT::raw* __restrict__ x, const float* gscale, ObserveOut o,
                    int64_t n_segments, int64_t items, QpCfg c) {
  constexpr int U = 8;
  const float gs = gscale ? gscale[0] : 1.0f;
  const int lane = threadIdx.x & 63;
  const int64_t s = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (s >= n_segments) return;
  const typename XT::raw* p = x + s * items * 8;
  float lo = __builtin_inff(), hi = -__builtin_inff();
  bool unordered = false;
  for (int64_t t = 0; t < items; t += 64 * U) {
    Vec<typename XT::raw, 8> a[U];
#pragma unroll
    for (int k = 0; k < U; ++k) {
      // min / max do not mind seeing an element twice: no bounds branches; streaming
      // loads (the tensor is read once): 5.0 TB/s against 4.3 with plain ones
      const int64_t i = t + k * 64 + lane;
      a[k] = ldg_nt<typename XT::raw, 8>(p + (i < items ? i : items - 1) * 8);
    }
#pragma unroll
    for (int k = 0; k < U; ++k) vec_minmax<XT>(a[k], &lo, &hi, &unordered);
  }
  group_minmax(64, &lo, &hi);
  if (group_any(64, unordered)) lo = hi = __builtin_nanf("");
  if (lane == 0) emit_segment<XT>(o, s, lo, hi, gs, c);
}

// launches a streaming form if the geometry allows; false = nothing launched
template <typename XT>
static bool observe_streaming(const void* x, const float* gscale, const ObserveOut& o,
                              const SegGeom& g, const QpCfg& c, hipStream_t st) {
  if (!g.vec || g.cols % g.seg_cols != 0) return false;
  const int64_t items = g.seg_cols / 8;
  const int64_t nvec = g.rows * g.cols / 8;
  const int64_t n_segments = g.rows * g.n_seg;
  using R = typename XT::raw;
  if (items <= 64 && (items & (items - 1)) == 0) {
    const int64_t blocks = cdiv(nvec, 256 * kObsUnroll);
    if (blocks >= (1ll << 31)) return false;
    hipLaunchKernelGGL(observe_flat_kernel<XT>, (unsigned)blocks, 256, 0, st, (const R*)x, gscale, o,
                       nvec, (int)items, c);
    return true;
  }
  if (items > 64) {
    const int64_t blocks = cdiv(n_segments, 4);
    if (blocks >= (1ll << 31)) return false;
    hipLaunchKernelGGL(observe_wide_kernel<XT>, (unsigned)blocks, 256, 0, st, (const R*)x, gscale, o,
                       n_segments, items, c);
    return true;
  }
  return false;
}

// ---- the streaming forms for several tensors per launch (scales and zero points only)
struct ObsChainJob {
  const void* x;
  void* scale;
  void* zp;
  const float* gscale;
};
struct ObsChainTable {  // the kernel's only argument: find_job_index reads its head
  uint32_t chunk_end[kMaxJobs];  // running total of workgroups, job 0 .. j (unused: 0xFFFFFFFF)
  uint32_t n_items[kMaxJobs];    // flat: vectors of the tensor; wide: its segments
  ObsChainJob job[kMaxJobs];
  uint32_t per[kMaxJobs];        // wide: vectors per segment
  int L;                         // flat: vectors per segment (one value per launch)
  QpCfg c;
};
static_assert(offsetof(ObsChainTable, chunk_end) == 0 && offsetof(ObsChainTable, n_items) == 32,
              "find_job_index");

// SYM (16-bit tensors, symmetric scheme): only max |x| matters, taken on the packed magnitude
// bits (two elements per instruction; the min / max form keeps the vector ALUs 95 % busy).
template <typename XT, bool SYM>
__global__ void __launch_bounds__(256) observe_flat_chain_kernel(const ObsChainTable t) {
  constexpr int U = kObsUnroll;
  uint32_t local, nvec;
  const ObsChainJob job = t.job[find_job_index(blockIdx.x, &local, &nvec)];
  const typename XT::raw* __restrict__ x = static_cast<const typename XT::raw*>(job.x);
  const int L = t.L;
  const float gs = job.gscale ? job.gscale[0] : 1.0f;
  const uint32_t v0 = local * (256 * U) + threadIdx.x;
  Vec<typename XT::raw, 8> a[U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const uint32_t v = v0 + k * 256;  // past the end: re-read the last vector (nothing is emitted for it)
    a[k] = ldg_nt<typename XT::raw, 8>(x + (int64_t)(v < nvec ? v : nvec - 1) * 8);
  }
  __shared__ float seg_lo[256 * U], seg_hi[256 * U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    float lo = __builtin_inff(), hi = -__builtin_inff();
    if constexpr (SYM) {
      const uint32_t m = group_umax(L, absmax8_bits<XT>(a[k]));
      constexpr uint32_t kInf = XT::id == CTMI_BF16 ? 0x7f80u : 0x7c00u;
      hi = m > kInf ? __builtin_nanf("") : XT::to_f32((typename XT::raw)m);
      lo = -hi;
    } else {
      bool unordered = false;
      vec_minmax<XT>(a[k], &lo, &hi, &unordered);
      group_minmax(L, &lo, &hi);
      if (group_any(L, unordered)) lo = hi = __builtin_nanf("");
    }
    if ((threadIdx.x & (L - 1)) == 0) {
      const int slot = (k * 256 + threadIdx.x) / L;
      seg_lo[slot] = lo;
      seg_hi[slot] = hi;
    }
  }
  __syncthreads();
  const ObserveOut o{job.scale, job.zp, nullptr, nullptr};
  const int per_wg = 256 * U / L;
  const int64_t first = (int64_t)local * per_wg, n_seg = nvec / L;
  for (int i = threadIdx.x; i < per_wg && first + i < n_seg; i += 256)
    emit_segment<XT>(o, first + i, seg_lo[i], seg_hi[i], gs, t.c);
}

template <typename XT>
__global__ void __launch_bounds__(256) observe_wide_chain_kernel(const ObsChainTable t) {
  constexpr int U = 8;
  uint32_t local, n_segments;
  const uint32_t ji = find_job_index(blockIdx.x, &local, &n_segments);
  const ObsChainJob job = t.job[ji];
  const int64_t items = t.per[ji];
  const float gs = job.gscale ? job.gscale[0] : 1.0f;
  const int lane = threadIdx.x & 63;
  const int64_t s = (int64_t)local * 4 + (threadIdx.x >> 6);
  if (s >= n_segments) return;
  const typename XT::raw* p = static_cast<const typename XT::raw*>(job.x) + s * items * 8;
  float lo = __builtin_inff(), hi = -__builtin_inff();
  bool unordered = false;
  for (int64_t i0 = 0; i0 < items; i0 += 64 * U) {
    Vec<typename XT::raw, 8> a[U];
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const int64_t i = i0 + k * 64 + lane;
      a[k] = ldg_nt<typename XT::raw, 8>(p + (i < items ? i : items - 1) * 8);
    }
#pragma unroll
    for (int k = 0; k < U; ++k) vec_minmax<XT>(a[k], &lo, &hi, &unordered);
  }
  group_minmax(64, &lo, &hi);
  if (group_any(64, unordered)) lo = hi = __builtin_nanf("");
  const ObserveOut o{job.scale, job.zp, nullptr, nullptr};
  if (lane == 0) emit_segment<XT>(o, s, lo, hi, gs, t.c);
}

// stage 2: fold `blk_rows` consecutive rows of a [rows, n_seg] min/max table;
// one workgroup per output cell
template <typename XT>
__global__ void __launch_bounds__(256)
minmax_fold_kernel(const typename XT::raw* __restrict__ mn_in,
                   const typename XT::raw* __restrict__ mx_in, typename XT::raw* __restrict__ mn,
                   typename XT::raw* __restrict__ mx, int64_t rows, int64_t n_seg,
                   int64_t blk_rows, int64_t out_rows) {
  __shared__ float slo[4], shi[4];
  const int64_t cells = out_rows * n_seg;
  for (int64_t cell = blockIdx.x; cell < cells; cell += gridDim.x) {
    const int64_t cr = cell / n_seg, cc = cell - cr * n_seg;
    int64_t r1 = (cr + 1) * blk_rows;
    if (r1 > rows) r1 = rows;
    float lo = __builtin_inff(), hi = -__builtin_inff();
    for (int64_t r = cr * blk_rows + threadIdx.x; r < r1; r += 256) {
      lo = nan_min(XT::to_f32(mn_in[r * n_seg + cc]), lo);
      hi = nan_max(XT::to_f32(mx_in[r * n_seg + cc]), hi);
    }
    for (int d = kWave / 2; d > 0; d >>= 1) {
      lo = nan_min(__shfl_xor(lo, d, kWave), lo);
      hi = nan_max(__shfl_xor(hi, d, kWave), hi);
    }
    if (lane_id() == 0) {
      slo[threadIdx.x / kWave] = lo;
      shi[threadIdx.x / kWave] = hi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      for (int w = 1; w < 4; ++w) {
        lo = nan_min(slo[w], lo);
        hi = nan_max(shi[w], hi);
      }
      mn[cell] = XT::from_f32(lo);
      mx[cell] = XT::from_f32(hi);
    }
    __syncthreads();
  }
}

int fill_qpcfg(QpCfg* c, int qtype, int num_bits, int symmetric, int mt, int mm_is_0d,
                      bool has_gscale, int scale_dtype, int zp_dtype) {
  int rc = quant_range(qtype, num_bits, &c->bit_min, &c->bit_max);
  if (rc) return rc;
  CTMI_REQUIRE(mt == CTMI_F32 || mt == CTMI_F16 || mt == CTMI_BF16, CTMI_ERR_UNSUPPORTED,
               "min/max must be float16/bfloat16/float32");
  const bool fp4 = qtype == CTMI_QTYPE_FLOAT && num_bits == 4;
  CTMI_REQUIRE(symmetric || !fp4, CTMI_ERR_UNSUPPORTED,
               "Asymmetric Quantization is not supported for FP4");
  c->range = c->bit_max - c->bit_min;
  c->sym_div = (float)((double)c->range / 2.0);
  c->qtype = qtype;
  c->num_bits = num_bits;
  c->symmetric = symmetric;
  c->mt = mt;
  c->zp_sub_dtype = mm_is_0d ? CTMI_F32 : mt;
  c->fp4_global = fp4 && symmetric && has_gscale;
  const int want_scale = c->fp4_global ? CTMI_F8E4M3 : mt;
  CTMI_REQUIRE(scale_dtype == want_scale, CTMI_ERR_VALUE,
               "scale output dtype %d does not match the dtype the reference produces (%d)",
               scale_dtype, want_scale);
  c->scale_dtype = scale_dtype;
  c->zp_dtype = zp_dtype;
  return CTMI_OK;
}

static void seg_geometry(SegGeom* g, const void* x, int esize, int64_t rows, int64_t cols,
                         int64_t blk_cols) {
  g->rows = rows;
  g->cols = cols;
  g->seg_cols = blk_cols < cols ? blk_cols : cols;
  g->n_seg = cdiv(cols, g->seg_cols);
  g->vec = (g->seg_cols % 8 == 0 && cols % 8 == 0 && (uintptr_t)x % (8 * esize) == 0) ? 1 : 0;
  int64_t items = g->vec ? g->seg_cols / 8 : g->seg_cols;
  int L = 1;
  while (L < 64 && L < items) L <<= 1;
  g->L = L;
}

static int seg_grid(const SegGeom& g) {
  const int64_t blocks = cdiv(g.rows * g.n_seg, 256 / g.L);
  const int64_t cap = 256 * 16;
  return (int)(blocks < cap ? (blocks < 1 ? 1 : blocks) : cap);
}

}  // namespace ctmi

using namespace ctmi;

#define CTMI_DISPATCH_XT(DTYPE, ...)                          \
  if ((DTYPE) == CTMI_BF16) { using XT = BF16; __VA_ARGS__; } \
  else if ((DTYPE) == CTMI_F16) { using XT = F16; __VA_ARGS__; } \
  else { using XT = F32; __VA_ARGS__; }

extern "C" int ctmi_calculate_qparams(const void* min_vals, const void* max_vals,
                                      int32_t mm_dtype, int32_t mm_is_0d, int64_t n,
                                      int32_t qtype, int32_t num_bits, int32_t symmetric,
                                      const float* global_scale, void* scale, int32_t scale_dtype,
                                      void* zero_point, int32_t zp_dtype, void* stream) {
  CTMI_REQUIRE(n >= 0, CTMI_ERR_VALUE, "negative size");
  QpCfg c;
  int rc = fill_qpcfg(&c, qtype, num_bits, symmetric, mm_dtype, mm_is_0d, global_scale != nullptr,
                      scale_dtype, zp_dtype);
  if (rc) return rc;
  if (n == 0) return CTMI_OK;
  CTMI_REQUIRE(min_vals && max_vals && scale, CTMI_ERR_VALUE, "NULL tensor pointer");
  const int64_t blocks = cdiv(n, 256);
  hipLaunchKernelGGL(qparams_kernel, (int)(blocks < 4096 ? blocks : 4096), 256, 0,
                     (hipStream_t)stream, min_vals, max_vals, global_scale, scale, zero_point, n, c);
  return check_launch("ctmi_calculate_qparams");
}

extern "C" int ctmi_generate_gparam(const void* min_vals, const void* max_vals, int32_t mm_dtype,
                                    int64_t n, float* out, void* stream) {
  CTMI_REQUIRE(n >= 0, CTMI_ERR_VALUE, "negative size");
  CTMI_REQUIRE(mm_dtype == CTMI_F32 || mm_dtype == CTMI_F16 || mm_dtype == CTMI_BF16,
               CTMI_ERR_UNSUPPORTED, "min/max must be float16/bfloat16/float32");
  if (n == 0) return CTMI_OK;
  CTMI_REQUIRE(min_vals && max_vals && out, CTMI_ERR_VALUE, "NULL tensor pointer");
  const int64_t blocks = cdiv(n, 256);
  hipLaunchKernelGGL(gparam_kernel, (int)(blocks < 4096 ? blocks : 4096), 256, 0,
                     (hipStream_t)stream, min_vals, max_vals, mm_dtype, out, n);
  return check_launch("ctmi_generate_gparam");
}

extern "C" int64_t ctmi_minmax_tmp_bytes(int64_t rows, int64_t cols, int64_t blk_rows,
                                         int64_t blk_cols, int32_t x_dtype) {
  if (blk_rows <= 1 || rows <= 0 || cols <= 0 || blk_cols <= 0) return 0;
  const int64_t seg = blk_cols < cols ? blk_cols : cols;
  return 2 * rows * cdiv(cols, seg) * dtype_size(x_dtype);
}

extern "C" int ctmi_minmax(const void* x, int32_t x_dtype, int64_t rows, int64_t cols,
                           int64_t blk_rows, int64_t blk_cols, void* min_out, void* max_out,
                           void* tmp, void* stream) {
  CTMI_REQUIRE(rows >= 1 && cols >= 1, CTMI_ERR_VALUE, "cannot reduce an empty tensor");
  CTMI_REQUIRE(blk_rows >= 1 && blk_cols >= 1, CTMI_ERR_VALUE, "empty cell");
  CTMI_REQUIRE(x_dtype == CTMI_F32 || x_dtype == CTMI_F16 || x_dtype == CTMI_BF16,
               CTMI_ERR_UNSUPPORTED, "min/max needs a float16/bfloat16/float32 tensor");
  CTMI_REQUIRE(x && min_out && max_out, CTMI_ERR_VALUE, "NULL tensor pointer");
  CTMI_REQUIRE(blk_rows == 1 || tmp, CTMI_ERR_VALUE, "multi-row cells need the tmp buffer");
  hipStream_t st = (hipStream_t)stream;
  SegGeom g;
  seg_geometry(&g, x, dtype_size(x_dtype), rows, cols, blk_cols);
  const int grid = seg_grid(g);
  QpCfg none{};
  if (blk_rows == 1) {
    const ObserveOut o{nullptr, nullptr, min_out, max_out};
    CTMI_DISPATCH_XT(x_dtype, {
      if (!observe_streaming<XT>(x, nullptr, o, g, none, st))
        hipLaunchKernelGGL(minmax_rows_kernel<XT>, grid, 256, 0, st, (const XT::raw*)x,
                           (XT::raw*)min_out, (XT::raw*)max_out, g);
    });
    return check_launch("ctmi_minmax");
  }
  const int64_t out_rows = cdiv(rows, blk_rows);
  const int64_t cells = out_rows * g.n_seg;
  const int es = dtype_size(x_dtype);
  void* tmn = tmp;
  void* tmx = (char*)tmp + rows * g.n_seg * es;
  const ObserveOut stage1{nullptr, nullptr, tmn, tmx};
  CTMI_DISPATCH_XT(x_dtype, {
    if (!observe_streaming<XT>(x, nullptr, stage1, g, none, st))
      hipLaunchKernelGGL(minmax_rows_kernel<XT>, grid, 256, 0, st, (const XT::raw*)x,
                         (XT::raw*)tmn, (XT::raw*)tmx, g);
    hipLaunchKernelGGL(minmax_fold_kernel<XT>, (int)(cells < 4096 ? cells : 4096), 256, 0, st,
                       (const XT::raw*)tmn, (const XT::raw*)tmx, (XT::raw*)min_out,
                       (XT::raw*)max_out, rows, g.n_seg, blk_rows, out_rows);
  });
  return check_launch("ctmi_minmax");
}

extern "C" int ctmi_observe_qparams(const void* x, int32_t x_dtype, int64_t rows, int64_t cols,
                                    int64_t blk_cols, int32_t qtype, int32_t num_bits,
                                    int32_t symmetric, const float* global_scale, void* scale,
                                    int32_t scale_dtype, void* zero_point, int32_t zp_dtype,
                                    void* min_out, void* max_out, void* stream) {
  CTMI_REQUIRE(rows >= 1 && cols >= 1, CTMI_ERR_VALUE, "cannot observe an empty tensor");
  CTMI_REQUIRE(blk_cols >= 1, CTMI_ERR_VALUE, "empty cell");
  QpCfg c;
  int rc = fill_qpcfg(&c, qtype, num_bits, symmetric, x_dtype, 0, global_scale != nullptr,
                      scale_dtype, zp_dtype);
  if (rc) return rc;
  CTMI_REQUIRE(x && scale, CTMI_ERR_VALUE, "NULL tensor pointer");
  SegGeom g;
  seg_geometry(&g, x, dtype_size(x_dtype), rows, cols, blk_cols);
  const ObserveOut o{scale, zero_point, min_out, max_out};
  // nvfp4 group-16 scales of a 16-bit tensor have a kernel of their own
  if (!min_out && !max_out && (!zero_point || zp_dtype == CTMI_F8E4M3) &&
      nvfp4_observe_try(x, x_dtype, rows, cols, blk_cols, global_scale, scale, zero_point, c,
                        (hipStream_t)stream))
    return check_launch("ctmi_observe_qparams");
  CTMI_DISPATCH_XT(x_dtype, {
    if (!observe_streaming<XT>(x, global_scale, o, g, c, (hipStream_t)stream))
      hipLaunchKernelGGL(observe_rows_kernel<XT>, seg_grid(g), 256, 0, (hipStream_t)stream,
                         (const XT::raw*)x, global_scale, scale, zero_point, (XT::raw*)min_out,
                         (XT::raw*)max_out, g, c);
  });
  return check_launch("ctmi_observe_qparams");
}

// A2 + A1 for a list of tensors: tensors whose cells stream (see observe_streaming) and share
// a dtype and a kind of kernel go into common launches, 8 per launch; any other tensor gets
// the launch ctmi_observe_qparams would give it.
extern "C" int ctmi_observe_qparams_many(const ctmi_observe_job* jobs, int64_t n, int32_t qtype,
                                         int32_t num_bits, int32_t symmetric, int32_t scale_dtype,
                                         int32_t zp_dtype, void* stream) {
  CTMI_REQUIRE(n >= 0 && (jobs || n == 0), CTMI_ERR_VALUE, "bad job list");
  struct Plan {
    QpCfg c;
    SegGeom g;
    int kind;  // 0: a launch of its own, 1: flat, 2: wide
    int64_t items;
  };
  std::vector<Plan> plans((size_t)n);
  for (int64_t i = 0; i < n; ++i) {  // every job is looked at before anything is enqueued
    const ctmi_observe_job& j = jobs[i];
    CTMI_REQUIRE(j.rows >= 1 && j.cols >= 1, CTMI_ERR_VALUE, "job %lld: cannot observe an empty tensor",
                 (long long)i);
    CTMI_REQUIRE(j.blk_cols >= 1, CTMI_ERR_VALUE, "job %lld: empty cell", (long long)i);
    Plan& p = plans[i];
    const bool fp4_global = qtype == CTMI_QTYPE_FLOAT && num_bits == 4 && symmetric && j.global_scale;
    int rc = fill_qpcfg(&p.c, qtype, num_bits, symmetric, j.x_dtype, 0, j.global_scale != nullptr,
                        scale_dtype < 0 ? (fp4_global ? CTMI_F8E4M3 : j.x_dtype) : scale_dtype,
                        zp_dtype);
    if (rc) return rc;
    CTMI_REQUIRE(j.x && j.scale, CTMI_ERR_VALUE, "job %lld: NULL tensor pointer", (long long)i);
    seg_geometry(&p.g, j.x, dtype_size(j.x_dtype), j.rows, j.cols, j.blk_cols);
    p.items = p.g.seg_cols / 8;
    p.kind = 0;
    const bool nvfp4_case = p.c.fp4_global && j.blk_cols == 16 && dtype_size(j.x_dtype) == 2;
    if (p.g.vec && p.g.cols % p.g.seg_cols == 0 && !nvfp4_case &&
        j.rows * j.cols / 8 < (1ll << 31)) {
      if (p.items <= 64 && (p.items & (p.items - 1)) == 0) p.kind = 1;
      else if (p.items > 64) p.kind = 2;
    }
  }
  hipStream_t st = (hipStream_t)stream;
  std::vector<char> done((size_t)n, 0);
  for (int64_t i = 0; i < n; ++i) {
    if (plans[i].kind != 0) continue;
    const ctmi_observe_job& j = jobs[i];
    int rc = ctmi_observe_qparams(j.x, j.x_dtype, j.rows, j.cols, j.blk_cols, qtype, num_bits, symmetric,
                                  j.global_scale, j.scale, plans[i].c.scale_dtype, j.zero_point,
                                  zp_dtype, nullptr, nullptr, stream);
    if (rc) return rc;
    done[i] = 1;
  }
  for (int64_t i = 0; i < n; ++i) {
    if (done[i]) continue;
    const Plan& lead = plans[i];
    const int xd = jobs[i].x_dtype;
    ObsChainTable t;
    std::memset(&t, 0, sizeof(t));
    t.c = lead.c;
    t.L = (int)lead.items;
    int cnt = 0;
    uint64_t chunks = 0;
    auto reset = [&]() {
      cnt = 0;
      chunks = 0;
      for (int k = 0; k < kMaxJobs; ++k) t.chunk_end[k] = 0xFFFFFFFFu;
    };
    reset();
    auto flush = [&]() {
      if (cnt == 0) return;
      CTMI_DISPATCH_XT(xd, {
        if (lead.kind == 1) {
          if constexpr (sizeof(typename XT::raw) == 2) {
            if (symmetric) hipLaunchKernelGGL((observe_flat_chain_kernel<XT, true>), (unsigned)chunks, 256, 0, st, t);
            else hipLaunchKernelGGL((observe_flat_chain_kernel<XT, false>), (unsigned)chunks, 256, 0, st, t);
          } else {
            hipLaunchKernelGGL((observe_flat_chain_kernel<XT, false>), (unsigned)chunks, 256, 0, st, t);
          }
        } else
          hipLaunchKernelGGL(observe_wide_chain_kernel<XT>, (unsigned)chunks, 256, 0, st, t);
      });
      reset();
    };
    for (int64_t k = i; k < n; ++k) {
      const Plan& p = plans[k];
      // (the scale dtype follows from the tensor's dtype and the global scale: part of what
      // tensors of one launch share)
      if (done[k] || p.kind != lead.kind || jobs[k].x_dtype != xd || p.c.scale_dtype != lead.c.scale_dtype ||
          p.c.fp4_global != lead.c.fp4_global || (lead.kind == 1 && p.items != lead.items))
        continue;
      const int64_t nvec = jobs[k].rows * jobs[k].cols / 8;
      const int64_t n_segments = jobs[k].rows * p.g.n_seg;
      const uint64_t c = (uint64_t)(lead.kind == 1 ? cdiv(nvec, 256 * kObsUnroll) : cdiv(n_segments, 4));
      if (cnt == kMaxJobs || chunks + c >= (1ull << 31)) flush();
      t.job[cnt] = ObsChainJob{jobs[k].x, jobs[k].scale, jobs[k].zero_point, jobs[k].global_scale};
      t.n_items[cnt] = (uint32_t)(lead.kind == 1 ? nvec : n_segments);
      t.per[cnt] = (uint32_t)p.items;
      chunks += c;
      t.chunk_end[cnt] = (uint32_t)chunks;
      ++cnt;
      done[k] = 1;
    }
    flush();
  }
  return n ? check_launch("ctmi_observe_qparams_many") : CTMI_OK;
}
