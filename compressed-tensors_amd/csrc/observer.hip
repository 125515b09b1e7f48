// Scale / zero-point derivation: min-max reduction and calculate_qparams.
//
//   calculate_qparams              quantization/utils/helpers.py:67-146
//   compute_dynamic_scales_and_zp  helpers.py:149-205
//   generate_gparam                helpers.py:414-434
//   min-max observer               tests/mock_observer.py:38-56 (amin / amax per slice)
//
// calculate_qparams is evaluated in the dtype of the min/max tensors (each op
// rounded to it), except where the reference's operands promote to fp32.
#include "ctmi_device.h"
#include "ctmi_host.h"

namespace ctmi {

// torch.min / torch.max / amin / amax propagate NaN
__device__ __forceinline__ float nan_min(float a, float b) { return (a < b || a != a) ? a : b; }
__device__ __forceinline__ float nan_max(float a, float b) { return (a > b || a != a) ? a : b; }

struct QpCfg {
  float bit_min, bit_max;
  float sym_div;     // float(bit_max - bit_min) / 2
  float range;       // float(bit_max - bit_min)
  int qtype, num_bits, symmetric;
  int mt;            // dtype of min/max (and of the non-fp8 scales)
  int zp_sub_dtype;  // dtype of `bit_min - min/scale`: mt, or fp32 when min/max are 0-d
  int fp4_global;    // fp4 with a global scale: fp8 scales
  int scale_dtype, zp_dtype;
};

// returns scale and zero point as fp32 values already rounded to their storage dtypes
__device__ __forceinline__ void qparams_value(float mn, float mx, float gs, const QpCfg& c,
                                              float* scale, float* zp) {
  constexpr float kEps = 1.1920928955078125e-07f;  // torch.finfo(torch.float32).eps
  mn = nan_min(mn, 0.0f);
  mx = nan_max(mx, 0.0f);
  float s, z;
  if (c.symmetric) {
    const float m = nan_max(fabsf(mn), fabsf(mx));
    if (c.fp4_global) {
      s = gs * round_to(m / 6.0f, c.mt);                 // fp32: global_scale is an fp32 tensor
      s = (s != s) ? s : fminf(fmaxf(s, -448.0f), 448.0f);
      s = f8e4m3_to_f32(f32_to_f8e4m3(s));
      if (s == 0.0f) s = 0.125f;
    } else {
      s = round_to(m / c.sym_div, c.mt);
      s = (s != s) ? s : fmaxf(s, kEps);
    }
    z = 0.0f;
  } else {
    s = round_to(round_to(mx - mn, c.mt) / c.range, c.mt);
    s = (s != s) ? s : fmaxf(s, kEps);
    z = round_to(c.bit_min - round_to(mn / s, c.mt), c.zp_sub_dtype);
    z = (z != z) ? z : fminf(fmaxf(z, c.bit_min), c.bit_max);
    if (c.qtype == CTMI_QTYPE_INT) z = rintf(z);
  }
  *scale = s;
  *zp = z;
}

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
    out[i] = round_to(2688.0f / m, mt);  // 448 * 6 / max|x| in the min/max dtype, then -> fp32
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

static int fill_qpcfg(QpCfg* c, int qtype, int num_bits, int symmetric, int mt, int mm_is_0d,
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
  if (blk_rows == 1) {
    CTMI_DISPATCH_XT(x_dtype, hipLaunchKernelGGL(minmax_rows_kernel<XT>, grid, 256, 0, st,
                                                 (const XT::raw*)x, (XT::raw*)min_out,
                                                 (XT::raw*)max_out, g));
    return check_launch("ctmi_minmax");
  }
  const int64_t out_rows = cdiv(rows, blk_rows);
  const int64_t cells = out_rows * g.n_seg;
  const int es = dtype_size(x_dtype);
  void* tmn = tmp;
  void* tmx = (char*)tmp + rows * g.n_seg * es;
  CTMI_DISPATCH_XT(x_dtype, {
    hipLaunchKernelGGL(minmax_rows_kernel<XT>, grid, 256, 0, st, (const XT::raw*)x, (XT::raw*)tmn,
                       (XT::raw*)tmx, g);
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
  CTMI_DISPATCH_XT(x_dtype, hipLaunchKernelGGL(observe_rows_kernel<XT>, seg_grid(g), 256, 0,
                                               (hipStream_t)stream, (const XT::raw*)x,
                                               global_scale, scale, zero_point,
                                               (XT::raw*)min_out, (XT::raw*)max_out, g, c));
  return check_launch("ctmi_observe_qparams");
}
