// calculate_qparams for one (min, max) pair (quantization/utils/helpers.py:67-146),
// shared by the observers and by kernels that derive scales in their epilogue.
#pragma once

#include "ctmi_device.h"
#include "qdq_core.h"

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

// Returns the scale rounded to its storage dtype, and the zero point before its
// storage cast, both as fp32.  MT >= 0 fixes the dtype of min / max at compile
// time (c.mt and c.zp_sub_dtype are then not looked at), which removes the dtype
// dispatch from every rounding step.
template <int MT = -1>
__device__ __forceinline__ void qparams_value(float mn, float mx, float gs, const QpCfg& cfg,
                                              float* scale, float* zp) {
  constexpr float kEps = 1.1920928955078125e-07f;  // torch.finfo(torch.float32).eps
  struct {
    float bit_min, bit_max, sym_div, range;
    int qtype, symmetric, mt, zp_sub_dtype, fp4_global;
  } c = {cfg.bit_min, cfg.bit_max, cfg.sym_div, cfg.range, cfg.qtype, cfg.symmetric,
         MT >= 0 ? MT : cfg.mt, MT >= 0 ? MT : cfg.zp_sub_dtype, cfg.fp4_global};
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

// The zero point as quantize / dequantize read it back from its storage dtype: fp8
// rounds it, an integer dtype has no -0 (rint of a small negative value gives one).
__device__ __forceinline__ float stored_zero_point(float z, const QpCfg& c) {
  return c.qtype == CTMI_QTYPE_INT ? z + 0.0f : round_to(z, c.zp_dtype);
}

// ------------------------------------------------------------------ compile-time forms
// calculate_qparams for an int or fp8 scheme without a global scale, min / max in
// XT, with the dtype and scheme dispatch of qparams_value resolved at compile time
// and the NaN bookkeeping left to the caller (has_nan: the cell holds a NaN).
constexpr float kScaleFloor = 1.1920928955078125e-07f;  // torch.finfo(torch.float32).eps

template <typename XT>
__device__ __forceinline__ float round_xt(float v) {
  float same = v;
  round2<XT::id>(v, same);
  return v;
}

// symmetric: scale = max(XT(max|x| / (range / 2)), eps)
template <typename XT>
__device__ __forceinline__ float symmetric_scale(float absmax, bool has_nan, float half_range) {
  float t;
  if constexpr (XT::id == CTMI_BF16) {
    // bf16 / bf16 (7.5, 127.5 and 448 are bf16 values): the product with the
    // reciprocal rounds to the same bf16 as the quotient
    t = absmax * __builtin_amdgcn_rcpf(half_range);
  } else {
    t = absmax / half_range;
  }
  const float s = __builtin_fmaxf(round_xt<XT>(t), kScaleFloor);
  return has_nan ? __builtin_nanf("") : s;
}

// asymmetric: scale = max(XT(XT(max - min) / range), eps),
//             zp = clamp(XT(qmin - XT(min / scale)), qmin, qmax), rounded to an integer
// (QK 0, stored as int8) or to fp8 (QK 1), as quantize / dequantize read it back
template <typename XT, int QK>
__device__ __forceinline__ void asymmetric_qparams(float lo, float hi, bool has_nan, float qmin,
                                                   float qmax, float* scale, float* zp) {
  const float mn = __builtin_fminf(lo, 0.0f), mx = __builtin_fmaxf(hi, 0.0f);
  float s = round_xt<XT>(round_xt<XT>(mx - mn) / (qmax - qmin));
  s = (s != s) ? s : __builtin_fmaxf(s, kScaleFloor);  // inf - inf
  float z = round_xt<XT>(qmin - round_xt<XT>(mn / s));
  z = (z != z) ? z : __builtin_fminf(__builtin_fmaxf(z, qmin), qmax);
  if constexpr (QK == 0) {
    z = rintf(z) + 0.0f;  // an int8 zero point has no -0
  } else {
    if (z == z) z = __builtin_amdgcn_cvt_f32_fp8(__builtin_amdgcn_cvt_pk_fp8_f32(z, z, 0, false), 0);
  }
  const float nan = __builtin_nanf("");
  *scale = has_nan ? nan : s;
  *zp = has_nan ? nan : z;
}

}  // namespace ctmi
