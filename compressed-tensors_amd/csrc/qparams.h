// calculate_qparams for one (min, max) pair (quantization/utils/helpers.py:67-146),
// shared by the observers and by kernels that derive scales in their epilogue.
#pragma once

#include "ctmi_device.h"

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

}  // namespace ctmi
