// Per-element quantize / dequantize arithmetic, shared by the generic and the
// vectorised kernels so that every code path rounds identically.
#pragma once

#include "ctmi_device.h"

namespace ctmi {

struct QuantCfg {
  float qmin, qmax;
  int qtype;     // CTMI_QTYPE_*
  int num_bits;
  int ct;        // dtype the quantize chain is evaluated in (promotion of x and scale)
  int dt;        // dtype the dequantize chain is evaluated in (the effective scale's dtype)
};

// torch.clamp: NaN propagates.
__device__ __forceinline__ float clamp_nan(float v, float lo, float hi) {
  return (v != v) ? v : fminf(fmaxf(v, lo), hi);
}

// FP4_E2M1_DATA.cast_to_fp4 (quant_args.py:55-68): bucket |v| onto the e2m1
// grid, then multiply by sign(v) — so an exact zero gives +0 and a negative
// value that rounds to zero gives -0.
__device__ __forceinline__ float cast_to_fp4(float v) {
  if (v != v) return v;
  float sgn = (v > 0.0f) ? 1.0f : ((v < 0.0f) ? -1.0f : 0.0f);
  return fp4_code_to_f32(fp4_bucket(fabsf(v))) * sgn;
}

template <int CT>
__device__ __forceinline__ float round_ct(float v) {
  if constexpr (CT == CTMI_BF16) return bf16_to_f32(f32_to_bf16(v));
  else if constexpr (CT == CTMI_F16) return f16_to_f32(f32_to_f16(v));
  else return v;
}

// _quantize, forward.py:471-482, evaluated in compute dtype `ct`.
//   x      input element as fp32
//   s      effective scale as fp32 (already divided by the global scale if any)
//   zq     zero_point.to(x.dtype) as fp32
__device__ __forceinline__ float quantize_value(float x, float s, float zq, bool has_zp,
                                                const QuantCfg& q) {
  float v = round_to(x / s, q.ct);
  if (has_zp) v = round_to(v + zq, q.ct);
  v = clamp_nan(v, q.qmin, q.qmax);
  if (q.qtype == CTMI_QTYPE_INT) {
    v = rintf(v);
  } else if (q.num_bits == 8) {
    v = f8e4m3_to_f32(f32_to_f8e4m3(v));
  } else {
    v = cast_to_fp4(v);
  }
  return v;
}

// _dequantize, forward.py:504-509, evaluated in dtype `dt`.
//   zd     zero_point.to(scale.dtype) as fp32
__device__ __forceinline__ float dequantize_value(float q, float s, float zd, bool has_zp, int dt) {
  float v = round_to(q, dt);
  if (has_zp) v = round_to(v - zd, dt);
  return round_to(v * s, dt);
}

}  // namespace ctmi
