// The arithmetic of quantize / dequantize / fake-quantize on 8 neighbouring
// elements that share one scale (forward.py:455-514), for float tensors whose
// scale has their dtype and codes that are int8 or float8_e4m3fn.  Shared by the
// streaming kernels and by the kernels that derive the scale themselves.
#pragma once

#include "ctmi_device.h"
#include "quant_core.h"
#include "quant_fast.h"

namespace ctmi {

constexpr int kKindFloat = 0, kKindI8 = 1, kKindF8 = 2;

template <int CT>
__device__ __forceinline__ void round2(float& a, float& b) {
  if constexpr (CT == CTMI_BF16) {
    const uint32_t p = pack_bf16x2(a, b);
    a = bf16_lo(p);
    b = bf16_hi(p);
  } else if constexpr (CT == CTMI_F16) {
    a = f16_to_f32(f32_to_f16(a));
    b = f16_to_f32(f32_to_f16(b));
  }
}

__device__ __forceinline__ float fp8_hw_decode(uint32_t word, int byte) {
  switch (byte) {
    case 0: return __builtin_amdgcn_cvt_f32_fp8((int)word, 0);
    case 1: return __builtin_amdgcn_cvt_f32_fp8((int)word, 1);
    case 2: return __builtin_amdgcn_cvt_f32_fp8((int)word, 2);
    default: return __builtin_amdgcn_cvt_f32_fp8((int)word, 3);
  }
}

// FT: float dtype tag of x / scale / float output.  IN / OUT: element kind of the
// input and output (kKindFloat, kKindI8, kKindF8).  QK: 0 = integer grid, 1 = fp8
// grid.  xf is read when IN is float, xc otherwise; out_float is written when OUT
// is float, out_codes otherwise.
// SS: 0 = one scale / zero point for the 8 elements (s[0], z[0]), 1 = one per
// element (s[i], z[i]: activation-ordered groups).
template <typename FT, int IN, int OUT, int QK, bool HAS_ZP, int SS>
__device__ __forceinline__ void qdq_vec8_impl(const Vec<typename FT::raw, 8>& xf,
                                              const Vec<uint8_t, 8>& xc, const float* s,
                                              const float* z, float qmin, float qmax,
                                              Vec<typename FT::raw, 8>* out_float,
                                              Vec<uint8_t, 8>* out_codes) {
  constexpr int CT = FT::id;
  constexpr bool DO_Q = IN == kKindFloat;
  constexpr bool DO_DQ = OUT == kKindFloat;
  using FR = typename FT::raw;
  float t[8];
  uint32_t codes[2] = {0u, 0u};  // 8 one-byte codes
  if constexpr (DO_Q) {
    bool tame = scale_is_tame(s[0]);
    if constexpr (SS != 0) {
#pragma unroll
      for (int i = 1; i < 8; ++i) tame &= scale_is_tame(s[i]);
    }
    const bool fast = CT == CTMI_BF16 && __builtin_expect(wave_all(tame), 1);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float a = FT::to_f32(xf.v[2 * j]), b = FT::to_f32(xf.v[2 * j + 1]);
      const float sa = s[SS * 2 * j], sb = s[SS * (2 * j + 1)];
      if (fast) { a *= __builtin_amdgcn_rcpf(sa); b *= __builtin_amdgcn_rcpf(sb); } else { a /= sa; b /= sb; }
      round2<CT>(a, b);
      if (HAS_ZP) { a += z[SS * 2 * j]; b += z[SS * (2 * j + 1)]; round2<CT>(a, b); }
      a = clamp_nan(a, qmin, qmax);
      b = clamp_nan(b, qmin, qmax);
      if constexpr (QK == 0) {
        a = rintf(a);
        b = rintf(b);
        if constexpr (OUT == kKindI8) {
          codes[j / 2] |= ((uint32_t)(uint8_t)(int8_t)f32_to_int(a)) << (16 * (j % 2));
          codes[j / 2] |= ((uint32_t)(uint8_t)(int8_t)f32_to_int(b)) << (16 * (j % 2) + 8);
        }
      } else {
        // two fp8 codes into the low or high half of the word
        if (j % 2 == 0) codes[j / 2] = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)codes[j / 2], false);
        else codes[j / 2] = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)codes[j / 2], true);
        if constexpr (DO_DQ) {
          a = fp8_hw_decode(codes[j / 2], 2 * (j % 2));
          b = fp8_hw_decode(codes[j / 2], 2 * (j % 2) + 1);
        }
      }
      t[2 * j] = a;
      t[2 * j + 1] = b;
    }
  } else {
    const Vec<uint32_t, 2> w = __builtin_bit_cast(Vec<uint32_t, 2>, xc);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if constexpr (IN == kKindI8) t[i] = (float)(int8_t)((w.v[i / 4] >> (8 * (i % 4))) & 0xffu);
      else t[i] = fp8_hw_decode(w.v[i / 4], i % 4);
    }
  }
  if constexpr (DO_DQ) {
    Vec<FR, 8> o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float a = t[2 * j], b = t[2 * j + 1];
      if (HAS_ZP) { a -= z[SS * 2 * j]; b -= z[SS * (2 * j + 1)]; round2<CT>(a, b); }
      a *= s[SS * 2 * j];
      b *= s[SS * (2 * j + 1)];
      if constexpr (CT == CTMI_BF16) {
        const uint32_t p = pack_bf16x2(a, b);
        o.v[2 * j] = (uint16_t)(p & 0xffffu);
        o.v[2 * j + 1] = (uint16_t)(p >> 16);
      } else {
        o.v[2 * j] = FT::from_f32(a);
        o.v[2 * j + 1] = FT::from_f32(b);
      }
    }
    *out_float = o;
  } else {
    Vec<uint32_t, 2> w;
    w.v[0] = codes[0];
    w.v[1] = codes[1];
    *out_codes = __builtin_bit_cast(Vec<uint8_t, 8>, w);
  }
}

template <typename FT, int IN, int OUT, int QK, bool HAS_ZP>
__device__ __forceinline__ void qdq_vec8(const Vec<typename FT::raw, 8>& xf,
                                         const Vec<uint8_t, 8>& xc, float s, float z, float qmin,
                                         float qmax, Vec<typename FT::raw, 8>* out_float,
                                         Vec<uint8_t, 8>* out_codes) {
  qdq_vec8_impl<FT, IN, OUT, QK, HAS_ZP, 0>(xf, xc, &s, &z, qmin, qmax, out_float, out_codes);
}

}  // namespace ctmi
