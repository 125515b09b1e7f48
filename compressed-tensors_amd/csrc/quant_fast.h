// Register-level building blocks of the vectorised quantize+pack and
// unpack+dequantize kernels: 8 neighbouring elements that share one scale.
//
// The generic versions replay the reference chain with an IEEE division per
// element.  The bf16-by-bf16 versions get the same bits with one multiply:
//
//   The reference computes t = bf16(fp32(x) / fp32(s)) (forward.py:471, bf16
//   tensors: fp32 divide, one rounding to bf16).  x and s carry 8-bit
//   significands, so the exact quotient X/S never sits on a bf16 rounding
//   midpoint and stays at least 2^-16.8 (relative) away from the nearest one
//   (checked for all 128 x 128 significand pairs).  Any approximation of the
//   quotient with a relative error below that gap therefore rounds to the same
//   bf16 value; x * v_rcp_f32(s) is within 2^-22.  Scales outside
//   [2^-100, 2^100] (and NaN) take the division path.
//
// Rounding to bf16 uses v_cvt_pk_bf16_f32, rounding to an integer code uses the
// 1.5 * 2^23 trick: adding it makes the fp32 adder round to nearest-even at
// integer granularity, and with the unsigned offset folded into the constant the
// low bits of the sum are the packed field.
#pragma once

#include "ctmi_device.h"
#include "quant_core.h"

namespace ctmi {

typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float bf16_lo(uint32_t w) { return u2f(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return u2f(w & 0xffff0000u); }

// True when `p` holds on every active lane of the wavefront.  Branching on it is a
// scalar branch: a rare slow path then costs the common one nothing.
__device__ __forceinline__ bool wave_all(bool p) { return __builtin_amdgcn_ballot_w64(!p) == 0; }

__device__ __forceinline__ bool scale_is_tame(float s) {
  const float a = fabsf(s);
  return a >= 7.888609052210118e-31f && a <= 1.2676506002282294e30f;  // 2^-100 .. 2^100
}

template <int BITS>
struct PackConst {
  static constexpr int PF = 32 / BITS;
  static constexpr int OFF = 1 << (BITS - 1);
  static constexpr float MAGIC = 12582912.0f + (float)OFF;  // 1.5 * 2^23 + offset
  // sum over the PF fields of a word of (0x4B400000 << BITS*i), modulo 2^32
  static constexpr uint32_t bias() {
    uint32_t b = 0;
    for (int i = 0; i < PF; ++i) b += 0x4B400000u << (BITS * i);
    return b;
  }
};

// ---------------------------------------------------------------- quantize + pack, 8 elements
// generic: IEEE division, software rounding to the compute dtype
template <typename XT, int CT, int BITS, bool HAS_ZP>
__device__ __forceinline__ Vec<int32_t, BITS / 4> quant_pack8_exact(
    const Vec<typename XT::raw, 8>& xv, float s, float z, float qmin, float qmax) {
  constexpr int W = BITS / 4;
  constexpr int PF = 32 / BITS;
  constexpr int OFF = 1 << (BITS - 1);
  Vec<int32_t, W> o;
#pragma unroll
  for (int w = 0; w < W; ++w) {
    uint32_t acc = 0;
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      float t = round_ct<CT>(XT::to_f32(xv.v[w * PF + i]) / s);
      if (HAS_ZP) t = round_ct<CT>(t + z);
      t = rintf(clamp_nan(t, qmin, qmax));
      acc |= ((uint32_t)(f32_to_int(t) + OFF) & ((1u << BITS) - 1u)) << (BITS * i);
    }
    o.v[w] = (int32_t)acc;
  }
  return o;
}

// bf16 input, bf16 scale: multiply by the reciprocal (see the header comment)
template <int BITS, bool HAS_ZP>
__device__ __forceinline__ Vec<int32_t, BITS / 4> quant_pack8_bf16(const Vec<uint16_t, 8>& xv,
                                                                  float s, float z, float qmin,
                                                                  float qmax) {
  using PC = PackConst<BITS>;
  constexpr int W = BITS / 4;
  if (__builtin_expect(!wave_all(scale_is_tame(s)), 0))
    return quant_pack8_exact<BF16, CTMI_BF16, BITS, HAS_ZP>(xv, s, z, qmin, qmax);
  const float r = __builtin_amdgcn_rcpf(s);
  const Vec<uint32_t, 4> xw = __builtin_bit_cast(Vec<uint32_t, 4>, xv);
  // a zero point of 0 leaves every code unchanged (it only turns -0 into +0)
  const bool add_zp = HAS_ZP && z != 0.0f;
  uint32_t acc[W];
#pragma unroll
  for (int w = 0; w < W; ++w) acc[w] = 0u - PC::bias();
#pragma unroll
  for (int j = 0; j < 4; ++j) {  // two elements per dword
    uint32_t t = pack_bf16x2(bf16_lo(xw.v[j]) * r, bf16_hi(xw.v[j]) * r);
    if (add_zp) t = pack_bf16x2(bf16_lo(t) + z, bf16_hi(t) + z);
    const float c0 = __builtin_amdgcn_fmed3f(bf16_lo(t), qmin, qmax) + PC::MAGIC;
    const float c1 = __builtin_amdgcn_fmed3f(bf16_hi(t), qmin, qmax) + PC::MAGIC;
    const int e0 = 2 * j, e1 = 2 * j + 1;
    acc[e0 / PC::PF] += f2u(c0) << (BITS * (e0 % PC::PF));
    acc[e1 / PC::PF] += f2u(c1) << (BITS * (e1 % PC::PF));
  }
  Vec<int32_t, W> o;
#pragma unroll
  for (int w = 0; w < W; ++w) o.v[w] = (int32_t)acc[w];
  return o;
}

template <typename XT, typename ST, int BITS, bool HAS_ZP>
__device__ __forceinline__ Vec<int32_t, BITS / 4> quant_pack8(const Vec<typename XT::raw, 8>& xv,
                                                             float s, float z, float qmin,
                                                             float qmax) {
  if constexpr (XT::id == CTMI_BF16 && ST::id == CTMI_BF16) {
    return quant_pack8_bf16<BITS, HAS_ZP>(xv, s, z, qmin, qmax);
  } else {
    constexpr int CT = (XT::id == ST::id) ? XT::id : CTMI_F32;
    return quant_pack8_exact<XT, CT, BITS, HAS_ZP>(xv, s, z, qmin, qmax);
  }
}

// ---------------------------------------------------------------- unpack + dequantize, 8 elements
// Byte k of a word as a float, in one instruction (extract + convert).
template <int K>
__device__ __forceinline__ float ubyte_to_f32(uint32_t w) {
  float f;
  if constexpr (K == 0) asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(f) : "v"(w));
  else if constexpr (K == 1) asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(f) : "v"(w));
  else if constexpr (K == 2) asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(f) : "v"(w));
  else asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(f) : "v"(w));
  return f;
}

// The reference computes (float(q) - zp) * scale with every step in the scale's
// dtype (forward.py:504-509).  q - zp is an integer of at most 8 bits, exact in
// every float type here, so the chain rounds once, at the end.  With u = q + OFF
// the stored code and off = OFF + zp:
//   fused form   fma(u, s, -(off * s)): u*s and off*s are exact in fp32 when s
//                has at most 11 significant bits (bf16 / fp16 scales) or off is a
//                power of two (no zero point), and the fma rounds the exact
//                (u - off) * s once: the same value as the two-step form.  Only
//                taken for scales of ordinary magnitude, where off * s can
//                neither overflow nor lose bits to underflow;
//   two-step     (u - off) * s, always valid.
template <typename ST, int BITS, bool HAS_ZP>
__device__ __forceinline__ Vec<typename ST::raw, 8> unpack_dequant8(const Vec<int32_t, BITS / 4>& pv,
                                                                    float s, float z) {
  constexpr int OFF = 1 << (BITS - 1);
  constexpr bool kFusable = ST::id != CTMI_F32 || !HAS_ZP;
  const float off = (float)OFF + (HAS_ZP ? z : 0.0f);
  uint32_t b[2];  // the 8 codes, one per byte
  if constexpr (BITS == 4) {
    const uint32_t w = (uint32_t)pv.v[0];
    b[0] = w & 0x0F0F0F0Fu;         // elements 0, 2, 4, 6
    b[1] = (w >> 4) & 0x0F0F0F0Fu;  // elements 1, 3, 5, 7
  } else {
    b[0] = (uint32_t)pv.v[0];
    b[1] = (uint32_t)pv.v[1];
  }
  float f[8];
  if constexpr (BITS == 4) {
    f[0] = ubyte_to_f32<0>(b[0]); f[1] = ubyte_to_f32<0>(b[1]);
    f[2] = ubyte_to_f32<1>(b[0]); f[3] = ubyte_to_f32<1>(b[1]);
    f[4] = ubyte_to_f32<2>(b[0]); f[5] = ubyte_to_f32<2>(b[1]);
    f[6] = ubyte_to_f32<3>(b[0]); f[7] = ubyte_to_f32<3>(b[1]);
  } else {
    f[0] = ubyte_to_f32<0>(b[0]); f[1] = ubyte_to_f32<1>(b[0]);
    f[2] = ubyte_to_f32<2>(b[0]); f[3] = ubyte_to_f32<3>(b[0]);
    f[4] = ubyte_to_f32<0>(b[1]); f[5] = ubyte_to_f32<1>(b[1]);
    f[6] = ubyte_to_f32<2>(b[1]); f[7] = ubyte_to_f32<3>(b[1]);
  }
  // (a negative scale takes the two-step form too: it gives -0 where the fma gives +0)
  if (kFusable && __builtin_expect(wave_all(s >= 7.888609052210118e-31f && s <= 1.2676506002282294e30f), 1)) {
    const float c = -(off * s);
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = __builtin_fmaf(f[i], s, c);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = (f[i] - off) * s;
  }
  Vec<typename ST::raw, 8> o;
  if constexpr (ST::id == CTMI_BF16) {
    Vec<uint32_t, 4> ow;
#pragma unroll
    for (int j = 0; j < 4; ++j) ow.v[j] = pack_bf16x2(f[2 * j], f[2 * j + 1]);
    o = __builtin_bit_cast(Vec<uint16_t, 8>, ow);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) o.v[i] = ST::from_f32(f[i]);
  }
  return o;
}

}  // namespace ctmi
