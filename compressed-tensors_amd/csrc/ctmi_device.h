// Device-side numeric helpers shared by every kernel: raw-bit conversions
// between fp32 and the storage formats (bf16, fp16, fp8 e4m3fn, fp4 e2m1) with
// exactly the rounding torch applies, 128-bit vector types, and wave64
// utilities.  gfx950 only.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ctmi.h"

namespace ctmi {

constexpr int kWave = 64;

// ---------------------------------------------------------------- bit casts
__device__ __forceinline__ uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }
__device__ __forceinline__ float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }

// ---------------------------------------------------------------- bf16
__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

// Round-to-nearest-even; every NaN becomes the canonical 0x7FC0, as c10::BFloat16 does.
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  uint32_t u = f2u(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7FC0;
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

// ---------------------------------------------------------------- fp16
__device__ __forceinline__ float f16_to_f32(uint16_t h) {
  return (float)__builtin_bit_cast(_Float16, h);
}
// The empty asm keeps the conversion an instruction of its own.  Left to itself the
// compiler folds a preceding multiplication into it as fma_mix(a, b, +0), and the
// +0 addend turns a product of -0 into +0.
__device__ __forceinline__ uint16_t f32_to_f16(float f) {
  asm("" : "+v"(f));
  return __builtin_bit_cast(uint16_t, (_Float16)f);
}

// ---------------------------------------------------------------- fp8 e4m3fn
// 1 sign, 4 exponent (bias 7), 3 mantissa bits; no infinities; 0x7F/0xFF = NaN; max 448.
__device__ __forceinline__ float f8e4m3_to_f32(uint8_t b) {
  uint32_t sign = (uint32_t)(b & 0x80) << 24;
  uint32_t mag = b & 0x7F;
  if (mag == 0x7F) return u2f(sign | 0x7FC00000u);
  uint32_t e = mag >> 3, m = mag & 7;
  float v;
  if (e == 0) {
    v = (float)m * 0.001953125f;  // m * 2^-9 (subnormal)
  } else {
    v = u2f(((e + 120u) << 23) | (m << 20));
  }
  return u2f(f2u(v) | sign);
}

// fp32 -> e4m3fn, round-to-nearest-even including the subnormal range (step
// 2^-9).  Magnitudes that round above 448 (> 464) and NaN give the NaN code,
// which is what torch's cast does (it does not saturate).
__device__ __forceinline__ uint8_t f32_to_f8e4m3(float f) {
  uint32_t u = f2u(f);
  uint8_t sign = (uint8_t)((u >> 24) & 0x80);
  u &= 0x7fffffffu;
  uint8_t r;
  if (u >= 0x43F00000u) {  // >= 480 (covers inf and NaN)
    r = 0x7F;
  } else if (u < 0x3C800000u) {  // < 2^-6: subnormal result, integer multiple of 2^-9
    // adding 2^14 aligns the value so that the fp32 adder performs the RNE at 2^-9
    float a = u2f(u) + 16384.0f;
    r = (uint8_t)(f2u(a) - 0x46800000u);
  } else {
    uint32_t odd = (u >> 20) & 1u;
    u += 0x7FFFFu + odd;        // RNE at bit 20
    u -= (120u << 23);          // rebias 127 -> 7
    r = (uint8_t)(u >> 20);     // 464 < |f| < 480 lands on 0x7F (NaN), as in torch
  }
  return r | sign;
}

// ---------------------------------------------------------------- fp4 e2m1
// Reference bucket rule (quant_args.py:55-68) on a non-negative magnitude.
// Returns the 3-bit magnitude code whose value is {0,.5,1,1.5,2,3,4,6}[code].
__device__ __forceinline__ int fp4_bucket(float a) {
  // boundaries: <=.25 | <.75 | <=1.25 | <1.75 | <=2.5 | <3.5 | <=5 | >5
  int c = 0;
  c += (a > 0.25f);
  c += (a >= 0.75f);
  c += (a > 1.25f);
  c += (a >= 1.75f);
  c += (a > 2.5f);
  c += (a >= 3.5f);
  c += (a > 5.0f);
  return c;
}

// fp32 bit pattern of the e2m1 magnitude {0,.5,1,1.5,2,3,4,6}[code3]: from 1.0 on
// the patterns are consecutive multiples of 2^22 starting at 254 << 22.
__device__ __forceinline__ uint32_t fp4_mag_bits(int code3) {
  const uint32_t c = (uint32_t)code3 & 7u;
  const uint32_t k = c + 252u - (c == 1u ? 1u : 0u);
  return c ? (k << 22) : 0u;
}

__device__ __forceinline__ float fp4_code_to_f32(int code3) { return u2f(fp4_mag_bits(code3)); }

// signed value of a 4-bit code (bit 3 = sign), assembled in the integer domain
__device__ __forceinline__ float fp4_decode(int code) {
  return u2f(fp4_mag_bits(code) | (((uint32_t)code & 8u) << 28));
}

// ---------------------------------------------------------------- dtype-generic scalar access
__device__ __forceinline__ float load_f32(const void* p, int dtype, int64_t i) {
  switch (dtype) {
    case CTMI_F32: return ((const float*)p)[i];
    case CTMI_F16: return f16_to_f32(((const uint16_t*)p)[i]);
    case CTMI_BF16: return bf16_to_f32(((const uint16_t*)p)[i]);
    case CTMI_F8E4M3: return f8e4m3_to_f32(((const uint8_t*)p)[i]);
    case CTMI_I8: return (float)((const int8_t*)p)[i];
    case CTMI_I16: return (float)((const int16_t*)p)[i];
    case CTMI_I32: return (float)((const int32_t*)p)[i];
    case CTMI_I64: return (float)((const int64_t*)p)[i];
    case CTMI_U8:
    case CTMI_BOOL: return (float)((const uint8_t*)p)[i];
  }
  return 0.0f;
}

// Round an fp32 value to the precision of a floating dtype and return it as fp32.
__device__ __forceinline__ float round_to(float v, int dtype) {
  switch (dtype) {
    case CTMI_F16: return f16_to_f32(f32_to_f16(v));
    case CTMI_BF16: return bf16_to_f32(f32_to_bf16(v));
    case CTMI_F8E4M3: return f8e4m3_to_f32(f32_to_f8e4m3(v));
    default: return v;
  }
}

// float -> integer cast of an already integral, in-range value; NaN -> 0.
__device__ __forceinline__ int32_t f32_to_int(float v) { return (v != v) ? 0 : (int32_t)v; }

__device__ __forceinline__ void store_from_f32(void* p, int dtype, int64_t i, float v) {
  switch (dtype) {
    case CTMI_F32: ((float*)p)[i] = v; break;
    case CTMI_F16: ((uint16_t*)p)[i] = f32_to_f16(v); break;
    case CTMI_BF16: ((uint16_t*)p)[i] = f32_to_bf16(v); break;
    case CTMI_F8E4M3: ((uint8_t*)p)[i] = f32_to_f8e4m3(v); break;
    case CTMI_I8: ((int8_t*)p)[i] = (int8_t)f32_to_int(v); break;
    case CTMI_I16: ((int16_t*)p)[i] = (int16_t)f32_to_int(v); break;
    case CTMI_I32: ((int32_t*)p)[i] = f32_to_int(v); break;
    case CTMI_U8: ((uint8_t*)p)[i] = (uint8_t)f32_to_int(v); break;
    default: break;
  }
}

// ---------------------------------------------------------------- typed storage traits
// (used by the vectorised fast paths; T is a tag type)
struct BF16 {
  using raw = uint16_t;
  static constexpr int id = CTMI_BF16;
  __device__ static __forceinline__ float to_f32(raw r) { return bf16_to_f32(r); }
  __device__ static __forceinline__ raw from_f32(float f) { return f32_to_bf16(f); }
};
struct F16 {
  using raw = uint16_t;
  static constexpr int id = CTMI_F16;
  __device__ static __forceinline__ float to_f32(raw r) { return f16_to_f32(r); }
  __device__ static __forceinline__ raw from_f32(float f) { return f32_to_f16(f); }
};
struct F32 {
  using raw = float;
  static constexpr int id = CTMI_F32;
  __device__ static __forceinline__ float to_f32(raw r) { return r; }
  __device__ static __forceinline__ raw from_f32(float f) { return f; }
};
struct F8 {
  using raw = uint8_t;
  static constexpr int id = CTMI_F8E4M3;
  __device__ static __forceinline__ float to_f32(raw r) { return f8e4m3_to_f32(r); }
  __device__ static __forceinline__ raw from_f32(float f) { return f32_to_f8e4m3(f); }
};

// 16-byte vector of N raw elements
template <typename R, int N>
struct alignas(sizeof(R) * N) Vec {
  R v[N];
};

// two fp32 -> two bf16 (round to nearest even) in one dword, by v_cvt_pk_bf16_f32: low
// half = a, high half = b.  Which NaN a NaN becomes is the instruction's choice
// (f32_to_bf16 makes every NaN 0x7FC0).
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  const f32x2 f = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
}

// 8 fp32 -> 8 elements of T with the bits T::from_f32 gives.  bfloat16 goes through the packed
// conversion; a lane whose vector holds a NaN (seen on the packed halves: magnitude above
// 0x7F80) redoes it element by element, which puts the canonical 0x7FC0 there.
template <typename T>
__device__ __forceinline__ Vec<typename T::raw, 8> pack8_exact_from_f32(const float* f) {
  if constexpr (T::id == CTMI_BF16) {
    typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));
    Vec<uint32_t, 4> w;
#pragma unroll
    for (int j = 0; j < 4; ++j) w.v[j] = pack_bf16x2(f[2 * j], f[2 * j + 1]);
    u16x2 top = __builtin_bit_cast(u16x2, w.v[0] & 0x7FFF7FFFu);
#pragma unroll
    for (int j = 1; j < 4; ++j)
      top = __builtin_elementwise_max(top, __builtin_bit_cast(u16x2, w.v[j] & 0x7FFF7FFFu));
    // + 0x7F carries into bit 15 exactly for the magnitudes above 0x7F80
    if (__builtin_expect(((__builtin_bit_cast(uint32_t, top) + 0x007F007Fu) & 0x80008000u) != 0, 0)) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        w.v[j] = (uint32_t)f32_to_bf16(f[2 * j]) | ((uint32_t)f32_to_bf16(f[2 * j + 1]) << 16);
    }
    return __builtin_bit_cast(Vec<uint16_t, 8>, w);
  } else {
    Vec<typename T::raw, 8> o;
#pragma unroll
    for (int i = 0; i < 8; ++i) o.v[i] = T::from_f32(f[i]);
    return o;
  }
}

// 8 fp32 -> 8 elements of T; bfloat16 through the packed conversion above, so for values
// that are not NaN or whose NaN bits nothing pins
template <typename T>
__device__ __forceinline__ Vec<typename T::raw, 8> pack8_from_f32(const float* f) {
  if constexpr (T::id == CTMI_BF16) {
    Vec<uint32_t, 4> w;
#pragma unroll
    for (int j = 0; j < 4; ++j) w.v[j] = pack_bf16x2(f[2 * j], f[2 * j + 1]);
    return __builtin_bit_cast(Vec<uint16_t, 8>, w);
  } else {
    Vec<typename T::raw, 8> o;
#pragma unroll
    for (int i = 0; i < 8; ++i) o.v[i] = T::from_f32(f[i]);
    return o;
  }
}

template <typename R, int N>
__device__ __forceinline__ Vec<R, N> ldg(const R* p) {
  return *reinterpret_cast<const Vec<R, N>*>(p);
}
template <typename R, int N>
__device__ __forceinline__ void stg(R* p, const Vec<R, N>& v) {
  *reinterpret_cast<Vec<R, N>*>(p) = v;
}

// Streaming (non-temporal) variants for data that is touched once: they keep
// the caches for the small operands that are reused (scales, zero points) and,
// measured on MI355X, raise the HBM rate of out-of-cache passes by 5-15 %.
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

template <int BYTES>
struct NativeVec;
template <>
struct NativeVec<1> { using type = uint8_t; };
template <>
struct NativeVec<2> { using type = uint16_t; };
template <>
struct NativeVec<4> { using type = uint32_t; };
template <>
struct NativeVec<8> { using type = u32x2_t; };
template <>
struct NativeVec<16> { using type = u32x4_t; };

template <typename R, int N>
__device__ __forceinline__ Vec<R, N> ldg_nt(const R* p) {
  constexpr int BYTES = sizeof(R) * N;
  if constexpr (BYTES == 32) {
    struct Two { u32x4_t a, b; };
    Two t;
    t.a = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
    t.b = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p) + 1);
    return __builtin_bit_cast(Vec<R, N>, t);
  } else {
    using NV = typename NativeVec<BYTES>::type;
    return __builtin_bit_cast(Vec<R, N>, __builtin_nontemporal_load(reinterpret_cast<const NV*>(p)));
  }
}
template <typename R, int N>
__device__ __forceinline__ void stg_nt(R* p, const Vec<R, N>& v) {
  constexpr int BYTES = sizeof(R) * N;
  if constexpr (BYTES == 32) {
    struct Two { u32x4_t a, b; };
    const Two t = __builtin_bit_cast(Two, v);
    __builtin_nontemporal_store(t.a, reinterpret_cast<u32x4_t*>(p));
    __builtin_nontemporal_store(t.b, reinterpret_cast<u32x4_t*>(p) + 1);
  } else {
    using NV = typename NativeVec<BYTES>::type;
    __builtin_nontemporal_store(__builtin_bit_cast(NV, v), reinterpret_cast<NV*>(p));
  }
}

// ---------------------------------------------------------------- wave64 helpers
__device__ __forceinline__ int lane_id() { return (int)(threadIdx.x & (kWave - 1)); }

template <typename T>
__device__ __forceinline__ T wave_shfl_xor(T v, int mask) {
  return __shfl_xor(v, mask, kWave);
}

// XCD-aware remap of a 1-D block index: consecutive logical tiles are placed on
// the same XCD (hardware hands consecutive workgroup ids round-robin to the 8
// XCDs), so that neighbouring tiles share that XCD's L2.
__device__ __forceinline__ int64_t xcd_remap(int64_t bid, int64_t nblocks) {
  constexpr int64_t kXcd = 8;
  int64_t full = (nblocks / kXcd) * kXcd;
  if (bid >= full) return bid;
  int64_t per = full / kXcd;
  return (bid % kXcd) * per + bid / kXcd;
}

}  // namespace ctmi
