// Min / max of the elements a lane holds and over groups of neighbouring lanes,
// for the observers and for kernels that derive scales from the data they hold.
#pragma once

#include "ctmi_device.h"

namespace ctmi {

// min / max of 8 elements folded into lo / hi with the hardware's 3-operand min
// and max (which skip NaNs); `unordered` collects whether a NaN was seen, for the
// caller to put back (torch's amin / amax propagate it).
template <typename XT>
__device__ __forceinline__ void vec_minmax(const Vec<typename XT::raw, 8>& a, float* lo, float* hi,
                                           bool* unordered) {
#pragma unroll
  for (int j = 0; j < 8; j += 2) {
    const float f0 = XT::to_f32(a.v[j]), f1 = XT::to_f32(a.v[j + 1]);
    *lo = __builtin_fminf(__builtin_fminf(*lo, f0), f1);
    *hi = __builtin_fmaxf(__builtin_fmaxf(*hi, f0), f1);
    *unordered |= __builtin_isunordered(f0, f1);
  }
}

// one step of a min / max reduction over neighbouring lanes, on the data-parallel
// permute path of the vector ALU (no LDS traffic): CTRL names the lane exchange
template <int CTRL>
__device__ __forceinline__ void dpp_minmax_step(float* lo, float* hi) {
  const float l = __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, *lo), CTRL, 0xf, 0xf, false));
  const float h = __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, *hi), CTRL, 0xf, 0xf, false));
  *lo = __builtin_fminf(*lo, l);
  *hi = __builtin_fmaxf(*hi, h);
}

// all-reduce over aligned groups of L lanes (L a power of two <= 64)
__device__ __forceinline__ void group_minmax(int L, float* lo, float* hi) {
  if (L >= 2) dpp_minmax_step<0xB1>(lo, hi);   // quad_perm [1,0,3,2]
  if (L >= 4) dpp_minmax_step<0x4E>(lo, hi);   // quad_perm [2,3,0,1]
  if (L >= 8) dpp_minmax_step<0x141>(lo, hi);  // row_half_mirror
  if (L >= 16) dpp_minmax_step<0x140>(lo, hi); // row_mirror
  for (int d = 16; d < L; d <<= 1) {
    *lo = __builtin_fminf(__shfl_xor(*lo, d, kWave), *lo);
    *hi = __builtin_fmaxf(__shfl_xor(*hi, d, kWave), *hi);
  }
}

// did any lane of this lane's group of L see a NaN?
__device__ __forceinline__ bool group_any(int L, bool flag) {
  const uint64_t m = __builtin_amdgcn_ballot_w64(flag);
  const uint64_t group = L >= 64 ? ~0ull : (((1ull << L) - 1) << (lane_id() & ~(L - 1)));
  return (m & group) != 0;
}

// ------------------------------------------------------------------ |x| maximum on the raw bits
// For a symmetric scheme only max|x| matters (helpers.py:87-110 with min <= 0 <= max:
// max(|min|, |max|) = max|x|).  The magnitude bits of a 16-bit float order like
// unsigned integers, NaNs above infinity, so two elements go through one packed
// integer maximum and a NaN shows in the result by itself.
typedef uint16_t u16x2_t __attribute__((ext_vector_type(2)));

template <typename XT>
__device__ __forceinline__ uint32_t absmax8_bits(const Vec<typename XT::raw, 8>& a) {
  static_assert(sizeof(typename XT::raw) == 2, "16-bit floats only");
  const Vec<uint32_t, 4> w = __builtin_bit_cast(Vec<uint32_t, 4>, a);
  u16x2_t m[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) m[j] = __builtin_bit_cast(u16x2_t, w.v[j] & 0x7fff7fffu);
  const u16x2_t r = __builtin_elementwise_max(__builtin_elementwise_max(m[0], m[1]),
                                              __builtin_elementwise_max(m[2], m[3]));
  return r.x > r.y ? (uint32_t)r.x : (uint32_t)r.y;
}

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_umax_step(uint32_t v) {
  const uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, false);
  return o > v ? o : v;
}

// all-reduce over aligned groups of L lanes (L a power of two <= 64)
__device__ __forceinline__ uint32_t group_umax(int L, uint32_t v) {
  if (L >= 2) v = dpp_umax_step<0xB1>(v);
  if (L >= 4) v = dpp_umax_step<0x4E>(v);
  if (L >= 8) v = dpp_umax_step<0x141>(v);
  if (L >= 16) v = dpp_umax_step<0x140>(v);
  for (int d = 16; d < L; d <<= 1) {
    const uint32_t o = (uint32_t)__shfl_xor((int)v, d, kWave);
    v = o > v ? o : v;
  }
  return v;
}

}  // namespace ctmi
