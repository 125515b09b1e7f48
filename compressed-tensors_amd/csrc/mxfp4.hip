// MXFP4 group scales: powers of two stored as uint8 exponents
// (quantization/utils/mxfp4_utils.py: convert_mxfp4_exp_scale :24-38,
// round_to_power_2 :41-73, generate_mxfp4_scales :76-97).  The tensors are one
// value per group of 32 weights, so these are small elementwise passes.
#include "ctmi_device.h"
#include "ctmi_host.h"

namespace ctmi {

// keep sign and exponent of a bfloat16 after adding half of the e2m1 mantissa step
// (1 << (7 - 1 - 1)): the power of two that, as a group scale, keeps the group's
// maximum inside the fp4 range
__device__ __forceinline__ uint16_t round_to_power_2_bits(uint16_t x) {
  return (uint16_t)(((uint32_t)x + 32u) & 0xFF80u);
}

__global__ void __launch_bounds__(256)
mxfp4_round_kernel(const uint16_t* __restrict__ x, uint16_t* __restrict__ out, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) out[i] = round_to_power_2_bits(x[i]);
}

// 127 + floor(log2(p)) - 2 clamped to uint8, p the rounded power of two: the biased
// exponent of p minus 2.  p <= 0, infinite or NaN has no logarithm to take; the
// reference's int cast of the NaN / infinity then lands on 0 after the clamp.
__global__ void __launch_bounds__(256)
mxfp4_scales_kernel(const uint16_t* __restrict__ x, uint8_t* __restrict__ out, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const uint16_t p = round_to_power_2_bits(x[i]);
  const uint32_t biased = (p >> 7) & 0xFFu;
  const bool no_log = (p & 0x8000u) || biased == 0xFFu || biased < 2u;
  out[i] = no_log ? (uint8_t)0 : (uint8_t)(biased - 2u);
}

// 2 ** (e - 127) as fp32 (2^-127 is subnormal, 2^128 overflows to infinity), then
// cast to the output dtype
__global__ void __launch_bounds__(256)
mxfp4_convert_kernel(const uint8_t* __restrict__ e, void* __restrict__ out, int out_dtype,
                     int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const uint32_t b = e[i];
  const float v = u2f(b == 0u ? 0x00400000u : (b << 23));
  store_from_f32(out, out_dtype, i, v);
}

static int check_n(int64_t n) {
  CTMI_REQUIRE(n >= 0, CTMI_ERR_VALUE, "negative size");
  CTMI_REQUIRE(cdiv(n, 256) < (1ll << 31), CTMI_ERR_VALUE, "too large");
  return CTMI_OK;
}

}  // namespace ctmi

using namespace ctmi;

extern "C" int ctmi_mxfp4_round_to_power_2(const void* x, void* out, int64_t n, void* stream) {
  int rc = check_n(n);
  if (rc) return rc;
  if (n == 0) return CTMI_OK;
  CTMI_REQUIRE(x && out, CTMI_ERR_VALUE, "NULL tensor pointer");
  hipLaunchKernelGGL(mxfp4_round_kernel, (unsigned)cdiv(n, 256), 256, 0, (hipStream_t)stream,
                     (const uint16_t*)x, (uint16_t*)out, n);
  return check_launch("ctmi_mxfp4_round_to_power_2");
}

extern "C" int ctmi_mxfp4_generate_scales(const void* x, uint8_t* out, int64_t n, void* stream) {
  int rc = check_n(n);
  if (rc) return rc;
  if (n == 0) return CTMI_OK;
  CTMI_REQUIRE(x && out, CTMI_ERR_VALUE, "NULL tensor pointer");
  hipLaunchKernelGGL(mxfp4_scales_kernel, (unsigned)cdiv(n, 256), 256, 0, (hipStream_t)stream,
                     (const uint16_t*)x, out, n);
  return check_launch("ctmi_mxfp4_generate_scales");
}

extern "C" int ctmi_mxfp4_convert_exp_scale(const uint8_t* exps, void* out, int32_t out_dtype,
                                            int64_t n, void* stream) {
  int rc = check_n(n);
  if (rc) return rc;
  CTMI_REQUIRE(out_dtype == CTMI_F32 || out_dtype == CTMI_F16 || out_dtype == CTMI_BF16,
               CTMI_ERR_UNSUPPORTED, "scales convert to float16/bfloat16/float32");
  if (n == 0) return CTMI_OK;
  CTMI_REQUIRE(exps && out, CTMI_ERR_VALUE, "NULL tensor pointer");
  hipLaunchKernelGGL(mxfp4_convert_kernel, (unsigned)cdiv(n, 256), 256, 0, (hipStream_t)stream,
                     exps, out, out_dtype, n);
  return check_launch("ctmi_mxfp4_convert_exp_scale");
}
