// A plain copy kernel of known size.  Hardware byte counters (FETCH_SIZE,
// WRITE_SIZE) are read for this kernel next to the kernels under study, and the
// ratio "counter / bytes really moved" calibrates them.
#include "ctmi_device.h"
#include "ctmi_host.h"

namespace ctmi {

__global__ void __launch_bounds__(256)
calib_copy_kernel(const u32x4_t* __restrict__ src, u32x4_t* __restrict__ dst, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) dst[i] = src[i];
}

}  // namespace ctmi

extern "C" int ctmi_calib_copy(const void* src, void* dst, int64_t bytes, void* stream) {
  CTMI_REQUIRE(bytes >= 0 && bytes % 16 == 0, CTMI_ERR_VALUE, "size must be a multiple of 16 bytes");
  CTMI_REQUIRE(bytes / 16 / 256 < (1ll << 31), CTMI_ERR_VALUE, "too large");
  if (bytes == 0) return CTMI_OK;
  CTMI_REQUIRE(src && dst, CTMI_ERR_VALUE, "NULL tensor pointer");
  CTMI_REQUIRE((uintptr_t)src % 16 == 0 && (uintptr_t)dst % 16 == 0, CTMI_ERR_VALUE,
               "buffers must be 16-byte aligned");
  const int64_t n = bytes / 16;
  hipLaunchKernelGGL(ctmi::calib_copy_kernel, (unsigned)ctmi::cdiv(n, 256), 256, 0,
                     (hipStream_t)stream, (const ctmi::u32x4_t*)src, (ctmi::u32x4_t*)dst, n);
  return ctmi::check_launch("ctmi_calib_copy");
}
