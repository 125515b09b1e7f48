// Entry points of the block (x) Sylvester transforms (kernels: block_sylvester_impl.h) and the
// kernels for bfloat16 tensors with Sylvester factors of 32, 64 and 128.
#include "block_sylvester_impl.h"

namespace ctmi {

CTMI_BS_ENTRY(bs_wide_bf16) { return bs_wide<false>(tab, inner, ma_t, k, sign_in, sign_out, scale, st); }

bool block_sylvester64_supported(int k, int inner, int io_dtype, bool both_signs) {
  const bool size = inner == 128 ? k <= 224
                                 : (inner == 64 || inner == 32 || inner == 16 || inner == 8 || inner == 4) && k <= 256;
  return (io_dtype == CTMI_BF16 || io_dtype == CTMI_F16) && k >= 1 && size && !both_signs;
}

int block_sylvester64_launch(const FwhtJob* jobs, int n_jobs, int io_dtype, int k, int inner,
                             const uint16_t* ma_t, const float* sign_in, const float* sign_out,
                             float scale, hipStream_t st) {
  CTMI_REQUIRE(block_sylvester64_supported(k, inner, io_dtype, sign_in && sign_out), CTMI_ERR_UNSUPPORTED,
               "bfloat16 or float16 tensors, a Sylvester factor of 4 ... 64 with blocks of up to 256 x 256 or of "
               "128 with blocks of up to 224 x 224, signs on one side");
  CTMI_REQUIRE(n_jobs >= 1 && n_jobs <= kFwhtMaxJobs, CTMI_ERR_VALUE, "1 to %d tensors a launch", kFwhtMaxJobs);
  CTMI_REQUIRE(ma_t && (uintptr_t)sign_in % 16 == 0 && (uintptr_t)sign_out % 16 == 0, CTMI_ERR_VALUE,
               "the block must be given; sign vectors must be 16-byte aligned");
  BsTable tab;
  int64_t total = 0;
  for (int i = 0; i < kFwhtMaxJobs; ++i) {
    const bool live = i < n_jobs;
    tab.x[i] = live ? jobs[i].x : nullptr;
    tab.out[i] = live ? jobs[i].out : nullptr;
    if (live) {
      CTMI_REQUIRE(jobs[i].rows > 0 && jobs[i].x && jobs[i].out, CTMI_ERR_VALUE,
                   "tensor %d: NULL pointer or no runs", i);
      CTMI_REQUIRE((uintptr_t)jobs[i].x % 16 == 0 && (uintptr_t)jobs[i].out % 16 == 0, CTMI_ERR_VALUE,
                   "tensors must be 16-byte aligned");
      // blocks above 224 take two launches, and the second reads the runs again
      CTMI_REQUIRE(k <= 224 || jobs[i].x != jobs[i].out, CTMI_ERR_VALUE,
                   "blocks of more than 224 rows are not transformed in place");
      total += jobs[i].rows;
    }
    tab.end[i] = live ? total : INT64_MAX;
  }
  tab.total = total;
  const bool half = io_dtype == CTMI_F16;
  if (inner >= 32)
    return half ? bs_wide_f16(tab, inner, ma_t, k, sign_in, sign_out, scale, st)
                : bs_wide_bf16(tab, inner, ma_t, k, sign_in, sign_out, scale, st);
  return half ? bs_narrow_f16(tab, inner, ma_t, k, sign_in, sign_out, scale, st)
              : bs_narrow_bf16(tab, inner, ma_t, k, sign_in, sign_out, scale, st);
}

}  // namespace ctmi
