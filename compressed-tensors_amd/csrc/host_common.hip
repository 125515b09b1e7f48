// Error reporting, argument validation and small host helpers of libctmi.so.
#include <string.h>

#include "ctmi_host.h"

namespace ctmi {

static thread_local char g_err[512] = "";

int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int quant_range(int qtype, int num_bits, float* qmin, float* qmax) {
  if (qtype == CTMI_QTYPE_INT) {
    CTMI_REQUIRE(num_bits >= 1 && num_bits <= 24, CTMI_ERR_VALUE,
                 "integer quantization supports 1..24 bits, got %d", num_bits);
    double half = (double)(1ll << num_bits) / 2.0;
    *qmin = (float)(-half);
    *qmax = (float)(half - 1.0);
    return CTMI_OK;
  }
  if (qtype == CTMI_QTYPE_FLOAT) {
    if (num_bits == 8) {
      *qmin = -448.0f;
      *qmax = 448.0f;
      return CTMI_OK;
    }
    if (num_bits == 4) {
      *qmin = -6.0f;
      *qmax = 6.0f;
      return CTMI_OK;
    }
    return set_error(CTMI_ERR_UNSUPPORTED, "Range calculation only supported for 4 and 8 bits");
  }
  return set_error(CTMI_ERR_VALUE, "Invalid quantization type %d", qtype);
}

int check_qparams(const ctmi_qparams* qp, int64_t rows, int64_t cols) {
  CTMI_REQUIRE(qp != nullptr, CTMI_ERR_VALUE, "qparams is NULL");
  CTMI_REQUIRE(qp->scale != nullptr, CTMI_ERR_VALUE, "scale is NULL");
  CTMI_REQUIRE(qp->scale_dtype == CTMI_F32 || qp->scale_dtype == CTMI_F16 ||
                   qp->scale_dtype == CTMI_BF16 || qp->scale_dtype == CTMI_F8E4M3,
               CTMI_ERR_UNSUPPORTED, "unsupported scale dtype %d", qp->scale_dtype);
  CTMI_REQUIRE(qp->scale_dtype != CTMI_F8E4M3 || qp->global_scale != nullptr, CTMI_ERR_UNSUPPORTED,
               "float8 scales need a global_scale (no float8 arithmetic exists otherwise)");
  CTMI_REQUIRE(qp->s_rows >= 1 && qp->s_cols >= 1, CTMI_ERR_VALUE, "empty scale grid");
  CTMI_REQUIRE(qp->blk_rows >= 1 && qp->blk_cols >= 1, CTMI_ERR_VALUE, "empty scale block");
  if (qp->zero_point != nullptr) {
    CTMI_REQUIRE(dtype_size(qp->zp_dtype) > 0 && qp->zp_dtype != CTMI_I64, CTMI_ERR_UNSUPPORTED,
                 "unsupported zero point dtype %d", qp->zp_dtype);
  }
  if (qp->col_group == nullptr && cols > 0) {
    CTMI_REQUIRE(cdiv(cols, qp->blk_cols) <= qp->s_cols, CTMI_ERR_VALUE,
                 "scale grid has %lld columns, tensor needs %lld", (long long)qp->s_cols,
                 (long long)cdiv(cols, qp->blk_cols));
  }
  (void)rows;
  float lo, hi;
  return quant_range(qp->qtype, qp->num_bits, &lo, &hi);
}

}  // namespace ctmi

extern "C" const char* ctmi_last_error(void) { return ctmi::g_err; }
extern "C" int ctmi_version(void) { return 1; }
