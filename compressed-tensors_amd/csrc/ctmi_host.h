// Host-side plumbing shared by the entry points: thread-local error message,
// argument checks that run before any HIP call, launch-error capture.
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "ctmi.h"

namespace ctmi {

int set_error(int code, const char* fmt, ...);

inline int dtype_size(int dtype) {
  switch (dtype) {
    case CTMI_F32: return 4;
    case CTMI_F16: return 2;
    case CTMI_BF16: return 2;
    case CTMI_F8E4M3: return 1;
    case CTMI_I8: return 1;
    case CTMI_I16: return 2;
    case CTMI_I32: return 4;
    case CTMI_I64: return 8;
    case CTMI_U8: return 1;
    case CTMI_BOOL: return 1;
  }
  return 0;
}

inline bool is_float_dtype(int dtype) {
  return dtype == CTMI_F32 || dtype == CTMI_F16 || dtype == CTMI_BF16 || dtype == CTMI_F8E4M3;
}

// torch type promotion restricted to the floating types that occur here.
// fp8 does not take part in promotion (torch raises), callers reject it first.
inline int promote_float(int a, int b) {
  if (a == b) return a;
  return CTMI_F32;  // f32 with anything, or f16 with bf16
}

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return set_error(CTMI_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
  return CTMI_OK;
}

inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Largest 1-D grid we launch; kernels that may exceed it use grid-stride loops.
constexpr int64_t kMaxGrid = 1 << 30;

#define CTMI_REQUIRE(cond, code, ...) \
  do {                                \
    if (!(cond)) return ::ctmi::set_error((code), __VA_ARGS__); \
  } while (0)

// Validated view of ctmi_qparams against an [rows, cols] tensor.
int check_qparams(const ctmi_qparams* qp, int64_t rows, int64_t cols);

// qmin / qmax of calculate_range (quantization/utils/helpers.py:208-234)
int quant_range(int qtype, int num_bits, float* qmin, float* qmax);

}  // namespace ctmi
