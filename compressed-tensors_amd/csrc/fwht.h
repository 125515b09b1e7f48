// Sylvester-Hadamard transforms of long runs (1024 ... 8192 elements) by butterflies in
// registers (fwht.hip), optionally with the W4A16 group-128 quantization in the same pass.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "qparams.h"

namespace ctmi {

constexpr int kFwhtMaxJobs = 8;

struct FwhtJob {
  const void* x;
  void* out;        // the rotated tensor (fused: optional)
  int32_t* packed;  // fused rotation + quantization: int32 [rows * n / 8]
  void* scale;      // fused: bf16 [rows * n / 128]
  int64_t rows;     // runs of n elements
};

inline bool fwht_size_supported(int64_t n) { return n == 1024 || n == 2048 || n == 4096 || n == 8192; }

// y = x * diag(sign_in) * Sylvester(n) * diag(sign_out) * (w0 ? *w0 : 1) * scale for every run
// of n elements of up to kFwhtMaxJobs tensors (16-byte aligned, as are the sign vectors).
// quant != NULL (bfloat16 only): y is rounded to bfloat16 and quantized in groups of 128 as
// symmetric integers of quant->num_bits = 4 bits, packed eight to an int32; job.out may then
// be NULL.  Returns a CTMI_* code; the launch is not checked.
int fwht_launch(const FwhtJob* jobs, int n_jobs, int io_dtype, int n, const float* sign_in,
                const float* sign_out, const float* w0, float scale, const QpCfg* quant,
                hipStream_t st);

// y = x * diag(sign_in) * (Ma (x) Sylvester(inner)) * diag(sign_out) * scale, inner = 4 ... 128,
// for every run of k * inner bfloat16 or float16 elements (block_sylvester.hip): ma_t = Ma^T,
// [k, k] bfloat16 with entries exact in bfloat16 (and, for float16 tensors, in float16), k up to
// 256 (224 for inner = 128; above 224 not in place); signs on at most one side.  job.packed /
// job.scale are not used.
bool block_sylvester64_supported(int k, int inner, int io_dtype, bool both_signs);
int block_sylvester64_launch(const FwhtJob* jobs, int n_jobs, int io_dtype, int k, int inner,
                             const uint16_t* ma_t, const float* sign_in, const float* sign_out,
                             float scale, hipStream_t st);

}  // namespace ctmi
