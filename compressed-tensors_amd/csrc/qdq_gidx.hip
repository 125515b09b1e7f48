// quantize / dequantize / fake-quantize for activation-ordered weights
// (quantization/lifecycle/forward.py:286-353 with a g_idx): the arithmetic of the
// column-ordered kernels (qdq_core.h) with every element's scale and zero point
// gathered from the rows of scales staged in LDS.
#include <type_traits>

#include "ctmi_device.h"
#include "ctmi_host.h"
#include "gidx.h"
#include "qdq_core.h"

namespace ctmi {

template <typename FT, int IN, int OUT, int QK, bool HAS_ZP, int RB>
__global__ void __launch_bounds__(kGidxThreads) qdq_gidx_kernel(GidxArgs a) {
  using FR = typename FT::raw;
  using InR = typename std::conditional<IN == kKindFloat, FR, uint8_t>::type;
  using OutR = typename std::conditional<OUT == kKindFloat, FR, uint8_t>::type;
  extern __shared__ float lds[];
  float* lds_s = lds;
  float* lds_z = lds + RB * a.s_cols;
  const uint32_t rowblk = blockIdx.x / a.tiles, tile = blockIdx.x - rowblk * a.tiles;
  const uint32_t row0 = rowblk * RB;
  const uint32_t cv = tile * kGidxThreads + threadIdx.x;
  const bool lane_ok = cv < a.vpr;
  const uint32_t cvc = lane_ok ? cv : a.vpr - 1;
  const InR* x = (const InR*)a.in;
  OutR* out = (OutR*)a.out;
  Vec<InR, 8> xv[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const uint32_t row = min(row0 + rb, a.rows - 1);
    xv[rb] = ldg_nt<InR, 8>(x + ((size_t)row * a.vpr + cvc) * 8);
  }
  uint32_t g[8];
  load_groups(a, cvc, g);
  stage_qparams<FT, HAS_ZP, RB, QK == 1>(a, row0, lds_s, lds_z, nullptr);
  __syncthreads();
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    float s[8], z[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      s[k] = lds_s[rb * a.s_cols + g[k]];
      z[k] = HAS_ZP ? lds_z[rb * a.s_cols + g[k]] : 0.0f;
    }
    Vec<FR, 8> xf, of;
    Vec<uint8_t, 8> xc, oc;
    if constexpr (IN == kKindFloat) xf = xv[rb]; else xc = xv[rb];
    qdq_vec8_impl<FT, IN, OUT, QK, HAS_ZP, 1>(xf, xc, s, z, a.qmin, a.qmax, &of, &oc);
    const uint32_t row = row0 + rb;
    if (lane_ok && row < a.rows) {
      if constexpr (OUT == kKindFloat) stg_nt<FR, 8>(out + ((size_t)row * a.vpr + cv) * 8, of);
      else stg_nt<uint8_t, 8>(out + ((size_t)row * a.vpr + cv) * 8, oc);
    }
  }
}

template <typename FT, int IN, int OUT, int QK, bool HAS_ZP>
static void launch_qdq_gidx_rb(const GidxArgs& a, int rb, size_t lds, hipStream_t st) {
  const unsigned grid = (unsigned)(cdiv(a.rows, rb) * a.tiles);
#define CTMI_G(RB) hipLaunchKernelGGL((qdq_gidx_kernel<FT, IN, OUT, QK, HAS_ZP, RB>), grid, kGidxThreads, lds, st, a)
  if (rb == 8) CTMI_G(8); else if (rb == 4) CTMI_G(4); else if (rb == 2) CTMI_G(2); else CTMI_G(1);
#undef CTMI_G
}

template <typename FT>
static bool launch_qdq_gidx_ft(const GidxArgs& a, int in_kind, int out_kind, int qk, bool has_zp,
                               int rb, size_t lds, hipStream_t st) {
#define CTMI_QG(IN, OUT, QK)                                                          \
  if (in_kind == IN && out_kind == OUT && qk == QK) {                                 \
    if (has_zp) launch_qdq_gidx_rb<FT, IN, OUT, QK, true>(a, rb, lds, st);            \
    else launch_qdq_gidx_rb<FT, IN, OUT, QK, false>(a, rb, lds, st);                  \
    return true;                                                                      \
  }
  CTMI_QG(kKindFloat, kKindI8, 0)
  CTMI_QG(kKindFloat, kKindF8, 1)
  CTMI_QG(kKindI8, kKindFloat, 0)
  CTMI_QG(kKindF8, kKindFloat, 1)
  CTMI_QG(kKindFloat, kKindFloat, 0)
  CTMI_QG(kKindFloat, kKindFloat, 1)
#undef CTMI_QG
  return false;
}

// Tries the streaming act-order path; false = nothing launched.  Same conditions on
// dtypes as the column-ordered kernels: float tensors whose scales have their dtype,
// int8 / fp8 codes, zero points in the code dtype.
bool qdq_gidx_try(const void* x, int x_dtype, void* out, int out_dtype, int64_t rows, int64_t cols,
                  const ctmi_qparams* qp, int do_q, int do_dq, hipStream_t st) {
  if (!qp->col_group || qp->global_scale) return false;
  const int sd = qp->scale_dtype;
  if (sd != CTMI_BF16 && sd != CTMI_F16 && sd != CTMI_F32) return false;
  int in_kind, out_kind, qk;
  if (!do_q) {
    if (x_dtype == CTMI_I8) qk = 0;
    else if (x_dtype == CTMI_F8E4M3) qk = 1;
    else return false;
  } else if (qp->qtype == CTMI_QTYPE_INT && qp->num_bits <= 8) {
    qk = 0;
  } else if (qp->qtype == CTMI_QTYPE_FLOAT && qp->num_bits == 8) {
    qk = 1;
  } else {
    return false;
  }
  const int code_dtype = qk == 0 ? CTMI_I8 : CTMI_F8E4M3;
  if (do_q && do_dq) {
    if (x_dtype != sd || out_dtype != sd) return false;
    in_kind = out_kind = kKindFloat;
  } else if (do_q) {
    if (x_dtype != sd || out_dtype != code_dtype) return false;
    in_kind = kKindFloat;
    out_kind = qk == 0 ? kKindI8 : kKindF8;
  } else {
    if (x_dtype != code_dtype || out_dtype != sd) return false;
    in_kind = qk == 0 ? kKindI8 : kKindF8;
    out_kind = kKindFloat;
  }
  if (qp->zero_point && qp->zp_dtype != code_dtype) return false;
  if (qp->blk_rows != 1 || qp->s_rows != rows) return false;
  if (cols % 8 || rows * (cols / 8) >= (1ll << 31) || rows >= (1ll << 31)) return false;
  const int arrays = qp->zero_point ? 2 : 1;
  const int rb = gidx_rows_per_block(qp->s_cols, arrays);
  if (rb == 0) return false;
  if ((uintptr_t)x % (8 * dtype_size(x_dtype)) || (uintptr_t)out % (8 * dtype_size(out_dtype)) ||
      (uintptr_t)qp->col_group % 16)
    return false;
  GidxArgs a{};
  a.in = x;
  a.out = out;
  a.scale = qp->scale;
  a.zp = (const int8_t*)qp->zero_point;
  a.col_group = qp->col_group;
  a.rows = (uint32_t)rows;
  a.vpr = (uint32_t)(cols / 8);
  a.s_cols = (uint32_t)qp->s_cols;
  a.tiles = (uint32_t)cdiv(cols / 8, kGidxThreads);
  if (cdiv(rows, rb) * a.tiles >= (1ll << 31)) return false;
  if (quant_range(qp->qtype, qp->num_bits, &a.qmin, &a.qmax)) return false;
  const size_t lds = (size_t)rb * qp->s_cols * 4 * arrays;
  const bool has_zp = qp->zero_point != nullptr;
  if (sd == CTMI_BF16) return launch_qdq_gidx_ft<BF16>(a, in_kind, out_kind, qk, has_zp, rb, lds, st);
  if (sd == CTMI_F16) return launch_qdq_gidx_ft<F16>(a, in_kind, out_kind, qk, has_zp, rb, lds, st);
  return launch_qdq_gidx_ft<F32>(a, in_kind, out_kind, qk, has_zp, rb, lds, st);
}

}  // namespace ctmi
