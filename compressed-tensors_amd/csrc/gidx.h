// Shared by the kernels for activation-ordered weights (the group of a column is
// g_idx[column], quantization/lifecycle/forward.py:286-296): a workgroup takes RB
// rows of a tile of 256 x 8 columns; a lane keeps the group indices of its 8
// columns in registers, the RB rows of scales (zero points) are staged in LDS as
// fp32 and gathered per element.
#pragma once

#include "ctmi_device.h"
#include "ctmi_host.h"
#include "quant_core.h"
#include "quant_fast.h"

namespace ctmi {

struct GidxArgs {
  const void* dense;          // pack-quantized: compress input / decompress output
  const int32_t* packed_in;   // pack-quantized decompress
  int32_t* packed_out;        // pack-quantized compress
  const void* in;             // quantize / dequantize: input and output tensors
  void* out;
  const void* scale;
  const int8_t* zp;
  const int32_t* col_group;
  uint32_t rows, vpr, s_cols, tiles;  // vpr: items (8 elements) per row
  float qmin, qmax;
};

constexpr int kGidxThreads = 256;

// One activation-ordered weight of a pack-quantized launch: dense -> packed
// (compress) or packed -> dense, `dense_dtype` the dense side's element type.
struct GidxWeight {
  const void* src;
  void* dst;
  int64_t rows, cols;
  const ctmi_qparams* qp;
  int dense_dtype;
};

// stage RB rows of scales (zero points) as fp32: lds_s[rb * s_cols + j]; with lds_r
// also their reciprocals.  Returns whether a staged scale is outside the range
// where the reciprocal path is exact.
template <typename ST, bool HAS_ZP, int RB, bool ZP_FP8 = false>
__device__ __forceinline__ bool stage_qparams(const GidxArgs& a, uint32_t row0, float* lds_s,
                                              float* lds_z, float* lds_r) {
  const auto* scale = (const typename ST::raw*)a.scale;
  bool wild = false;
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const uint32_t row = min(row0 + rb, a.rows - 1);
    for (uint32_t j = threadIdx.x; j < a.s_cols; j += kGidxThreads) {
      const size_t si = (size_t)row * a.s_cols + j;
      const float sv = ST::to_f32(scale[si]);
      lds_s[rb * a.s_cols + j] = sv;
      if (lds_r) {
        lds_r[rb * a.s_cols + j] = __builtin_amdgcn_rcpf(sv);
        wild |= !scale_is_tame(sv);
      }
      if constexpr (HAS_ZP)
        lds_z[rb * a.s_cols + j] = ZP_FP8 ? f8e4m3_to_f32((uint8_t)a.zp[si]) : (float)a.zp[si];
    }
  }
  return wild;
}

__device__ __forceinline__ void load_groups(const GidxArgs& a, uint32_t cv, uint32_t* g) {
  const Vec<int32_t, 4> lo = ldg<int32_t, 4>(a.col_group + (size_t)cv * 8);
  const Vec<int32_t, 4> hi = ldg<int32_t, 4>(a.col_group + (size_t)cv * 8 + 4);
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    // an index outside the scale row must not leave the staged window
    g[k] = min((uint32_t)max(lo.v[k], 0), a.s_cols - 1);
    g[4 + k] = min((uint32_t)max(hi.v[k], 0), a.s_cols - 1);
  }
}

// quantize + pack 8 elements, every element with its own scale / zero point: the
// reference chain with one IEEE division per element
template <typename XT, typename ST, int BITS, bool HAS_ZP>
__device__ __forceinline__ Vec<int32_t, BITS / 4> quant_pack8_each_exact(
    const Vec<typename XT::raw, 8>& xv, const float* s, const float* z, float qmin, float qmax) {
  constexpr int W = BITS / 4;
  constexpr int PF = 32 / BITS;
  constexpr int OFF = 1 << (BITS - 1);
  constexpr int CT = (XT::id == ST::id) ? XT::id : CTMI_F32;
  Vec<int32_t, W> o;
#pragma unroll
  for (int w = 0; w < W; ++w) {
    uint32_t acc = 0;
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int e = w * PF + i;
      float t = round_ct<CT>(XT::to_f32(xv.v[e]) / s[e]);
      if (HAS_ZP) t = round_ct<CT>(t + z[e]);
      t = rintf(clamp_nan(t, qmin, qmax));
      acc |= ((uint32_t)(f32_to_int(t) + OFF) & ((1u << BITS) - 1u)) << (BITS * i);
    }
    o.v[w] = (int32_t)acc;
  }
  return o;
}

// bf16 input, bf16 scales of ordinary magnitude: products with the staged
// reciprocals (they round to the same bf16 as the quotients), hardware bf16
// conversions, integer rounding and packing by the magic-number addition
template <int BITS, bool HAS_ZP>
__device__ __forceinline__ Vec<int32_t, BITS / 4> quant_pack8_each_bf16(
    const Vec<uint16_t, 8>& xv, const float* r, const float* z, float qmin, float qmax) {
  using PC = PackConst<BITS>;
  constexpr int W = BITS / 4;
  const Vec<uint32_t, 4> xw = __builtin_bit_cast(Vec<uint32_t, 4>, xv);
  uint32_t acc[W];
#pragma unroll
  for (int w = 0; w < W; ++w) acc[w] = 0u - PC::bias();
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int e0 = 2 * j, e1 = 2 * j + 1;
    uint32_t t = pack_bf16x2(bf16_lo(xw.v[j]) * r[e0], bf16_hi(xw.v[j]) * r[e1]);
    if (HAS_ZP) t = pack_bf16x2(bf16_lo(t) + z[e0], bf16_hi(t) + z[e1]);
    const float c0 = __builtin_amdgcn_fmed3f(bf16_lo(t), qmin, qmax) + PC::MAGIC;
    const float c1 = __builtin_amdgcn_fmed3f(bf16_hi(t), qmin, qmax) + PC::MAGIC;
    acc[e0 / PC::PF] += f2u(c0) << (BITS * (e0 % PC::PF));
    acc[e1 / PC::PF] += f2u(c1) << (BITS * (e1 % PC::PF));
  }
  Vec<int32_t, W> o;
#pragma unroll
  for (int w = 0; w < W; ++w) o.v[w] = (int32_t)acc[w];
  return o;
}

// rows per workgroup so that the staged fp32 arrays (scales, for compression their
// reciprocals, zero points) stay within 32 KB
static inline int gidx_rows_per_block(int64_t s_cols, int arrays) {
  const int64_t per_row = s_cols * 4 * arrays;
  for (int rb = 8; rb >= 1; rb >>= 1)
    if (rb * per_row <= 32 * 1024) return rb;
  return 0;
}

}  // namespace ctmi
