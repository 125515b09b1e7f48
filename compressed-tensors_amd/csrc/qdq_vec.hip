// Vectorised quantize / dequantize / fake-quantize for the common layouts:
// input, scale and (for the float side) output share one float dtype, scales
// cover runs of at least 8 columns (per tensor, channel, token or group), codes
// are int8 or float8_e4m3fn.  Same arithmetic as the generic kernel in
// quant.hip (forward.py:455-514), 8 elements per lane, 16-byte accesses, one
// workgroup per chunk, streaming hints on the dense data.
//
// bf16 tensors quantize with a reciprocal multiply (same bits as the division,
// see quant_fast.h); fp8 codes use the hardware converters
// (v_cvt_pk_fp8_f32 / v_cvt_f32_fp8: OCP e4m3, round-to-nearest-even), which the
// GPU tests compare with torch's cast on every bf16 bit pattern.
#include <type_traits>

#include "ctmi_device.h"
#include "ctmi_host.h"
#include "quant_core.h"
#include "quant_fast.h"
#include "qdq_core.h"
#include "vec_geom.h"
#include "job_table.h"

namespace ctmi {

constexpr int kQdqBlock = 512, kQdqUnroll = 2;

// FT: float dtype tag of x / scale / float output.  IN / OUT: element kind of the
// input and output tensors.  QK: 0 = integer grid, 1 = fp8 grid.
// One chunk (kQdqBlock * kQdqUnroll items) of one tensor; `index_of` maps an item
// to its scale.
template <typename FT, int IN, int OUT, int QK, bool HAS_ZP, typename IndexOf>
__device__ __forceinline__ void qdq_chunk(const void* __restrict__ xin,
                                          const typename FT::raw* __restrict__ scale,
                                          const uint8_t* __restrict__ zp, void* __restrict__ yout,
                                          uint32_t nvec, uint32_t chunk, IndexOf index_of,
                                          float qmin, float qmax) {
  constexpr int CT = FT::id;
  constexpr int B = kQdqBlock, U = kQdqUnroll;
  constexpr bool DO_Q = IN == kKindFloat;
  constexpr bool DO_DQ = OUT == kKindFloat;
  using FR = typename FT::raw;
  const uint32_t v0 = chunk * (B * U) + threadIdx.x;
  // A chunk wholly inside the tensor (all but the last) runs without per-lane
  // bounds checks: straight-line code, every load of the workgroup issued before
  // the first loaded value is looked at.
  const bool full = (chunk + 1) * (uint32_t)(B * U) <= nvec;
  auto body = [&](auto guard) {
    constexpr bool GUARD = decltype(guard)::value;
    Vec<FR, 8> xf[U];
    Vec<uint8_t, 8> xc[U];
    FR sraw[U];
    uint8_t zraw[U];
    uint32_t si[U];
#pragma unroll
    for (int k = 0; k < U; ++k) si[k] = index_of(min(v0 + k * B, nvec - 1));
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const uint32_t v = v0 + k * B;
      if (!GUARD || v < nvec) {
        if constexpr (DO_Q) xf[k] = ldg_nt<FR, 8>((const FR*)xin + (size_t)v * 8);
        else xc[k] = ldg_nt<uint8_t, 8>((const uint8_t*)xin + (size_t)v * 8);
        sraw[k] = scale[si[k]];
        if constexpr (HAS_ZP) zraw[k] = zp[si[k]];
      }
    }
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const uint32_t v = v0 + k * B;
      if (GUARD && v >= nvec) continue;
      const float s = FT::to_f32(sraw[k]);
      float z = 0.0f;
      if constexpr (HAS_ZP) z = QK == 0 ? (float)(int8_t)zraw[k] : f8e4m3_to_f32(zraw[k]);
      Vec<FR, 8> of;
      Vec<uint8_t, 8> oc;
      qdq_vec8<FT, IN, OUT, QK, HAS_ZP>(xf[k], xc[k], s, z, qmin, qmax, &of, &oc);
      if constexpr (DO_DQ) stg_nt<FR, 8>((FR*)yout + (size_t)v * 8, of);
      else stg_nt<uint8_t, 8>((uint8_t*)yout + (size_t)v * 8, oc);
    }
  };
  if (full) body(std::false_type{});
  else body(std::true_type{});
}

template <typename FT, int IN, int OUT, int QK, bool HAS_ZP>
__global__ void __launch_bounds__(kQdqBlock)
qdq_vec_kernel(const void* __restrict__ xin, const typename FT::raw* __restrict__ scale,
               const uint8_t* __restrict__ zp, void* __restrict__ yout, VecGeom g, float qmin,
               float qmax) {
  qdq_chunk<FT, IN, OUT, QK, HAS_ZP>(xin, scale, zp, yout, g.nvec, blockIdx.x,
                                     [&](uint32_t v) { return scale_index(v, g); }, qmin, qmax);
}

// several tensors per launch (job_table.h); the table must be the only argument
template <typename FT, int IN, int OUT, int QK, bool HAS_ZP, bool FLAT>
__global__ void __launch_bounds__(kQdqBlock) qdq_vec_many_kernel(const ChainTable t) {
  uint32_t chunk, nvec;
  const ChainJob job = find_job(t, blockIdx.x, &chunk, &nvec);
  qdq_chunk<FT, IN, OUT, QK, HAS_ZP>(job.src, (const typename FT::raw*)job.scale,
                                     (const uint8_t*)job.zp, job.dst, nvec, chunk,
                                     [&](uint32_t v) { return chain_scale_index<FLAT>(v, job); },
                                     t.qmin, t.qmax);
}

template <typename FT, int IN, int OUT, int QK>
static void launch_qdq(bool has_zp, const void* x, const void* scale, const void* zp, void* out,
                       const VecGeom& g, float qmin, float qmax, hipStream_t st) {
  const unsigned grid = (unsigned)cdiv(g.nvec, kQdqBlock * kQdqUnroll);
  using FR = typename FT::raw;
  if (has_zp)
    hipLaunchKernelGGL((qdq_vec_kernel<FT, IN, OUT, QK, true>), grid, kQdqBlock, 0, st, x,
                       (const FR*)scale, (const uint8_t*)zp, out, g, qmin, qmax);
  else
    hipLaunchKernelGGL((qdq_vec_kernel<FT, IN, OUT, QK, false>), grid, kQdqBlock, 0, st, x,
                       (const FR*)scale, (const uint8_t*)zp, out, g, qmin, qmax);
}

template <typename FT>
static void dispatch_mode(int in_kind, int out_kind, int qk, bool has_zp, const void* x,
                          const void* scale, const void* zp, void* out, const VecGeom& g,
                          float qmin, float qmax, hipStream_t st) {
#define CTMI_QDQ(IN, OUT, QK)                              \
  if (in_kind == IN && out_kind == OUT && qk == QK) {      \
    launch_qdq<FT, IN, OUT, QK>(has_zp, x, scale, zp, out, g, qmin, qmax, st); \
    return;                                                \
  }
  CTMI_QDQ(kKindFloat, kKindI8, 0)
  CTMI_QDQ(kKindFloat, kKindF8, 1)
  CTMI_QDQ(kKindI8, kKindFloat, 0)
  CTMI_QDQ(kKindF8, kKindFloat, 1)
  CTMI_QDQ(kKindFloat, kKindFloat, 0)
  CTMI_QDQ(kKindFloat, kKindFloat, 1)
#undef CTMI_QDQ
}

// Which instance of the vectorised kernels takes this problem, if any.
struct QdqKey {
  int sd, in_kind, out_kind, qk, has_zp, flat;
  bool operator==(const QdqKey& o) const {
    return sd == o.sd && in_kind == o.in_kind && out_kind == o.out_kind && qk == o.qk &&
           has_zp == o.has_zp && flat == o.flat;
  }
};

// All arguments have been validated by the caller.  false = does not fit.
bool qdq_classify(const void* x, int x_dtype, const void* out, int out_dtype, int64_t rows,
                  int64_t cols, const ctmi_qparams* qp, int do_q, int do_dq, QdqKey* key,
                  VecGeom* g, float* qmin, float* qmax) {
  const int sd = qp->scale_dtype;
  if (sd != CTMI_BF16 && sd != CTMI_F16 && sd != CTMI_F32) return false;
  int in_kind, out_kind, qk;
  if (!do_q) {
    // dequantize only looks at the stored codes, whatever grid produced them
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
  if (!vec_geometry(qp, rows, cols, g)) return false;
  if (cdiv(g->nvec, kQdqBlock * kQdqUnroll) >= (1ll << 30)) return false;
  const int in_bytes = 8 * dtype_size(x_dtype), out_bytes = 8 * dtype_size(out_dtype);
  if ((uintptr_t)x % in_bytes || (uintptr_t)out % out_bytes) return false;
  if (quant_range(qp->qtype, qp->num_bits, qmin, qmax)) return false;
  *key = QdqKey{sd, in_kind, out_kind, qk, qp->zero_point != nullptr, g->mode == 0};
  return true;
}

// Tries the vectorised path; returns false (nothing launched) if the problem
// does not fit it.
bool qdq_try_vectorised(const void* x, int x_dtype, void* out, int out_dtype, int64_t rows,
                        int64_t cols, const ctmi_qparams* qp, int do_q, int do_dq,
                        hipStream_t st) {
  QdqKey k;
  VecGeom g;
  float qmin, qmax;
  if (!qdq_classify(x, x_dtype, out, out_dtype, rows, cols, qp, do_q, do_dq, &k, &g, &qmin, &qmax))
    return false;
  if (k.sd == CTMI_BF16)
    dispatch_mode<BF16>(k.in_kind, k.out_kind, k.qk, k.has_zp, x, qp->scale, qp->zero_point, out, g, qmin, qmax, st);
  else if (k.sd == CTMI_F16)
    dispatch_mode<F16>(k.in_kind, k.out_kind, k.qk, k.has_zp, x, qp->scale, qp->zero_point, out, g, qmin, qmax, st);
  else
    dispatch_mode<F32>(k.in_kind, k.out_kind, k.qk, k.has_zp, x, qp->scale, qp->zero_point, out, g, qmin, qmax, st);
  return true;
}

// ---- chained launches
template <typename FT, int IN, int OUT, int QK>
static void launch_many2(const QdqKey& k, const ChainTable& t, unsigned grid, hipStream_t st) {
#define CTMI_QM(ZP, FLAT) \
  hipLaunchKernelGGL((qdq_vec_many_kernel<FT, IN, OUT, QK, ZP, FLAT>), grid, kQdqBlock, 0, st, t)
  if (k.has_zp) { if (k.flat) CTMI_QM(true, true); else CTMI_QM(true, false); }
  else { if (k.flat) CTMI_QM(false, true); else CTMI_QM(false, false); }
#undef CTMI_QM
}

template <typename FT>
static void launch_many1(const QdqKey& k, const ChainTable& t, unsigned grid, hipStream_t st) {
#define CTMI_QDQ(IN, OUT, QK)                                        \
  if (k.in_kind == IN && k.out_kind == OUT && k.qk == QK) {          \
    launch_many2<FT, IN, OUT, QK>(k, t, grid, st);                   \
    return;                                                          \
  }
  CTMI_QDQ(kKindFloat, kKindI8, 0)
  CTMI_QDQ(kKindFloat, kKindF8, 1)
  CTMI_QDQ(kKindI8, kKindFloat, 0)
  CTMI_QDQ(kKindF8, kKindFloat, 1)
  CTMI_QDQ(kKindFloat, kKindFloat, 0)
  CTMI_QDQ(kKindFloat, kKindFloat, 1)
#undef CTMI_QDQ
}

void qdq_launch_chain(const QdqKey& k, const ChainTable& t, unsigned grid, hipStream_t st) {
  if (k.sd == CTMI_BF16) launch_many1<BF16>(k, t, grid, st);
  else if (k.sd == CTMI_F16) launch_many1<F16>(k, t, grid, st);
  else launch_many1<F32>(k, t, grid, st);
}

int qdq_chunk_items() { return kQdqBlock * kQdqUnroll; }

}  // namespace ctmi
