// Observer, calculate_qparams, quantize and pack_to_int32 in one pass over a weight whose
// groups are not runs of neighbouring lanes: activation-ordered weights (the group of a
// column is its place in the order sorted by g_idx, quantization/lifecycle/forward.py:286-303)
// and column-ordered groups of any size that tiles the row.
//
//   min / max per group                     tests/mock_observer.py:38-113
//   calculate_qparams                       quantization/utils/helpers.py:67-146
//   quantize (with g_idx)                   quantization/lifecycle/forward.py:286-331
//   pack_to_int32                           compressors/quantized_compressors/pack_quantized.py:186-246
//
// A workgroup holds RB whole rows in registers (8 items of 8 elements a lane).  Every
// element goes to its group's cell in LDS with one integer maximum (symmetric: on the bits
// of |x|, which order like the values and put a NaN above everything) or a maximum and a
// minimum on order-preserving keys (asymmetric); after a barrier one thread per (row, group)
// turns the cell into scale and zero point, writes them out and leaves them, with the
// scale's reciprocal, in LDS; after a second barrier the rows are quantized from the
// registers, every element with its group's parameters, and packed.  The weight is read
// once: 2 bytes in and num_bits / 8 out per bf16 element, plus the scales.
#include <type_traits>

#include "ctmi_device.h"
#include "ctmi_host.h"
#include "gidx.h"
#include "qparams.h"

namespace ctmi {

struct ObsTableArgs {
  const void* x;
  int32_t* packed;
  void* scale;
  int8_t* zp;                // optional
  const int32_t* col_group;  // group of every column, or NULL: column / blk_cols
  uint32_t rows, vpr, s_cols, blk_cols, rowblks;
  float qmin, qmax;
};

constexpr int kObsTableThreads = 256;
constexpr int kObsTableItems = 8;  // items a lane holds: NT per row times RB rows

__device__ __forceinline__ uint32_t order_key(float f) {
  const uint32_t b = __float_as_uint(f);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ __forceinline__ float order_value(uint32_t k) {
  return __uint_as_float((k & 0x80000000u) ? (k ^ 0x80000000u) : ~k);
}

template <typename XT, int BITS, bool SYM, int NT>
__global__ void __launch_bounds__(kObsTableThreads) observe_pack_table_kernel(ObsTableArgs a) {
  using XR = typename XT::raw;
  constexpr int RB = kObsTableItems / NT;
  constexpr int W = BITS / 4;
  constexpr bool kBf16 = XT::id == CTMI_BF16;
  extern __shared__ uint32_t lds[];
  const uint32_t S = a.s_cols, cells = RB * S, tid = threadIdx.x;
  uint32_t* m_hi = lds;               // symmetric: bits of max |x|; else key of the maximum
  uint32_t* m_lo = lds + cells;       // key of the minimum
  uint32_t* m_nan = lds + 2 * cells;  // the cell holds a NaN
  float* lds_s = reinterpret_cast<float*>(lds + 3 * cells);
  float* lds_r = lds_s + cells;
  float* lds_z = lds_r + cells;

  // the groups of this lane's columns, a byte each (s_cols <= 256), for every row it will see
  uint32_t gid[NT][2], cvc[NT];
  bool ok[NT];
#pragma unroll
  for (int k = 0; k < NT; ++k) {
    const uint32_t cv = k * kObsTableThreads + tid;
    ok[k] = cv < a.vpr;
    cvc[k] = ok[k] ? cv : a.vpr - 1;
    uint32_t g[8];
    if (a.col_group) {
      const Vec<int32_t, 4> lo = ldg<int32_t, 4>(a.col_group + (size_t)cvc[k] * 8);
      const Vec<int32_t, 4> hi = ldg<int32_t, 4>(a.col_group + (size_t)cvc[k] * 8 + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {  // an index outside the scale row must not leave the cells
        g[e] = min((uint32_t)max(lo.v[e], 0), S - 1);
        g[4 + e] = min((uint32_t)max(hi.v[e], 0), S - 1);
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) g[e] = (cvc[k] * 8 + e) / a.blk_cols;
    }
    gid[k][0] = g[0] | (g[1] << 8) | (g[2] << 16) | (g[3] << 24);
    gid[k][1] = g[4] | (g[5] << 8) | (g[6] << 16) | (g[7] << 24);
  }
  for (uint32_t i = tid; i < cells; i += kObsTableThreads) {
    m_hi[i] = 0u;
    if constexpr (!SYM) {
      m_lo[i] = 0xFFFFFFFFu;
      m_nan[i] = 0u;
    }
  }
  __syncthreads();

  const XR* __restrict__ x = static_cast<const XR*>(a.x);
  XR* __restrict__ scale = static_cast<XR*>(a.scale);
  for (uint32_t rowblk = blockIdx.x; rowblk < a.rowblks; rowblk += gridDim.x) {
    const uint32_t row0 = rowblk * RB;
    Vec<XR, 8> xv[RB][NT];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const uint32_t row = min(row0 + rb, a.rows - 1);  // past the end: the last row again, not stored
#pragma unroll
      for (int k = 0; k < NT; ++k) xv[rb][k] = ldg_nt<XR, 8>(x + ((size_t)row * a.vpr + cvc[k]) * 8);
    }
    // ---- observer: every element into its group's cell
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int k = 0; k < NT; ++k) {
        if (!ok[k]) continue;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const uint32_t cell = rb * S + ((gid[k][e >> 2] >> (8 * (e & 3))) & 0xffu);
          const float f = XT::to_f32(xv[rb][k].v[e]);
          if constexpr (SYM) {
            atomicMax(&m_hi[cell], __float_as_uint(fabsf(f)));
          } else {
            if (f != f) {
              atomicOr(&m_nan[cell], 1u);
            } else {
              const uint32_t key = order_key(f);
              atomicMax(&m_hi[cell], key);
              atomicMin(&m_lo[cell], key);
            }
          }
        }
      }
    __syncthreads();
    // ---- calculate_qparams, one thread per (row, group); the cell goes back to its start value
    bool wild = false;
    for (uint32_t i = tid; i < cells; i += kObsTableThreads) {
      const uint32_t rb = i / S, g = i - rb * S, row = row0 + rb;
      float sv, zv = 0.0f;
      if constexpr (SYM) {
        const uint32_t m = m_hi[i];
        sv = symmetric_scale<XT>(__uint_as_float(m), m > 0x7F800000u, (a.qmax - a.qmin) * 0.5f);
        m_hi[i] = 0u;
      } else {
        asymmetric_qparams<XT, 0>(order_value(m_lo[i]), order_value(m_hi[i]), m_nan[i] != 0u, a.qmin,
                                  a.qmax, &sv, &zv);
        m_hi[i] = 0u;
        m_lo[i] = 0xFFFFFFFFu;
        m_nan[i] = 0u;
      }
      if (row < a.rows) {
        scale[(size_t)row * S + g] = XT::from_f32(sv);
        if (a.zp) a.zp[(size_t)row * S + g] = SYM ? (int8_t)0 : (int8_t)f32_to_int(zv);
      }
      lds_s[i] = sv;
      lds_r[i] = __builtin_amdgcn_rcpf(sv);
      lds_z[i] = zv;
      wild |= !scale_is_tame(sv);
    }
    // the barrier that publishes the parameters; bf16 with scales of ordinary magnitude
    // takes the products with the reciprocals (they round to the same bf16 as the quotients)
    const bool fast = kBf16 && !__syncthreads_or(wild);
    if constexpr (!kBf16) __syncthreads();
    // ---- quantize + pack from the registers
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int k = 0; k < NT; ++k) {
        float s[8], z[8];
        const float* from = fast ? lds_r : lds_s;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const uint32_t cell = rb * S + ((gid[k][e >> 2] >> (8 * (e & 3))) & 0xffu);
          s[e] = from[cell];
          z[e] = SYM ? 0.0f : lds_z[cell];
        }
        Vec<int32_t, W> w;
        if constexpr (kBf16) {
          if (fast) w = quant_pack8_each_bf16<BITS, !SYM>(xv[rb][k], s, z, a.qmin, a.qmax);
          else w = quant_pack8_each_exact<XT, XT, BITS, !SYM>(xv[rb][k], s, z, a.qmin, a.qmax);
        } else {
          w = quant_pack8_each_exact<XT, XT, BITS, !SYM>(xv[rb][k], s, z, a.qmin, a.qmax);
        }
        const uint32_t row = row0 + rb;
        if (ok[k] && row < a.rows)
          stg_nt<int32_t, W>(a.packed + ((size_t)row * a.vpr + k * kObsTableThreads + tid) * W, w);
      }
    // no barrier here: the next round's cells were reset before the barrier above, and its
    // parameters are written only after its own first barrier, which every lane reaches
    // after it has read this round's
  }
}

static bool obs_table_supported(int x_dtype, int64_t rows, int64_t cols, int64_t blk_cols, int num_bits) {
  if (x_dtype != CTMI_BF16 && x_dtype != CTMI_F16 && x_dtype != CTMI_F32) return false;
  if (num_bits != 4 && num_bits != 8) return false;
  if (rows < 1 || cols < 1 || blk_cols < 1 || rows >= (1ll << 31)) return false;
  if (cols % 8 || cols % blk_cols) return false;
  if (cols / 8 > kObsTableThreads * kObsTableItems) return false;  // a row fits a workgroup's registers
  if (cols / blk_cols > 256) return false;                         // a group index fits a byte
  return rows * (cols / 8) < (1ll << 31);
}

template <typename XT, int BITS, bool SYM>
static void launch_obs_table_nt(const ObsTableArgs& a, int nt, unsigned grid, size_t lds, hipStream_t st) {
#define CTMI_OT(NT)                                                                                   \
  hipLaunchKernelGGL((observe_pack_table_kernel<XT, BITS, SYM, NT>), grid, kObsTableThreads, lds, st, a)
  if (nt == 1) CTMI_OT(1); else if (nt == 2) CTMI_OT(2); else if (nt == 4) CTMI_OT(4); else CTMI_OT(8);
#undef CTMI_OT
}

template <typename XT>
static void launch_obs_table_xt(const ObsTableArgs& a, int bits, bool sym, int nt, unsigned grid,
                                size_t lds, hipStream_t st) {
  if (bits == 4) {
    if (sym) launch_obs_table_nt<XT, 4, true>(a, nt, grid, lds, st);
    else launch_obs_table_nt<XT, 4, false>(a, nt, grid, lds, st);
  } else {
    if (sym) launch_obs_table_nt<XT, 8, true>(a, nt, grid, lds, st);
    else launch_obs_table_nt<XT, 8, false>(a, nt, grid, lds, st);
  }
}

}  // namespace ctmi

using namespace ctmi;

extern "C" int ctmi_observe_pack_quantized_gidx_supported(int32_t x_dtype, int64_t rows, int64_t cols,
                                                          int64_t blk_cols, int32_t num_bits) {
  return obs_table_supported(x_dtype, rows, cols, blk_cols, num_bits) ? 1 : 0;
}

extern "C" int ctmi_observe_pack_quantized_gidx(const void* x, int32_t x_dtype, int64_t rows,
                                                int64_t cols, int64_t blk_cols, int32_t num_bits,
                                                int32_t symmetric, const int32_t* col_group,
                                                int32_t* packed, void* scale, int8_t* zero_point,
                                                void* stream) {
  CTMI_REQUIRE(rows >= 1 && cols >= 1, CTMI_ERR_VALUE, "cannot observe an empty tensor");
  CTMI_REQUIRE(blk_cols >= 1, CTMI_ERR_VALUE, "empty cell");
  ObsTableArgs a;
  int rc = quant_range(CTMI_QTYPE_INT, num_bits, &a.qmin, &a.qmax);
  if (rc) return rc;
  CTMI_REQUIRE(x_dtype == CTMI_F32 || x_dtype == CTMI_F16 || x_dtype == CTMI_BF16, CTMI_ERR_UNSUPPORTED,
               "weights must be float16/bfloat16/float32");
  CTMI_REQUIRE(x && packed && scale, CTMI_ERR_VALUE, "NULL tensor pointer");
  CTMI_REQUIRE(obs_table_supported(x_dtype, rows, cols, blk_cols, num_bits), CTMI_ERR_UNSUPPORTED,
               "no fused kernel for this layout (rows of up to 16384 elements in multiples of 8, up to "
               "256 groups a row): run the observer and the compressor separately");
  CTMI_REQUIRE((uintptr_t)x % (8 * dtype_size(x_dtype)) == 0 && (uintptr_t)packed % (4 * (num_bits / 4)) == 0 &&
                   (uintptr_t)scale % dtype_size(x_dtype) == 0 && (uintptr_t)col_group % 16 == 0,
               CTMI_ERR_VALUE, "tensors must be aligned to 8 elements");
  a.x = x;
  a.packed = packed;
  a.scale = scale;
  a.zp = zero_point;
  a.col_group = col_group;
  a.rows = (uint32_t)rows;
  a.vpr = (uint32_t)(cols / 8);
  a.s_cols = (uint32_t)(cols / blk_cols);
  a.blk_cols = (uint32_t)blk_cols;
  int nt = 1;
  while (nt * kObsTableThreads < (int)a.vpr) nt *= 2;
  const int rb = kObsTableItems / nt;
  a.rowblks = (uint32_t)cdiv(rows, rb);
  // every workgroup takes the same number of row blocks (one more or less): the groups of its
  // columns are looked up once
  const int64_t rounds = cdiv((int64_t)a.rowblks, 2048);
  const unsigned grid = (unsigned)cdiv((int64_t)a.rowblks, rounds);
  const size_t lds = (size_t)rb * a.s_cols * 6 * sizeof(uint32_t);
  hipStream_t st = (hipStream_t)stream;
  const bool sym = symmetric != 0;
  if (x_dtype == CTMI_BF16) launch_obs_table_xt<BF16>(a, num_bits, sym, nt, grid, lds, st);
  else if (x_dtype == CTMI_F16) launch_obs_table_xt<F16>(a, num_bits, sym, nt, grid, lds, st);
  else launch_obs_table_xt<F32>(a, num_bits, sym, nt, grid, lds, st);
  return check_launch("ctmi_observe_pack_quantized_gidx");
}
