// int4/int8 -> int32 packing (pack-quantized format): standalone pack / unpack
// and the fused quantize+pack / unpack+dequantize passes.
//
//   pack_to_int32      compressors/quantized_compressors/pack_quantized.py:186-246
//   unpack_from_int32  pack_quantized.py:249-309
//   compress_weight / decompress_weight  pack_quantized.py:88-183
//
// Layout: element i of a run of pf = 32/num_bits neighbours sits in bits
// [b*i, b*i+b) of the word, stored as (value + 2^(b-1)) mod 256; a ragged tail
// is padded with zero bits.
#include <vector>

#include <cstddef>
#include <cstring>
#include <type_traits>

#include "ctmi_device.h"
#include "ctmi_host.h"
#include "quant_core.h"
#include "quant_fast.h"
#include "vec_geom.h"
#include "job_table.h"
#include "gidx.h"

namespace ctmi {

// ------------------------------------------------------------------ standalone pack / unpack
// packed_dim == 1: one thread per output word.
__global__ void __launch_bounds__(256)
pack_dim1_kernel(const int8_t* __restrict__ in, int32_t* __restrict__ out, int64_t rows,
                 int64_t cols, int64_t pcols, int bits) {
  const int pf = 32 / bits;
  const int offset = 1 << (bits - 1);
  const int64_t total = rows * pcols;
  for (int64_t w = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; w < total;
       w += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = w / pcols, j = w - r * pcols;
    const int8_t* src = in + r * cols + j * pf;
    const int n = (int)((cols - j * pf) < pf ? (cols - j * pf) : pf);
    uint32_t acc = 0;
    for (int i = 0; i < n; ++i) {
      uint32_t u = (uint8_t)(src[i] + offset);
      acc += u << (bits * i);  // the reference sums shifted terms (carries included)
    }
    out[w] = (int32_t)acc;
  }
}

// vectors a lane of the streaming pack / unpack kernels takes, all of them asked for before
// any is used
constexpr int kPackVecs = 4;

// 4- or 8-bit, cols % 16 == 0: 16 input bytes per vector.  The tensor is read and written
// once: streaming loads and stores.
template <int BITS>
__global__ void __launch_bounds__(256)
pack_dim1_vec_kernel(const int8_t* __restrict__ in, int32_t* __restrict__ out, int64_t nvec) {
  constexpr int W = BITS * 16 / 32;  // words produced per 16 inputs
  constexpr int PF = 32 / BITS;
  constexpr int OFF = 1 << (BITS - 1);
  constexpr int U = kPackVecs;
  const int64_t v0 = (int64_t)blockIdx.x * (256 * U) + threadIdx.x;
  Vec<int8_t, 16> a[U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t v = v0 + k * 256;
    a[k] = ldg_nt<int8_t, 16>(in + (v < nvec ? v : nvec - 1) * 16);  // past the end: re-read, not stored
  }
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t v = v0 + k * 256;
    Vec<int32_t, W> o;
#pragma unroll
    for (int w = 0; w < W; ++w) {
      uint32_t acc = 0;
#pragma unroll
      for (int i = 0; i < PF; ++i) acc += (uint32_t)(uint8_t)(a[k].v[w * PF + i] + OFF) << (BITS * i);
      o.v[w] = (int32_t)acc;
    }
    if (v < nvec) stg_nt<int32_t, W>(out + v * W, o);
  }
}

// packed_dim == 0: out[j, c] packs in[j*pf + i, c]; one thread per output word.
__global__ void __launch_bounds__(256)
pack_dim0_kernel(const int8_t* __restrict__ in, int32_t* __restrict__ out, int64_t rows,
                 int64_t cols, int64_t prows, int bits) {
  const int pf = 32 / bits;
  const int offset = 1 << (bits - 1);
  const int64_t total = prows * cols;
  for (int64_t w = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; w < total;
       w += (int64_t)gridDim.x * blockDim.x) {
    const int64_t j = w / cols, c = w - j * cols;
    uint32_t acc = 0;
    for (int i = 0; i < pf; ++i) {
      const int64_t r = j * pf + i;
      if (r < rows) acc += (uint32_t)(uint8_t)(in[r * cols + c] + offset) << (bits * i);
    }
    out[w] = (int32_t)acc;
  }
}

// one thread per output element, either packed dim
__global__ void __launch_bounds__(256)
unpack_kernel(const int32_t* __restrict__ in, int8_t* __restrict__ out, int64_t rows, int64_t cols,
              int bits, int packed_dim) {
  const int pf = 32 / bits;
  const uint32_t mask = (bits == 32) ? 0xffffffffu : ((1u << bits) - 1u);
  const int offset = 1 << (bits - 1);
  const int64_t pcols = packed_dim == 1 ? (cols + pf - 1) / pf : cols;
  const int64_t total = rows * cols;
  for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < total;
       e += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = e / cols, c = e - r * cols;
    uint32_t word;
    int i;
    if (packed_dim == 1) {
      word = (uint32_t)in[r * pcols + c / pf];
      i = (int)(c % pf);
    } else {
      word = (uint32_t)in[(r / pf) * pcols + c];
      i = (int)(r % pf);
    }
    out[e] = (int8_t)((int)((word >> (bits * i)) & mask) - offset);
  }
}

// 4- or 8-bit, packed_dim 1, cols % 16 == 0: 16 output bytes per vector
template <int BITS>
__global__ void __launch_bounds__(256)
unpack_dim1_vec_kernel(const int32_t* __restrict__ in, int8_t* __restrict__ out, int64_t nvec) {
  constexpr int W = BITS * 16 / 32;
  constexpr int PF = 32 / BITS;
  constexpr int OFF = 1 << (BITS - 1);
  constexpr uint32_t MASK = (1u << BITS) - 1u;
  constexpr int U = kPackVecs;
  const int64_t v0 = (int64_t)blockIdx.x * (256 * U) + threadIdx.x;
  Vec<int32_t, W> a[U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t v = v0 + k * 256;
    a[k] = ldg_nt<int32_t, W>(in + (v < nvec ? v : nvec - 1) * W);  // past the end: re-read, not stored
  }
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t v = v0 + k * 256;
    Vec<int8_t, 16> o;
#pragma unroll
    for (int w = 0; w < W; ++w)
#pragma unroll
      for (int i = 0; i < PF; ++i)
        o.v[w * PF + i] = (int8_t)((int)(((uint32_t)a[k].v[w] >> (BITS * i)) & MASK) - OFF);
    if (v < nvec) stg_nt<int8_t, 16>(out + v * 16, o);
  }
}

// ------------------------------------------------------------------ fused, generic
struct FusedArgs {
  const void* x;        // compress: dense input; decompress: packed words
  void* out;            // compress: packed words; decompress: dense output
  const void* scale;
  const void* zp;
  const float* gscale;
  const int32_t* col_group;
  int64_t rows, cols, pcols;
  int64_t s_rows, s_cols, blk_rows, blk_cols;
  int x_dtype, out_dtype, scale_dtype, zp_dtype;
  QuantCfg q;
};

__device__ __forceinline__ void load_qp(const FusedArgs& a, int64_t r, int64_t c, int zq_dtype,
                                        float* s, float* z) {
  const int64_t srow = (r / a.blk_rows) % a.s_rows;
  const int64_t scol = a.col_group ? (int64_t)a.col_group[c] : c / a.blk_cols;
  const int64_t si = srow * a.s_cols + scol;
  float sv = load_f32(a.scale, a.scale_dtype, si);
  if (a.gscale) sv = sv / a.gscale[0];
  *s = sv;
  *z = a.zp ? round_to(load_f32(a.zp, a.zp_dtype, si), zq_dtype) : 0.0f;
}

__global__ void __launch_bounds__(256) pq_compress_generic_kernel(FusedArgs a) {
  const int bits = a.q.num_bits;
  const int pf = 32 / bits;
  const int offset = 1 << (bits - 1);
  const int64_t total = a.rows * a.pcols;
  for (int64_t w = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; w < total;
       w += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = w / a.pcols, j = w - r * a.pcols;
    uint32_t acc = 0;
    for (int i = 0; i < pf; ++i) {
      const int64_t c = j * pf + i;
      if (c >= a.cols) break;
      float s, z;
      load_qp(a, r, c, a.x_dtype, &s, &z);
      float v = quantize_value(load_f32(a.x, a.x_dtype, r * a.cols + c), s, z, a.zp != nullptr, a.q);
      acc += (uint32_t)(uint8_t)((int8_t)f32_to_int(v) + offset) << (bits * i);
    }
    ((int32_t*)a.out)[w] = (int32_t)acc;
  }
}

__global__ void __launch_bounds__(256) pq_decompress_generic_kernel(FusedArgs a) {
  const int bits = a.q.num_bits;
  const int pf = 32 / bits;
  const uint32_t mask = (1u << bits) - 1u;
  const int offset = 1 << (bits - 1);
  const int64_t total = a.rows * a.cols;
  for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < total;
       e += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = e / a.cols, c = e - r * a.cols;
    const uint32_t word = (uint32_t)((const int32_t*)a.x)[r * a.pcols + c / pf];
    const int8_t qv = (int8_t)((int)((word >> (bits * (int)(c % pf))) & mask) - offset);
    float s, z;
    load_qp(a, r, c, a.q.dt, &s, &z);
    float v = dequantize_value((float)qv, s, z, a.zp != nullptr, a.q.dt);
    store_from_f32(a.out, a.out_dtype, e, v);
  }
}

// ------------------------------------------------------------------ fused, vectorised
// Work item = 8 neighbouring elements of one row that share a scale (the scale
// block is a multiple of 8 columns wide): a 16-byte load for 2-byte inputs.
// One workgroup handles one chunk of BLOCK*UNROLL items and exits: launching a
// workgroup per chunk lets the dispatcher sweep HBM front to back, which
// measured 20-30 % faster here than a capped grid with a grid-stride loop.  All
// loads of a chunk are issued before the arithmetic.  Dense data is streamed
// with non-temporal accesses; scales and zero points go through the caches.
//
// One launch covers up to kMaxJobs tensors: a kernel start costs about 3 us
// here (dispatch ramp and drain), as much as streaming a 1024 x 4096 weight,
// so the weights of a state dict are chained into one grid.  The job table
// travels in the kernel arguments; a workgroup finds its tensor by a scan over
// the running chunk counts (uniform, scalar registers).
#ifndef CTMI_PQ_TUNING
#define CTMI_PQ_TUNING 512, 2, 512, 2, 8
#endif
constexpr int kPqTuning[5] = {CTMI_PQ_TUNING};
constexpr int kCompressBlock = kPqTuning[0], kCompressUnroll = kPqTuning[1];
constexpr int kDecompressBlock = kPqTuning[2], kDecompressUnroll = kPqTuning[3];
static_assert(kPqTuning[4] == kMaxJobs, "jobs per launch are fixed by job_table.h");

template <typename XT, typename ST, int BITS, bool HAS_ZP, bool FLAT>
__global__ void __launch_bounds__(kCompressBlock) pq_compress_vec_kernel(const ChainTable t) {
  constexpr int W = BITS / 4;  // output words per item
  constexpr int B = kCompressBlock, U = kCompressUnroll;
  uint32_t chunk, nvec;
  const ChainJob job = find_job(t, blockIdx.x, &chunk, &nvec);
  const auto* __restrict__ x = (const typename XT::raw*)job.src;
  const auto* __restrict__ scale = (const typename ST::raw*)job.scale;
  const int8_t* __restrict__ zp = job.zp;
  int32_t* __restrict__ out = (int32_t*)job.dst;
  const uint32_t v0 = chunk * (B * U) + threadIdx.x;
  // A chunk that lies wholly inside its weight (all but the last one) runs
  // without per-lane bounds checks: straight-line code, every load of the
  // workgroup issued before the first value is looked at.
  const bool full = (chunk + 1) * (uint32_t)(B * U) <= nvec;
  auto body = [&](auto guard) {
    constexpr bool GUARD = decltype(guard)::value;
    Vec<typename XT::raw, 8> xv[U];
    typename ST::raw sraw[U];
    int8_t zraw[U];
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const uint32_t v = v0 + k * B;
      if (!GUARD || v < nvec) {
        xv[k] = ldg_nt<typename XT::raw, 8>(x + (size_t)v * 8);
        const uint32_t si = chain_scale_index<FLAT>(v, job);
        sraw[k] = scale[si];
        if constexpr (HAS_ZP) zraw[k] = zp[si];
      }
    }
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const uint32_t v = v0 + k * B;
      if (!GUARD || v < nvec) {
        const float s = ST::to_f32(sraw[k]), z = HAS_ZP ? (float)zraw[k] : 0.0f;
        stg_nt<int32_t, W>(out + (size_t)v * W,
                           quant_pack8<XT, ST, BITS, HAS_ZP>(xv[k], s, z, t.qmin, t.qmax));
      }
    }
  };
  if (full) body(std::false_type{});
  else body(std::true_type{});
}

template <typename ST, int BITS, bool HAS_ZP, bool FLAT>
__global__ void __launch_bounds__(kDecompressBlock) pq_decompress_vec_kernel(const ChainTable t) {
  constexpr int W = BITS / 4;
  constexpr int B = kDecompressBlock, U = kDecompressUnroll;
  uint32_t chunk, nvec;
  const ChainJob job = find_job(t, blockIdx.x, &chunk, &nvec);
  const int32_t* __restrict__ packed = (const int32_t*)job.src;
  const auto* __restrict__ scale = (const typename ST::raw*)job.scale;
  const int8_t* __restrict__ zp = job.zp;
  auto* __restrict__ out = (typename ST::raw*)job.dst;
  const uint32_t v0 = chunk * (B * U) + threadIdx.x;
  const bool full = (chunk + 1) * (uint32_t)(B * U) <= nvec;  // see pq_compress_vec_kernel
  auto body = [&](auto guard) {
    constexpr bool GUARD = decltype(guard)::value;
    Vec<int32_t, W> pv[U];
    typename ST::raw sraw[U];
    int8_t zraw[U];
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const uint32_t v = v0 + k * B;
      if (!GUARD || v < nvec) {
        pv[k] = ldg<int32_t, W>(packed + (size_t)v * W);
        const uint32_t si = chain_scale_index<FLAT>(v, job);
        sraw[k] = scale[si];
        if constexpr (HAS_ZP) zraw[k] = zp[si];
      }
    }
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const uint32_t v = v0 + k * B;
      if (!GUARD || v < nvec) {
        const float s = ST::to_f32(sraw[k]), z = HAS_ZP ? (float)zraw[k] : 0.0f;
        stg_nt<typename ST::raw, 8>(out + (size_t)v * 8,
                                    unpack_dequant8<ST, BITS, HAS_ZP>(pv[k], s, z));
      }
    }
  };
  if (full) body(std::false_type{});
  else body(std::true_type{});
}

// key of a vectorised job: which template instance runs it
struct VecKey {
  int x_dtype, scale_dtype, bits, has_zp, flat;
  bool operator==(const VecKey& o) const {
    return x_dtype == o.x_dtype && scale_dtype == o.scale_dtype && bits == o.bits &&
           has_zp == o.has_zp && flat == o.flat;
  }
};

template <typename XT, typename ST, bool FLAT>
static void launch_compress_flat(const VecKey& k, const ChainTable& t, unsigned grid,
                                 hipStream_t st) {
  constexpr int B = kCompressBlock;
  if (k.bits == 4) {
    if (k.has_zp) hipLaunchKernelGGL((pq_compress_vec_kernel<XT, ST, 4, true, FLAT>), grid, B, 0, st, t);
    else hipLaunchKernelGGL((pq_compress_vec_kernel<XT, ST, 4, false, FLAT>), grid, B, 0, st, t);
  } else {
    if (k.has_zp) hipLaunchKernelGGL((pq_compress_vec_kernel<XT, ST, 8, true, FLAT>), grid, B, 0, st, t);
    else hipLaunchKernelGGL((pq_compress_vec_kernel<XT, ST, 8, false, FLAT>), grid, B, 0, st, t);
  }
}

template <typename XT, typename ST>
static void launch_compress_table(const VecKey& k, const ChainTable& t, unsigned grid,
                                  hipStream_t st) {
  if (k.flat) launch_compress_flat<XT, ST, true>(k, t, grid, st);
  else launch_compress_flat<XT, ST, false>(k, t, grid, st);
}

static void launch_compress_vec(const VecKey& k, const ChainTable& t, unsigned grid,
                                hipStream_t st) {
#define CTMI_DISPATCH_S(XT)                                                              \
  if (k.scale_dtype == CTMI_BF16) launch_compress_table<XT, BF16>(k, t, grid, st);       \
  else if (k.scale_dtype == CTMI_F16) launch_compress_table<XT, F16>(k, t, grid, st);    \
  else launch_compress_table<XT, F32>(k, t, grid, st);
  if (k.x_dtype == CTMI_BF16) { CTMI_DISPATCH_S(BF16) }
  else if (k.x_dtype == CTMI_F16) { CTMI_DISPATCH_S(F16) }
  else { CTMI_DISPATCH_S(F32) }
#undef CTMI_DISPATCH_S
}

template <typename ST, bool FLAT>
static void launch_decompress_flat(const VecKey& k, const ChainTable& t, unsigned grid,
                                   hipStream_t st) {
  constexpr int B = kDecompressBlock;
  if (k.bits == 4) {
    if (k.has_zp) hipLaunchKernelGGL((pq_decompress_vec_kernel<ST, 4, true, FLAT>), grid, B, 0, st, t);
    else hipLaunchKernelGGL((pq_decompress_vec_kernel<ST, 4, false, FLAT>), grid, B, 0, st, t);
  } else {
    if (k.has_zp) hipLaunchKernelGGL((pq_decompress_vec_kernel<ST, 8, true, FLAT>), grid, B, 0, st, t);
    else hipLaunchKernelGGL((pq_decompress_vec_kernel<ST, 8, false, FLAT>), grid, B, 0, st, t);
  }
}

template <typename ST>
static void launch_decompress_table(const VecKey& k, const ChainTable& t, unsigned grid,
                                    hipStream_t st) {
  if (k.flat) launch_decompress_flat<ST, true>(k, t, grid, st);
  else launch_decompress_flat<ST, false>(k, t, grid, st);
}

static void launch_decompress_vec(const VecKey& k, const ChainTable& t, unsigned grid,
                                  hipStream_t st) {
  if (k.scale_dtype == CTMI_BF16) launch_decompress_table<BF16>(k, t, grid, st);
  else if (k.scale_dtype == CTMI_F16) launch_decompress_table<F16>(k, t, grid, st);
  else launch_decompress_table<F32>(k, t, grid, st);
}

static int fill_fused(FusedArgs* a, const ctmi_qparams* qp, int64_t rows, int64_t cols) {
  a->scale = qp->scale;
  a->zp = qp->zero_point;
  a->gscale = qp->global_scale;
  a->col_group = qp->col_group;
  a->rows = rows;
  a->cols = cols;
  a->pcols = cdiv(cols, 32 / qp->num_bits);
  a->s_rows = qp->s_rows;
  a->s_cols = qp->s_cols;
  a->blk_rows = qp->blk_rows;
  a->blk_cols = qp->blk_cols;
  a->scale_dtype = qp->scale_dtype;
  a->zp_dtype = qp->zp_dtype;
  a->q.qtype = qp->qtype;
  a->q.num_bits = qp->num_bits;
  return quant_range(qp->qtype, qp->num_bits, &a->q.qmin, &a->q.qmax);
}

}  // namespace ctmi

using namespace ctmi;

static int check_bits(int32_t num_bits) {
  CTMI_REQUIRE(num_bits <= 8, CTMI_ERR_VALUE, "Packing is only supported for less than 8 bits");
  CTMI_REQUIRE(num_bits >= 1, CTMI_ERR_VALUE, "num_bits must be at least 1, got %d", num_bits);
  return CTMI_OK;
}

extern "C" int ctmi_pack_to_int32(const int8_t* in, int32_t* out, int64_t rows, int64_t cols,
                                  int32_t num_bits, int32_t packed_dim, void* stream) {
  int rc = check_bits(num_bits);
  if (rc) return rc;
  CTMI_REQUIRE(packed_dim == 0 || packed_dim == 1, CTMI_ERR_VALUE, "packed_dim must be 0 or 1");
  CTMI_REQUIRE(rows >= 0 && cols >= 0, CTMI_ERR_VALUE, "negative shape");
  if (rows == 0 || cols == 0) return CTMI_OK;
  CTMI_REQUIRE(in && out, CTMI_ERR_VALUE, "NULL tensor pointer");
  hipStream_t st = (hipStream_t)stream;
  const int pf = 32 / num_bits;
  if (packed_dim == 1) {
    const bool vec = (num_bits == 4 || num_bits == 8) && cols % 16 == 0 &&
                     ((uintptr_t)in % 16 == 0) && ((uintptr_t)out % 8 == 0);
    if (vec) {
      const int64_t nvec = rows * cols / 16;
      const unsigned grid = (unsigned)cdiv(nvec, 256 * kPackVecs);
      if (num_bits == 4) hipLaunchKernelGGL(pack_dim1_vec_kernel<4>, grid, 256, 0, st, in, out, nvec);
      else hipLaunchKernelGGL(pack_dim1_vec_kernel<8>, grid, 256, 0, st, in, out, nvec);
    } else {
      const int64_t pcols = cdiv(cols, pf);
      hipLaunchKernelGGL(pack_dim1_kernel, grid_for(rows * pcols, 256), 256, 0, st, in, out, rows,
                         cols, pcols, num_bits);
    }
  } else {
    const int64_t prows = cdiv(rows, pf);
    hipLaunchKernelGGL(pack_dim0_kernel, grid_for(prows * cols, 256), 256, 0, st, in, out, rows,
                       cols, prows, num_bits);
  }
  return check_launch("ctmi_pack_to_int32");
}

extern "C" int ctmi_unpack_from_int32(const int32_t* in, int8_t* out, int64_t rows, int64_t cols,
                                      int32_t num_bits, int32_t packed_dim, void* stream) {
  CTMI_REQUIRE(num_bits <= 8, CTMI_ERR_VALUE, "Unpacking is only supported for less than 8 bits");
  CTMI_REQUIRE(num_bits >= 1, CTMI_ERR_VALUE, "num_bits must be at least 1, got %d", num_bits);
  CTMI_REQUIRE(packed_dim == 0 || packed_dim == 1, CTMI_ERR_VALUE, "packed_dim must be 0 or 1");
  CTMI_REQUIRE(rows >= 0 && cols >= 0, CTMI_ERR_VALUE, "negative shape");
  if (rows == 0 || cols == 0) return CTMI_OK;
  CTMI_REQUIRE(in && out, CTMI_ERR_VALUE, "NULL tensor pointer");
  hipStream_t st = (hipStream_t)stream;
  const bool vec = packed_dim == 1 && (num_bits == 4 || num_bits == 8) && cols % 16 == 0 &&
                   ((uintptr_t)out % 16 == 0) && ((uintptr_t)in % 8 == 0);
  if (vec) {
    const int64_t nvec = rows * cols / 16;
    const unsigned grid = (unsigned)cdiv(nvec, 256 * kPackVecs);
    if (num_bits == 4) hipLaunchKernelGGL(unpack_dim1_vec_kernel<4>, grid, 256, 0, st, in, out, nvec);
    else hipLaunchKernelGGL(unpack_dim1_vec_kernel<8>, grid, 256, 0, st, in, out, nvec);
  } else {
    hipLaunchKernelGGL(unpack_kernel, grid_for(rows * cols, 256), 256, 0, st, in, out, rows, cols,
                       num_bits, packed_dim);
  }
  return check_launch("ctmi_unpack_from_int32");
}

namespace ctmi {
bool gidx_geometry(const ctmi_qparams* qp, int64_t rows, int64_t cols, int dense_dtype,
                   const void* dense, const void* packed);
bool gidx_same_launch(const GidxWeight& a, const GidxWeight& b, bool compress);
void gidx_launch_many(const GidxWeight* w, int n, bool compress, hipStream_t st);
}  // namespace ctmi

// ---- pack-quantized compress / decompress: validate (no HIP call), then launch.
// A plan is the validated, classified form of one weight.
struct PqPlan {
  bool empty;   // nothing to launch
  bool vec;     // runs in the vectorised multi-tensor kernel
  bool gidx;    // activation-ordered groups: runs in the streaming g_idx kernel
  ctmi_qparams qp;  // for the g_idx launch
  const void* src;
  void* dst;
  int64_t rows, cols;
  int dense_dtype;
  VecKey key;
  VecJob job;
  FusedArgs generic;
};

static int plan_compress(const void* x, int32_t x_dtype, int32_t* out, int64_t rows, int64_t cols,
                         const ctmi_qparams* qp, PqPlan* p) {
  CTMI_REQUIRE(rows >= 0 && cols >= 0, CTMI_ERR_VALUE, "negative shape");
  CTMI_REQUIRE(x_dtype == CTMI_F32 || x_dtype == CTMI_F16 || x_dtype == CTMI_BF16,
               CTMI_ERR_UNSUPPORTED, "quantize needs a float16/bfloat16/float32 input");
  int rc = check_qparams(qp, rows, cols);
  if (rc) return rc;
  CTMI_REQUIRE(qp->global_scale == nullptr, CTMI_ERR_VALUE,
               "global_scale is not supported for the PackQuantizationCompressor");
  CTMI_REQUIRE(qp->qtype == CTMI_QTYPE_INT, CTMI_ERR_VALUE,
               "Tensor must be quantized to torch.int8 before packing");
  rc = check_bits(qp->num_bits);
  if (rc) return rc;
  p->empty = rows == 0 || cols == 0;
  p->vec = p->gidx = false;
  if (p->empty) return CTMI_OK;
  CTMI_REQUIRE(x && out, CTMI_ERR_VALUE, "NULL tensor pointer");

  const bool zp_ok = qp->zero_point == nullptr || qp->zp_dtype == CTMI_I8;
  const bool aligned = ((uintptr_t)x % (8 * dtype_size(x_dtype)) == 0) && ((uintptr_t)out % 8 == 0);
  p->vec = (qp->num_bits == 4 || qp->num_bits == 8) && zp_ok && aligned &&
           qp->scale_dtype != CTMI_F8E4M3 && vec_geometry(qp, rows, cols, &p->job.g) &&
           cdiv(p->job.g.nvec, kCompressBlock * kCompressUnroll) < (1ll << 30);
  if (p->vec) {
    p->key = VecKey{x_dtype, qp->scale_dtype, qp->num_bits, qp->zero_point != nullptr,
                    flat_geometry(p->job.g)};
    p->job.src = x;
    p->job.dst = out;
    p->job.scale = qp->scale;
    p->job.zp = (const int8_t*)qp->zero_point;
    return CTMI_OK;
  }
  p->gidx = gidx_geometry(qp, rows, cols, x_dtype, x, out);
  if (p->gidx) {
    p->qp = *qp;
    p->src = x;
    p->dst = out;
    p->rows = rows;
    p->cols = cols;
    p->dense_dtype = x_dtype;
    return CTMI_OK;
  }
  FusedArgs& a = p->generic;
  rc = fill_fused(&a, qp, rows, cols);
  if (rc) return rc;
  a.x = x;
  a.out = out;
  a.x_dtype = x_dtype;
  a.out_dtype = CTMI_I32;
  a.q.dt = qp->scale_dtype;
  a.q.ct = promote_float(x_dtype, qp->scale_dtype);
  return CTMI_OK;
}

static int plan_decompress(const int32_t* packed, void* out, int32_t out_dtype, int64_t rows,
                           int64_t cols, const ctmi_qparams* qp, PqPlan* p) {
  CTMI_REQUIRE(rows >= 0 && cols >= 0, CTMI_ERR_VALUE, "negative shape");
  CTMI_REQUIRE(out_dtype == CTMI_F32 || out_dtype == CTMI_F16 || out_dtype == CTMI_BF16,
               CTMI_ERR_UNSUPPORTED, "dequantize output must be float16/bfloat16/float32");
  int rc = check_qparams(qp, rows, cols);
  if (rc) return rc;
  CTMI_REQUIRE(qp->num_bits <= 8, CTMI_ERR_VALUE,
               "Unpacking is only supported for less than 8 bits");
  CTMI_REQUIRE(qp->qtype == CTMI_QTYPE_INT, CTMI_ERR_VALUE, "pack-quantized holds integer codes");
  p->empty = rows == 0 || cols == 0;
  p->vec = p->gidx = false;
  if (p->empty) return CTMI_OK;
  CTMI_REQUIRE(packed && out, CTMI_ERR_VALUE, "NULL tensor pointer");

  const bool zp_ok = qp->zero_point == nullptr || qp->zp_dtype == CTMI_I8;
  const bool aligned =
      ((uintptr_t)out % (8 * dtype_size(out_dtype)) == 0) && ((uintptr_t)packed % 8 == 0);
  p->vec = (qp->num_bits == 4 || qp->num_bits == 8) && zp_ok && aligned &&
           out_dtype == qp->scale_dtype && vec_geometry(qp, rows, cols, &p->job.g) &&
           cdiv(p->job.g.nvec, kDecompressBlock * kDecompressUnroll) < (1ll << 30);
  if (p->vec) {
    p->key = VecKey{out_dtype, qp->scale_dtype, qp->num_bits, qp->zero_point != nullptr,
                    flat_geometry(p->job.g)};
    p->job.src = packed;
    p->job.dst = out;
    p->job.scale = qp->scale;
    p->job.zp = (const int8_t*)qp->zero_point;
    return CTMI_OK;
  }
  p->gidx = out_dtype == qp->scale_dtype && gidx_geometry(qp, rows, cols, out_dtype, out, packed);
  if (p->gidx) {
    p->qp = *qp;
    p->src = packed;
    p->dst = out;
    p->rows = rows;
    p->cols = cols;
    p->dense_dtype = out_dtype;
    return CTMI_OK;
  }
  FusedArgs& a = p->generic;
  rc = fill_fused(&a, qp, rows, cols);
  if (rc) return rc;
  a.x = packed;
  a.out = out;
  a.x_dtype = CTMI_I32;
  a.out_dtype = out_dtype;
  a.q.dt = qp->global_scale ? CTMI_F32 : qp->scale_dtype;
  a.q.ct = a.q.dt;
  return CTMI_OK;
}

// Enqueue validated plans: vectorised ones are chained, kMaxJobs per launch and
// per template instance; the others get a launch of the generic kernel each.
// With `count_only` set nothing is enqueued and the number of launches is stored there.
static int run_plans(PqPlan* plans, int64_t n, bool compress, hipStream_t st, const char* what,
                     int64_t* count_only = nullptr) {
  int64_t launches = 0;
  const int per_block = compress ? kCompressBlock * kCompressUnroll
                                 : kDecompressBlock * kDecompressUnroll;
  std::vector<char> done((size_t)n, 0);
  for (int64_t i = 0; i < n; ++i) {
    if (done[i] || plans[i].empty) continue;
    if (plans[i].gidx) {
      // every remaining activation-ordered weight of the same template instance
      auto weight = [&](int64_t k) {
        const PqPlan& g = plans[k];
        return GidxWeight{g.src, g.dst, g.rows, g.cols, &g.qp, g.dense_dtype};
      };
      GidxWeight w[kMaxJobs];
      int m = 0;
      auto flush_gidx = [&]() {
        if (m == 0) return;
        ++launches;
        if (!count_only) gidx_launch_many(w, m, compress, st);
        m = 0;
      };
      for (int64_t k = i; k < n; ++k) {
        if (done[k] || plans[k].empty || !plans[k].gidx) continue;
        if (k != i && !gidx_same_launch(weight(i), weight(k), compress)) continue;
        if (m == kMaxJobs) flush_gidx();
        w[m++] = weight(k);
        done[k] = 1;
      }
      flush_gidx();
      continue;
    }
    if (!plans[i].vec) {
      const FusedArgs& a = plans[i].generic;
      ++launches;
      if (count_only) {
      } else if (compress)
        hipLaunchKernelGGL(pq_compress_generic_kernel, grid_for(a.rows * a.pcols, 256), 256, 0, st, a);
      else
        hipLaunchKernelGGL(pq_decompress_generic_kernel, grid_for(a.rows * a.cols, 256), 256, 0, st, a);
      done[i] = 1;
      continue;
    }
    // gather every remaining job with the same key, kMaxJobs at a time
    const VecKey key = plans[i].key;
    ChainTable t;
    std::memset(&t, 0, sizeof(t));
    uint64_t chunks = 0;
    auto reset = [&]() {
      t.n = 0;
      chunks = 0;
      for (int k = 0; k < kMaxJobs; ++k) t.chunk_end[k] = 0xFFFFFFFFu;
    };
    reset();
    quant_range(CTMI_QTYPE_INT, key.bits, &t.qmin, &t.qmax);
    auto flush = [&]() {
      if (t.n == 0) return;
      ++launches;
      if (count_only) {
      } else if (compress) launch_compress_vec(key, t, (unsigned)chunks, st);
      else launch_decompress_vec(key, t, (unsigned)chunks, st);
      reset();
    };
    for (int64_t j = i; j < n; ++j) {
      if (done[j] || plans[j].empty || !plans[j].vec || !(plans[j].key == key)) continue;
      const uint64_t c = (uint64_t)cdiv(plans[j].job.g.nvec, per_block);
      if (t.n == kMaxJobs || chunks + c >= (1ull << 31)) flush();
      t.job[t.n] = make_chain_job(plans[j].job);
      t.nvec[t.n] = plans[j].job.g.nvec;
      chunks += c;
      t.chunk_end[t.n] = (uint32_t)chunks;
      ++t.n;
      done[j] = 1;
    }
    flush();
  }
  if (count_only) {
    *count_only = launches;
    return CTMI_OK;
  }
  return check_launch(what);
}

extern "C" int ctmi_pack_quantized_compress(const void* x, int32_t x_dtype, int32_t* out,
                                            int64_t rows, int64_t cols, const ctmi_qparams* qp,
                                            void* stream) {
  PqPlan p;
  int rc = plan_compress(x, x_dtype, out, rows, cols, qp, &p);
  if (rc) return rc;
  return run_plans(&p, 1, true, (hipStream_t)stream, "ctmi_pack_quantized_compress");
}

extern "C" int ctmi_pack_quantized_decompress(const int32_t* packed, void* out, int32_t out_dtype,
                                              int64_t rows, int64_t cols, const ctmi_qparams* qp,
                                              void* stream) {
  PqPlan p;
  int rc = plan_decompress(packed, out, out_dtype, rows, cols, qp, &p);
  if (rc) return rc;
  return run_plans(&p, 1, false, (hipStream_t)stream, "ctmi_pack_quantized_decompress");
}

// ------------------------------------------------------------------ many weights, one call
// The state-dict loops of the compressors hand over every weight of a model at
// once.  Every job is validated before anything is enqueued.
extern "C" int ctmi_pack_quantized_compress_many(const ctmi_weight_job* jobs, int64_t n,
                                                 void* stream) {
  CTMI_REQUIRE(n >= 0 && (jobs || n == 0), CTMI_ERR_VALUE, "bad job list");
  std::vector<PqPlan> plans((size_t)n);
  for (int64_t i = 0; i < n; ++i) {
    const ctmi_weight_job& j = jobs[i];
    int rc = plan_compress(j.src, j.dense_dtype, (int32_t*)j.dst, j.rows, j.cols, &j.qp, &plans[i]);
    if (rc) return rc;
  }
  return run_plans(plans.data(), n, true, (hipStream_t)stream, "ctmi_pack_quantized_compress_many");
}

extern "C" int64_t ctmi_pack_quantized_launches(const ctmi_weight_job* jobs, int64_t n,
                                                int32_t compress) {
  CTMI_REQUIRE(n >= 0 && (jobs || n == 0), CTMI_ERR_VALUE, "bad job list");
  std::vector<PqPlan> plans((size_t)n);
  for (int64_t i = 0; i < n; ++i) {
    const ctmi_weight_job& j = jobs[i];
    int rc = compress ? plan_compress(j.src, j.dense_dtype, (int32_t*)j.dst, j.rows, j.cols, &j.qp, &plans[i])
                      : plan_decompress((const int32_t*)j.src, j.dst, j.dense_dtype, j.rows, j.cols, &j.qp, &plans[i]);
    if (rc) return rc;
  }
  int64_t count = 0;
  run_plans(plans.data(), n, compress != 0, nullptr, "ctmi_pack_quantized_launches", &count);
  return count;
}

extern "C" int ctmi_pack_quantized_decompress_many(const ctmi_weight_job* jobs, int64_t n,
                                                   void* stream) {
  CTMI_REQUIRE(n >= 0 && (jobs || n == 0), CTMI_ERR_VALUE, "bad job list");
  std::vector<PqPlan> plans((size_t)n);
  for (int64_t i = 0; i < n; ++i) {
    const ctmi_weight_job& j = jobs[i];
    int rc = plan_decompress((const int32_t*)j.src, j.dst, j.dense_dtype, j.rows, j.cols, &j.qp,
                             &plans[i]);
    if (rc) return rc;
  }
  return run_plans(plans.data(), n, false, (hipStream_t)stream,
                   "ctmi_pack_quantized_decompress_many");
}
