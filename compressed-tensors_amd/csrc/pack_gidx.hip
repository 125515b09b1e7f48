// pack-quantized compress / decompress for activation-ordered weights: the group
// of a column is g_idx[column] instead of column / group_size
// (quantization/lifecycle/forward.py:286-296, pack_quantized.py:88-183).
//
// A workgroup takes RB rows of a tile of 256 x 8 columns.  A lane keeps the group
// indices of its 8 columns in registers for all RB rows; the RB rows of scales
// (and zero points) are staged in LDS as fp32 once and gathered from there, so the
// only per-element global traffic is the dense / packed data itself, in 16-byte
// pieces as in the column-ordered kernels.
#include <algorithm>
#include <type_traits>

#include "ctmi_device.h"
#include "ctmi_host.h"
#include "quant_core.h"
#include "quant_fast.h"
#include "gidx.h"
#include "job_table.h"

namespace ctmi {

// Kernel argument of a launch over up to kMaxJobs activation-ordered weights: the
// head find_job_index reads (running totals of workgroups; the second row of
// counts is not used here), then what each weight's workgroups need.
struct GidxTable {
  uint32_t chunk_end[kMaxJobs];
  uint32_t unused[kMaxJobs];
  GidxArgs job[kMaxJobs];
};
static_assert(offsetof(GidxTable, chunk_end) == 0 && offsetof(GidxTable, job) == 64,
              "find_job_index reads the first 16 dwords of the kernel argument");

// unpack + dequantize 8 elements: (q - zp) is an integer of at most 8 bits, exact in
// every float type here, so the reference's chain rounds once, in the product
template <typename ST, int BITS, bool HAS_ZP>
__device__ __forceinline__ Vec<typename ST::raw, 8> unpack_dequant8_each(
    const Vec<int32_t, BITS / 4>& pv, const float* s, const float* z) {
  constexpr int PF = 32 / BITS;
  constexpr int OFF = 1 << (BITS - 1);
  float f[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const uint32_t word = (uint32_t)pv.v[e / PF];
    const int q = (int)((word >> (BITS * (e % PF))) & ((1u << BITS) - 1u)) - OFF;
    float t = (float)q;
    if (HAS_ZP) t -= z[e];
    f[e] = t * s[e];
  }
  return pack8_exact_from_f32<ST>(f);
}

template <typename XT, typename ST, int BITS, bool HAS_ZP, int RB>
__global__ void __launch_bounds__(kGidxThreads) pq_gidx_compress_kernel(GidxTable t) {
  uint32_t blk, unused;
  const GidxArgs a = t.job[find_job_index(blockIdx.x, &blk, &unused)];
  using XR = typename XT::raw;
  constexpr int W = BITS / 4;
  constexpr bool kBf16 = XT::id == CTMI_BF16 && ST::id == CTMI_BF16;
  extern __shared__ float lds[];
  float* lds_s = lds;
  float* lds_r = lds + RB * a.s_cols;
  float* lds_z = lds + 2 * RB * a.s_cols;
  const uint32_t rowblk = blk / a.tiles, tile = blk - rowblk * a.tiles;
  const uint32_t row0 = rowblk * RB;
  const uint32_t cv = tile * kGidxThreads + threadIdx.x;
  const bool lane_ok = cv < a.vpr;
  const uint32_t cvc = lane_ok ? cv : a.vpr - 1;
  const XR* x = (const XR*)a.dense;
  Vec<XR, 8> xv[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const uint32_t row = min(row0 + rb, a.rows - 1);
    xv[rb] = ldg_nt<XR, 8>(x + ((size_t)row * a.vpr + cvc) * 8);
  }
  uint32_t g[8];
  load_groups(a, cvc, g);
  const bool wild = stage_qparams<ST, HAS_ZP, RB>(a, row0, lds_s, lds_z, lds_r);
  const bool fast = kBf16 && !__syncthreads_or(wild);  // the barrier that publishes the staged rows
  if constexpr (!kBf16) __syncthreads();
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    float s[8], z[8];
    const float* from = fast ? lds_r : lds_s;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      s[k] = from[rb * a.s_cols + g[k]];
      z[k] = HAS_ZP ? lds_z[rb * a.s_cols + g[k]] : 0.0f;
    }
    Vec<int32_t, W> w;
    if constexpr (kBf16) {
      if (fast) w = quant_pack8_each_bf16<BITS, HAS_ZP>(xv[rb], s, z, a.qmin, a.qmax);
      else w = quant_pack8_each_exact<XT, ST, BITS, HAS_ZP>(xv[rb], s, z, a.qmin, a.qmax);
    } else {
      w = quant_pack8_each_exact<XT, ST, BITS, HAS_ZP>(xv[rb], s, z, a.qmin, a.qmax);
    }
    const uint32_t row = row0 + rb;
    if (lane_ok && row < a.rows)
      stg_nt<int32_t, W>(a.packed_out + ((size_t)row * a.vpr + cv) * W, w);
  }
}

template <typename ST, int BITS, bool HAS_ZP, int RB>
__global__ void __launch_bounds__(kGidxThreads) pq_gidx_decompress_kernel(GidxTable t) {
  uint32_t blk, unused;
  const GidxArgs a = t.job[find_job_index(blockIdx.x, &blk, &unused)];
  using SR = typename ST::raw;
  constexpr int W = BITS / 4;
  extern __shared__ float lds[];
  float* lds_s = lds;
  float* lds_z = lds + RB * a.s_cols;
  const uint32_t rowblk = blk / a.tiles, tile = blk - rowblk * a.tiles;
  const uint32_t row0 = rowblk * RB;
  const uint32_t cv = tile * kGidxThreads + threadIdx.x;
  const bool lane_ok = cv < a.vpr;
  const uint32_t cvc = lane_ok ? cv : a.vpr - 1;
  Vec<int32_t, W> pv[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const uint32_t row = min(row0 + rb, a.rows - 1);
    pv[rb] = ldg_nt<int32_t, W>(a.packed_in + ((size_t)row * a.vpr + cvc) * W);
  }
  uint32_t g[8];
  load_groups(a, cvc, g);
  stage_qparams<ST, HAS_ZP, RB>(a, row0, lds_s, lds_z, nullptr);
  __syncthreads();
  SR* out = (SR*)a.dense;
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    float s[8], z[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      s[k] = lds_s[rb * a.s_cols + g[k]];
      z[k] = HAS_ZP ? lds_z[rb * a.s_cols + g[k]] : 0.0f;
    }
    const Vec<SR, 8> o = unpack_dequant8_each<ST, BITS, HAS_ZP>(pv[rb], s, z);
    const uint32_t row = row0 + rb;
    if (lane_ok && row < a.rows) stg_nt<SR, 8>(out + ((size_t)row * a.vpr + cv) * 8, o);
  }
}

// One launch for the weights of a table; they share the template instance named by `key`.
struct GidxKey {
  int dense_dtype, scale_dtype, bits, rb;
  bool has_zp;
  bool operator==(const GidxKey& o) const {
    return dense_dtype == o.dense_dtype && scale_dtype == o.scale_dtype && bits == o.bits &&
           rb == o.rb && has_zp == o.has_zp;
  }
};

template <typename XT, typename ST, int BITS, bool HAS_ZP>
static void launch_gidx_compress_rb(const GidxTable& t, int rb, unsigned grid, size_t lds, hipStream_t st) {
#define CTMI_G(RB) hipLaunchKernelGGL((pq_gidx_compress_kernel<XT, ST, BITS, HAS_ZP, RB>), grid, kGidxThreads, lds, st, t)
  if (rb == 8) CTMI_G(8); else if (rb == 4) CTMI_G(4); else if (rb == 2) CTMI_G(2); else CTMI_G(1);
#undef CTMI_G
}

template <typename ST, int BITS, bool HAS_ZP>
static void launch_gidx_decompress_rb(const GidxTable& t, int rb, unsigned grid, size_t lds, hipStream_t st) {
#define CTMI_G(RB) hipLaunchKernelGGL((pq_gidx_decompress_kernel<ST, BITS, HAS_ZP, RB>), grid, kGidxThreads, lds, st, t)
  if (rb == 8) CTMI_G(8); else if (rb == 4) CTMI_G(4); else if (rb == 2) CTMI_G(2); else CTMI_G(1);
#undef CTMI_G
}

template <typename XT, typename ST>
static void launch_gidx_compress_st(const GidxKey& k, const GidxTable& t, unsigned grid, size_t lds,
                                    hipStream_t st) {
  if (k.bits == 4) {
    if (k.has_zp) launch_gidx_compress_rb<XT, ST, 4, true>(t, k.rb, grid, lds, st);
    else launch_gidx_compress_rb<XT, ST, 4, false>(t, k.rb, grid, lds, st);
  } else {
    if (k.has_zp) launch_gidx_compress_rb<XT, ST, 8, true>(t, k.rb, grid, lds, st);
    else launch_gidx_compress_rb<XT, ST, 8, false>(t, k.rb, grid, lds, st);
  }
}

template <typename XT>
static void launch_gidx_compress_xt(const GidxKey& k, const GidxTable& t, unsigned grid, size_t lds,
                                    hipStream_t st) {
  if (k.scale_dtype == CTMI_BF16) launch_gidx_compress_st<XT, BF16>(k, t, grid, lds, st);
  else if (k.scale_dtype == CTMI_F16) launch_gidx_compress_st<XT, F16>(k, t, grid, lds, st);
  else launch_gidx_compress_st<XT, F32>(k, t, grid, lds, st);
}

template <typename ST>
static void launch_gidx_decompress_st(const GidxKey& k, const GidxTable& t, unsigned grid, size_t lds,
                                      hipStream_t st) {
  if (k.bits == 4) {
    if (k.has_zp) launch_gidx_decompress_rb<ST, 4, true>(t, k.rb, grid, lds, st);
    else launch_gidx_decompress_rb<ST, 4, false>(t, k.rb, grid, lds, st);
  } else {
    if (k.has_zp) launch_gidx_decompress_rb<ST, 8, true>(t, k.rb, grid, lds, st);
    else launch_gidx_decompress_rb<ST, 8, false>(t, k.rb, grid, lds, st);
  }
}

// Can the streaming act-order kernels take this weight?  (every row its own scale
// row, 4- or 8-bit codes, columns in multiples of 8, int8 zero points)
bool gidx_geometry(const ctmi_qparams* qp, int64_t rows, int64_t cols, int dense_dtype,
                   const void* dense, const void* packed) {
  if (!qp->col_group || qp->global_scale) return false;
  if (qp->num_bits != 4 && qp->num_bits != 8) return false;
  if (qp->blk_rows != 1 || qp->s_rows != rows) return false;
  if (cols % 8 || rows * (cols / 8) >= (1ll << 31) || rows >= (1ll << 31)) return false;
  if (qp->scale_dtype != CTMI_BF16 && qp->scale_dtype != CTMI_F16 && qp->scale_dtype != CTMI_F32)
    return false;
  if (qp->zero_point && qp->zp_dtype != CTMI_I8) return false;
  if (gidx_rows_per_block(qp->s_cols, 3) == 0) return false;
  if ((uintptr_t)dense % (8 * dtype_size(dense_dtype)) || (uintptr_t)packed % 8 ||
      (uintptr_t)qp->col_group % 16)
    return false;
  const int64_t tiles = cdiv(cols / 8, kGidxThreads);
  return cdiv(rows, 1) * tiles < (1ll << 31);
}

static GidxArgs gidx_args(const ctmi_qparams* qp, int64_t rows, int64_t cols) {
  GidxArgs a;
  a.dense = nullptr;
  a.packed_in = nullptr;
  a.packed_out = nullptr;
  a.in = nullptr;
  a.out = nullptr;
  a.scale = qp->scale;
  a.zp = (const int8_t*)qp->zero_point;
  a.col_group = qp->col_group;
  a.rows = (uint32_t)rows;
  a.vpr = (uint32_t)(cols / 8);
  a.s_cols = (uint32_t)qp->s_cols;
  a.tiles = (uint32_t)cdiv(cols / 8, kGidxThreads);
  quant_range(CTMI_QTYPE_INT, qp->num_bits, &a.qmin, &a.qmax);
  return a;
}

static GidxKey gidx_key(const GidxWeight& w, bool compress) {
  const int arrays = (compress ? 2 : 1) + (w.qp->zero_point ? 1 : 0);
  return GidxKey{w.dense_dtype, w.qp->scale_dtype, w.qp->num_bits,
                 gidx_rows_per_block(w.qp->s_cols, arrays), w.qp->zero_point != nullptr};
}

// Do two weights run in the same template instance (and so may share a launch)?
bool gidx_same_launch(const GidxWeight& a, const GidxWeight& b, bool compress) {
  return gidx_key(a, compress) == gidx_key(b, compress);
}

// Enqueue up to kMaxJobs weights that gidx_geometry accepted and gidx_same_launch
// groups, as one launch.  Weights are cut so that the grid stays below 2^31 workgroups.
void gidx_launch_many(const GidxWeight* w, int n, bool compress, hipStream_t st) {
  const GidxKey key = gidx_key(w[0], compress);
  const int arrays = (compress ? 2 : 1) + (key.has_zp ? 1 : 0);
  GidxTable t;
  auto reset = [&]() {
    for (int k = 0; k < kMaxJobs; ++k) {
      t.chunk_end[k] = 0xFFFFFFFFu;
      t.unused[k] = 0;
      t.job[k] = GidxArgs{};
    }
  };
  int filled = 0;
  uint64_t groups = 0;
  size_t lds = 0;
  auto flush = [&]() {
    if (filled == 0) return;
    if (compress) {
      if (key.dense_dtype == CTMI_BF16) launch_gidx_compress_xt<BF16>(key, t, (unsigned)groups, lds, st);
      else if (key.dense_dtype == CTMI_F16) launch_gidx_compress_xt<F16>(key, t, (unsigned)groups, lds, st);
      else launch_gidx_compress_xt<F32>(key, t, (unsigned)groups, lds, st);
    } else {
      if (key.scale_dtype == CTMI_BF16) launch_gidx_decompress_st<BF16>(key, t, (unsigned)groups, lds, st);
      else if (key.scale_dtype == CTMI_F16) launch_gidx_decompress_st<F16>(key, t, (unsigned)groups, lds, st);
      else launch_gidx_decompress_st<F32>(key, t, (unsigned)groups, lds, st);
    }
    filled = 0;
    groups = 0;
    lds = 0;
    reset();
  };
  reset();
  for (int i = 0; i < n; ++i) {
    GidxArgs a = gidx_args(w[i].qp, w[i].rows, w[i].cols);
    if (compress) {
      a.dense = w[i].src;
      a.packed_out = (int32_t*)w[i].dst;
    } else {
      a.packed_in = (const int32_t*)w[i].src;
      a.dense = w[i].dst;
    }
    const uint64_t mine = (uint64_t)cdiv(w[i].rows, key.rb) * a.tiles;
    if (filled == kMaxJobs || groups + mine >= (1ull << 31)) flush();
    t.job[filled] = a;
    groups += mine;
    t.chunk_end[filled] = (uint32_t)groups;
    lds = std::max(lds, (size_t)key.rb * w[i].qp->s_cols * 4 * arrays);
    ++filled;
  }
  flush();
}

// ------------------------------------------------------------------ g_idx -> group of a column
// The reference sorts the columns by g_idx and cuts the sorted order into runs of
// group_size (forward.py:286-303): the group of column c is position(c) / group_size
// with position(c) = #{c' : (g[c'], c') < (g[c], c)}, the place of c in a stable
// sort.  Counted directly, tiled over (c, c') with integer atomics (the sum does not
// depend on their order); a g_idx that holds a -1 is unset and means column order.
constexpr int kRankTile = 1024;

__global__ void __launch_bounds__(256)
column_rank_zero_kernel(int32_t* __restrict__ rank, int cols) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c < cols) rank[c] = 0;
}

__global__ void __launch_bounds__(256)
column_rank_kernel(const int32_t* __restrict__ g, int32_t* __restrict__ rank, int cols) {
  __shared__ uint64_t key[kRankTile];
  const int c = blockIdx.x * 256 + threadIdx.x;
  const int base = blockIdx.y * kRankTile;
  // (g, column) as one unsigned key that orders like the signed pair: any int32 g
  for (int i = threadIdx.x; i < kRankTile; i += 256) {
    const int c2 = base + i;
    key[i] = c2 < cols ? ((uint64_t)((uint32_t)g[c2] ^ 0x80000000u) << 32) | (uint32_t)c2
                       : ~0ull;
  }
  __syncthreads();
  if (c >= cols) return;
  const uint64_t mine = ((uint64_t)((uint32_t)g[c] ^ 0x80000000u) << 32) | (uint32_t)c;
  int below = 0;
#pragma unroll 8
  for (int i = 0; i < kRankTile; ++i) below += key[i] < mine ? 1 : 0;
  if (below) atomicAdd(rank + c, below);
}

__global__ void __launch_bounds__(1024)
column_group_finish_kernel(const int32_t* __restrict__ g, int32_t* __restrict__ rank_to_group,
                           int cols, int group_size) {
  bool unset = false;
  for (int c = threadIdx.x; c < cols; c += 1024) unset |= g[c] == -1;
  unset = __syncthreads_or(unset);
  for (int c = threadIdx.x; c < cols; c += 1024)
    rank_to_group[c] = (unset ? c : rank_to_group[c]) / group_size;
}

}  // namespace ctmi

extern "C" int ctmi_column_groups(const int32_t* g_idx, int64_t cols, int64_t group_size,
                                  int32_t* col_group, void* stream) {
  using namespace ctmi;
  CTMI_REQUIRE(cols >= 0 && group_size >= 1, CTMI_ERR_VALUE, "bad shape");
  CTMI_REQUIRE(cols < (1 << 16), CTMI_ERR_UNSUPPORTED, "at most 65535 columns");
  if (cols == 0) return CTMI_OK;
  CTMI_REQUIRE(g_idx && col_group, CTMI_ERR_VALUE, "NULL tensor pointer");
  hipStream_t st = (hipStream_t)stream;
  const unsigned col_blocks = (unsigned)cdiv(cols, 256);
  hipLaunchKernelGGL(column_rank_zero_kernel, col_blocks, 256, 0, st, col_group, (int)cols);
  hipLaunchKernelGGL(column_rank_kernel, dim3(col_blocks, (unsigned)cdiv(cols, kRankTile)), 256, 0,
                     st, g_idx, col_group, (int)cols);
  hipLaunchKernelGGL(column_group_finish_kernel, 1, 1024, 0, st, g_idx, col_group, (int)cols,
                     (int)group_size);
  return check_launch("ctmi_column_groups");
}
