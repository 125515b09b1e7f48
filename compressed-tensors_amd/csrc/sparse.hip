// Bitmask sparsity formats.
//
//   pack_bitmasks / unpack_bitmasks     utils/helpers.py:302-339
//   bitmask_compress / decompress       compressors/sparse_compressors/sparse_bitmask.py:131-169
//   get_24_bytemasks                    compressors/sparse_compressors/sparse_24_bitmask.py:227-260
//   sparse24_bitmask_compress / decompress   sparse_24_bitmask.py:162-224
//
// Bit j of bitmask byte k of a row flags column 8k+j (numpy packbits,
// bitorder="little"); the last byte of a row is zero padded.  Compacted values
// are stored in row-major order of the set bits.
#include "ctmi_device.h"
#include "ctmi_host.h"
#include "topk24_lut.h"
#include "vec_geom.h"

namespace ctmi {

static const uint8_t kTopk24LutHost[4096] = CTMI_TOPK24_LUT_INIT;
__constant__ uint8_t kTopk24LutDev[4096] = CTMI_TOPK24_LUT_INIT;

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / kWave;

// ------------------------------------------------------------------ block scan
__device__ __forceinline__ int wave_inclusive_scan(int v) {
  const int lane = lane_id();
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int t = __shfl_up(v, d, kWave);
    if (lane >= d) v += t;
  }
  return v;
}

// exclusive prefix of `cnt` over the workgroup and the workgroup total
__device__ __forceinline__ void block_exclusive_scan(int cnt, int* pre, int* total, int* smem) {
  const int inc = wave_inclusive_scan(cnt);
  const int wave = threadIdx.x / kWave;
  if (lane_id() == kWave - 1) smem[wave] = inc;
  __syncthreads();
  int woff = 0, tot = 0;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) {
    const int s = smem[w];
    if (w < wave) woff += s;
    tot += s;
  }
  *pre = woff + inc - cnt;
  *total = tot;
  __syncthreads();
}

__device__ __forceinline__ int64_t block_sum(int64_t v, int64_t* smem) {
#pragma unroll
  for (int d = kWave / 2; d > 0; d >>= 1) v += __shfl_xor(v, d, kWave);
  if (lane_id() == 0) smem[threadIdx.x / kWave] = v;
  __syncthreads();
  int64_t t = 0;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) t += smem[w];
  __syncthreads();
  return t;
}

// ------------------------------------------------------------------ pack / unpack bitmasks
__global__ void __launch_bounds__(kBlock)
pack_bitmasks_kernel(const uint8_t* __restrict__ mask, uint8_t* __restrict__ packed, int64_t rows,
                     int64_t cols, int64_t pc) {
  const int64_t total = rows * pc;
  const bool vec = (cols % 8 == 0) && ((uintptr_t)mask % 8 == 0);
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / pc, b = i - r * pc;
    uint32_t bits = 0;
    if (vec) {
      const uint64_t w = *reinterpret_cast<const uint64_t*>(mask + r * cols + b * 8);
#pragma unroll
      for (int j = 0; j < 8; ++j) bits |= (uint32_t)(((w >> (8 * j)) & 0xffu) != 0) << j;
    } else {
      for (int j = 0; j < 8; ++j) {
        const int64_t c = b * 8 + j;
        if (c < cols) bits |= (uint32_t)(mask[r * cols + c] != 0) << j;
      }
    }
    packed[i] = (uint8_t)bits;
  }
}

__global__ void __launch_bounds__(kBlock)
unpack_bitmasks_kernel(const uint8_t* __restrict__ packed, uint8_t* __restrict__ mask, int64_t rows,
                       int64_t cols, int64_t pc) {
  const int64_t total = rows * pc;
  const bool vec = (cols % 8 == 0) && ((uintptr_t)mask % 8 == 0);
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / pc, b = i - r * pc;
    const uint32_t bits = packed[i];
    if (vec) {
      uint64_t w = 0;
#pragma unroll
      for (int j = 0; j < 8; ++j) w |= (uint64_t)((bits >> j) & 1u) << (8 * j);
      *reinterpret_cast<uint64_t*>(mask + r * cols + b * 8) = w;
    } else {
      for (int j = 0; j < 8; ++j) {
        const int64_t c = b * 8 + j;
        if (c < cols) mask[r * cols + c] = (uint8_t)((bits >> j) & 1u);
      }
    }
  }
}

// ------------------------------------------------------------------ sparse-bitmask: mask + counts
// One workgroup per row.  Thread t of an iteration owns 8 neighbouring
// columns = one bitmask byte.  nz_mask strips the sign bit of floating types
// so that -0.0 counts as zero while NaN stays non-zero.
template <typename R>
__global__ void __launch_bounds__(kBlock)
bitmask_count_kernel(const R* __restrict__ x, uint32_t nz_mask, uint8_t* __restrict__ bitmask,
                     int64_t* __restrict__ counts, int64_t rows, int64_t cols, int64_t pc) {
  __shared__ int64_t red[kWaves];
  const bool vec = (cols % 8 == 0) && ((uintptr_t)x % (8 * sizeof(R)) == 0);
  for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
    const R* row = x + r * cols;
    int64_t cnt = 0;
    for (int64_t b = threadIdx.x; b < pc; b += kBlock) {
      uint32_t bits = 0;
      if (vec) {
        Vec<R, 8> a = ldg<R, 8>(row + b * 8);
#pragma unroll
        for (int j = 0; j < 8; ++j) bits |= (uint32_t)(((uint32_t)a.v[j] & nz_mask) != 0) << j;
      } else {
        for (int j = 0; j < 8; ++j) {
          const int64_t c = b * 8 + j;
          if (c < cols) bits |= (uint32_t)(((uint32_t)row[c] & nz_mask) != 0) << j;
        }
      }
      bitmask[r * pc + b] = (uint8_t)bits;
      cnt += __popc(bits);
    }
    const int64_t t = block_sum(cnt, red);
    if (threadIdx.x == 0) counts[r] = t;
  }
}

// per-row popcount of an existing bitmask (bits at columns >= cols ignored)
__global__ void __launch_bounds__(kBlock)
bitmask_popcount_kernel(const uint8_t* __restrict__ bitmask, int64_t* __restrict__ counts,
                        int64_t rows, int64_t cols, int64_t pc) {
  __shared__ int64_t red[kWaves];
  const uint32_t tail = (cols % 8) ? ((1u << (cols % 8)) - 1u) : 0xffu;
  for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
    int64_t cnt = 0;
    for (int64_t b = threadIdx.x; b < pc; b += kBlock) {
      uint32_t bits = bitmask[r * pc + b];
      if (b == pc - 1) bits &= tail;
      cnt += __popc(bits);
    }
    const int64_t t = block_sum(cnt, red);
    if (threadIdx.x == 0) counts[r] = t;
  }
}

// exclusive scan of counts[rows] -> offsets[rows], total; single workgroup
__global__ void __launch_bounds__(1024)
row_offsets_kernel(const int64_t* __restrict__ counts, int64_t* __restrict__ offsets,
                   int64_t* __restrict__ total, int64_t rows) {
  __shared__ int64_t wsum[16];
  __shared__ int64_t carry_s;
  if (threadIdx.x == 0) carry_s = 0;
  __syncthreads();
  const int lane = lane_id(), wave = threadIdx.x / kWave;
  for (int64_t base = 0; base < rows; base += 1024) {
    const int64_t i = base + threadIdx.x;
    const int64_t c = i < rows ? counts[i] : 0;
    int64_t inc = c;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const int64_t t = __shfl_up(inc, d, kWave);
      if (lane >= d) inc += t;
    }
    if (lane == kWave - 1) wsum[wave] = inc;
    __syncthreads();
    int64_t woff = 0, tot = 0;
    for (int w = 0; w < 16; ++w) {
      const int64_t s = wsum[w];
      if (w < wave) woff += s;
      tot += s;
    }
    const int64_t carry = carry_s;
    if (i < rows) offsets[i] = carry + woff + inc - c;
    __syncthreads();
    if (threadIdx.x == 0) carry_s = carry + tot;
    __syncthreads();
  }
  if (threadIdx.x == 0 && total) *total = carry_s;
}

// ------------------------------------------------------------------ sparse-bitmask: compaction
// One workgroup per row, 2048 columns per iteration.  Survivors are first
// gathered into LDS at their rank within the iteration, then the contiguous
// run is written to HBM by the whole workgroup, so global stores are dense
// regardless of where the non-zeros sit.
template <typename R>
__global__ void __launch_bounds__(kBlock)
bitmask_compact_kernel(const R* __restrict__ x, const uint8_t* __restrict__ bitmask,
                       const int64_t* __restrict__ row_offsets, R* __restrict__ values,
                       int64_t rows, int64_t cols, int64_t pc) {
  __shared__ int scan_s[kWaves];
  __shared__ R stage[kBlock * 8];
  const bool vec = (cols % 8 == 0) && ((uintptr_t)x % (8 * sizeof(R)) == 0);
  const uint32_t tail = (cols % 8) ? ((1u << (cols % 8)) - 1u) : 0xffu;
  for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
    const R* row = x + r * cols;
    R* dst = values + row_offsets[r];
    for (int64_t b0 = 0; b0 < pc; b0 += kBlock) {
      const int64_t b = b0 + threadIdx.x;
      uint32_t bits = 0;
      Vec<R, 8> a;
      if (b < pc) {
        bits = bitmask[r * pc + b];
        if (b == pc - 1) bits &= tail;
        if (vec) {
          a = ldg<R, 8>(row + b * 8);
        } else {
          for (int j = 0; j < 8; ++j) {
            const int64_t c = b * 8 + j;
            a.v[j] = c < cols ? row[c] : (R)0;
          }
        }
      }
      int pre, total;
      block_exclusive_scan(__popc(bits), &pre, &total, scan_s);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if ((bits >> j) & 1u) stage[pre++] = a.v[j];
      }
      __syncthreads();
      for (int i = threadIdx.x; i < total; i += kBlock) dst[i] = stage[i];
      dst += total;
      __syncthreads();
    }
  }
}

// ------------------------------------------------------------------ bitmask decompress (scatter)
template <typename R>
__global__ void __launch_bounds__(kBlock)
bitmask_scatter_kernel(const R* __restrict__ values, int64_t nvalues,
                       const uint8_t* __restrict__ bitmask,
                       const int64_t* __restrict__ row_offsets, R* __restrict__ out, int64_t rows,
                       int64_t cols, int64_t pc) {
  __shared__ int scan_s[kWaves];
  __shared__ R stage[kBlock * 8];
  const bool vec = (cols % 8 == 0) && ((uintptr_t)out % (8 * sizeof(R)) == 0);
  const uint32_t tail = (cols % 8) ? ((1u << (cols % 8)) - 1u) : 0xffu;
  for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
    R* row = out + r * cols;
    int64_t src = row_offsets[r];
    for (int64_t b0 = 0; b0 < pc; b0 += kBlock) {
      const int64_t b = b0 + threadIdx.x;
      uint32_t bits = 0;
      if (b < pc) {
        bits = bitmask[r * pc + b];
        if (b == pc - 1) bits &= tail;
      }
      int pre, total;
      block_exclusive_scan(__popc(bits), &pre, &total, scan_s);
      // a bitmask with more set bits than there are values reads zeros, never past the end
      for (int i = threadIdx.x; i < total; i += kBlock)
        stage[i] = (src + i < nvalues) ? values[src + i] : (R)0;
      src += total;
      __syncthreads();
      if (b < pc) {
        Vec<R, 8> o;
#pragma unroll
        for (int j = 0; j < 8; ++j) o.v[j] = ((bits >> j) & 1u) ? stage[pre++] : (R)0;
        if (vec) {
          stg<R, 8>(row + b * 8, o);
        } else {
          for (int j = 0; j < 8; ++j) {
            const int64_t c = b * 8 + j;
            if (c < cols) row[c] = o.v[j];
          }
        }
      }
      __syncthreads();
    }
  }
}

// ------------------------------------------------------------------ 2:4 selection
// Ranking key of one element: |value| compared the way torch.topk compares
// it (NaN above everything, all NaNs equal); for 1-byte integer views abs() is
// evaluated in int8, so -128 stays -128 and ranks lowest.
template <int DT>
__device__ __forceinline__ uint32_t key24(uint32_t raw) {
  if constexpr (DT == CTMI_BF16) {
    const uint32_t m = raw & 0x7FFFu;
    return m > 0x7F80u ? 0xFFFFFFFFu : m;
  } else if constexpr (DT == CTMI_F16) {
    const uint32_t m = raw & 0x7FFFu;
    return m > 0x7C00u ? 0xFFFFFFFFu : m;
  } else if constexpr (DT == CTMI_F32) {
    const uint32_t m = raw & 0x7FFFFFFFu;
    return m > 0x7F800000u ? 0xFFFFFFFFu : m;
  } else {  // int8 view (int8 and float8 tensors)
    const int v = (int)(int8_t)raw;
    const int a = (v == -128) ? -128 : (v < 0 ? -v : v);
    return (uint32_t)(a + 128);
  }
}

__device__ __forceinline__ uint32_t cmp3(uint32_t a, uint32_t b) {
  return a > b ? 2u : (a == b ? 1u : 0u);
}

// 4-bit keep mask of one group, looked up by the six pairwise comparisons
__device__ __forceinline__ uint32_t keep24(uint32_t k0, uint32_t k1, uint32_t k2, uint32_t k3,
                                           const uint8_t* lut) {
  const uint32_t idx = cmp3(k0, k1) | (cmp3(k0, k2) << 2) | (cmp3(k0, k3) << 4) |
                       (cmp3(k1, k2) << 6) | (cmp3(k1, k3) << 8) | (cmp3(k2, k3) << 10);
  return lut[idx];
}

__device__ __forceinline__ void load_lut(uint8_t* lds_lut) {
  // 4096 bytes, 16 per thread of a 256-thread workgroup
  reinterpret_cast<uint4*>(lds_lut)[threadIdx.x] =
      reinterpret_cast<const uint4*>(kTopk24LutDev)[threadIdx.x];
  __syncthreads();
}

template <typename R, int DT>
__global__ void __launch_bounds__(kBlock)
bytemask24_kernel(const R* __restrict__ x, uint8_t* __restrict__ mask, int64_t ngroups) {
  __shared__ __align__(16) uint8_t lut[4096];
  load_lut(lut);
  for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < ngroups;
       g += (int64_t)gridDim.x * blockDim.x) {
    const R* p = x + g * 4;
    const uint32_t keep = keep24(key24<DT>(p[0]), key24<DT>(p[1]), key24<DT>(p[2]),
                                 key24<DT>(p[3]), lut);
    uint32_t w = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) w |= ((keep >> j) & 1u) << (8 * j);
    *reinterpret_cast<uint32_t*>(mask + g * 4) = w;
  }
}

// Fused 2:4 compress, cols % 8 == 0.  Work item = N elements (N/4 groups):
// one 16-byte load, N/2 survivors stored as one vector, N/8 bitmask bytes.
template <typename R, int DT, int N>
__global__ void __launch_bounds__(kBlock)
sparse24_compress_kernel(const R* __restrict__ x, R* __restrict__ values,
                         uint8_t* __restrict__ bitmask, int64_t nitems) {
  __shared__ __align__(16) uint8_t lut[4096];
  load_lut(lut);
  for (int64_t it = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; it < nitems;
       it += (int64_t)gridDim.x * blockDim.x) {
    Vec<R, N> a = ldg<R, N>(x + it * N);
    Vec<R, N / 2> o;
    Vec<uint8_t, N / 8> m;
#pragma unroll
    for (int q = 0; q < N / 4; ++q) {
      const uint32_t keep = keep24(key24<DT>(a.v[4 * q]), key24<DT>(a.v[4 * q + 1]),
                                   key24<DT>(a.v[4 * q + 2]), key24<DT>(a.v[4 * q + 3]), lut);
      // the two survivors in column order
      const int lo = __ffs(keep) - 1;
      const int hi = 31 - __clz(keep);
      o.v[2 * q] = a.v[4 * q + lo];
      o.v[2 * q + 1] = a.v[4 * q + hi];
      if (q & 1) m.v[q / 2] |= (uint8_t)(keep << 4);
      else m.v[q / 2] = (uint8_t)keep;
    }
    stg<R, N / 2>(values + it * (N / 2), o);
    stg<uint8_t, N / 8>(bitmask + it * (N / 8), m);
  }
}

// Any shape with numel % 4 == 0 (groups may straddle rows): survivors per group.
template <typename R, int DT>
__global__ void __launch_bounds__(kBlock)
sparse24_values_kernel(const R* __restrict__ x, R* __restrict__ values, int64_t ngroups) {
  __shared__ __align__(16) uint8_t lut[4096];
  load_lut(lut);
  for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < ngroups;
       g += (int64_t)gridDim.x * blockDim.x) {
    const R* p = x + g * 4;
    const uint32_t keep = keep24(key24<DT>(p[0]), key24<DT>(p[1]), key24<DT>(p[2]),
                                 key24<DT>(p[3]), lut);
    values[2 * g] = p[__ffs(keep) - 1];
    values[2 * g + 1] = p[31 - __clz(keep)];
  }
}

// ... and the row-structured bitmask for that case: one thread per bitmask byte
template <typename R, int DT>
__global__ void __launch_bounds__(kBlock)
sparse24_bitmask_kernel(const R* __restrict__ x, uint8_t* __restrict__ bitmask, int64_t rows,
                        int64_t cols, int64_t pc) {
  __shared__ __align__(16) uint8_t lut[4096];
  load_lut(lut);
  const int64_t total = rows * pc;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / pc, b = i - r * pc;
    uint32_t bits = 0;
    for (int j = 0; j < 8; ++j) {
      const int64_t c = b * 8 + j;
      if (c >= cols) break;
      const int64_t e = r * cols + c;
      const R* p = x + (e / 4) * 4;
      const uint32_t keep = keep24(key24<DT>(p[0]), key24<DT>(p[1]), key24<DT>(p[2]),
                                   key24<DT>(p[3]), lut);
      bits |= ((keep >> (e % 4)) & 1u) << j;
    }
    bitmask[i] = (uint8_t)bits;
  }
}

__global__ void __launch_bounds__(kBlock) zero_i64_kernel(int64_t* p, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x)
    p[i] = 0;
}

static int rows_grid(int64_t rows) {
  const int64_t cap = 256 * 32;
  return (int)(rows < cap ? (rows < 1 ? 1 : rows) : cap);
}

}  // namespace ctmi

using namespace ctmi;

extern "C" void ctmi_topk24_lut(uint8_t* out4096) {
  for (int i = 0; i < 4096; ++i) out4096[i] = kTopk24LutHost[i];
}

extern "C" int ctmi_pack_bitmasks(const uint8_t* mask, uint8_t* packed, int64_t rows, int64_t cols,
                                  void* stream) {
  CTMI_REQUIRE(rows >= 0 && cols >= 0, CTMI_ERR_VALUE, "negative shape");
  if (rows == 0 || cols == 0) return CTMI_OK;
  CTMI_REQUIRE(mask && packed, CTMI_ERR_VALUE, "NULL tensor pointer");
  const int64_t pc = cdiv(cols, 8);
  hipLaunchKernelGGL(pack_bitmasks_kernel, grid_for(rows * pc, kBlock), kBlock, 0,
                     (hipStream_t)stream, mask, packed, rows, cols, pc);
  return check_launch("ctmi_pack_bitmasks");
}

extern "C" int ctmi_unpack_bitmasks(const uint8_t* packed, uint8_t* mask, int64_t rows,
                                    int64_t cols, void* stream) {
  CTMI_REQUIRE(rows >= 0 && cols >= 0, CTMI_ERR_VALUE, "negative shape");
  if (rows == 0 || cols == 0) return CTMI_OK;
  CTMI_REQUIRE(mask && packed, CTMI_ERR_VALUE, "NULL tensor pointer");
  const int64_t pc = cdiv(cols, 8);
  hipLaunchKernelGGL(unpack_bitmasks_kernel, grid_for(rows * pc, kBlock), kBlock, 0,
                     (hipStream_t)stream, packed, mask, rows, cols, pc);
  return check_launch("ctmi_unpack_bitmasks");
}

extern "C" int64_t ctmi_bitmask_tmp_bytes(int64_t rows) { return (rows < 1 ? 1 : rows) * 8; }

static int check_elem(int32_t elem_size) {
  CTMI_REQUIRE(elem_size == 1 || elem_size == 2 || elem_size == 4, CTMI_ERR_UNSUPPORTED,
               "element size must be 1, 2 or 4 bytes, got %d", elem_size);
  return CTMI_OK;
}

extern "C" int ctmi_bitmask_count(const void* x, int32_t elem_size, int32_t is_float,
                                  uint8_t* bitmask, int64_t* row_offsets, int64_t* total_nnz,
                                  void* tmp, int64_t rows, int64_t cols, void* stream) {
  CTMI_REQUIRE(rows >= 0 && cols >= 0, CTMI_ERR_VALUE, "negative shape");
  int rc = check_elem(elem_size);
  if (rc) return rc;
  CTMI_REQUIRE(total_nnz != nullptr, CTMI_ERR_VALUE, "total_nnz is NULL");
  hipStream_t st = (hipStream_t)stream;
  if (rows == 0 || cols == 0) {
    CTMI_REQUIRE(rows == 0 || row_offsets, CTMI_ERR_VALUE, "NULL tensor pointer");
    if (rows > 0)
      hipLaunchKernelGGL(zero_i64_kernel, grid_for(rows, kBlock), kBlock, 0, st, row_offsets, rows);
    hipLaunchKernelGGL(zero_i64_kernel, 1, kBlock, 0, st, total_nnz, (int64_t)1);
    return check_launch("ctmi_bitmask_count");
  }
  CTMI_REQUIRE(x && bitmask && row_offsets && tmp, CTMI_ERR_VALUE, "NULL tensor pointer");
  const int64_t pc = cdiv(cols, 8);
  int64_t* counts = (int64_t*)tmp;
  const int grid = rows_grid(rows);
  if (elem_size == 1) {
    hipLaunchKernelGGL(bitmask_count_kernel<uint8_t>, grid, kBlock, 0, st, (const uint8_t*)x,
                       is_float ? 0x7Fu : 0xFFu, bitmask, counts, rows, cols, pc);
  } else if (elem_size == 2) {
    hipLaunchKernelGGL(bitmask_count_kernel<uint16_t>, grid, kBlock, 0, st, (const uint16_t*)x,
                       is_float ? 0x7FFFu : 0xFFFFu, bitmask, counts, rows, cols, pc);
  } else {
    hipLaunchKernelGGL(bitmask_count_kernel<uint32_t>, grid, kBlock, 0, st, (const uint32_t*)x,
                       is_float ? 0x7FFFFFFFu : 0xFFFFFFFFu, bitmask, counts, rows, cols, pc);
  }
  hipLaunchKernelGGL(row_offsets_kernel, 1, 1024, 0, st, counts, row_offsets, total_nnz, rows);
  return check_launch("ctmi_bitmask_count");
}

extern "C" int ctmi_bitmask_compact(const void* x, int32_t elem_size, const uint8_t* bitmask,
                                    const int64_t* row_offsets, void* values, int64_t rows,
                                    int64_t cols, void* stream) {
  CTMI_REQUIRE(rows >= 0 && cols >= 0, CTMI_ERR_VALUE, "negative shape");
  int rc = check_elem(elem_size);
  if (rc) return rc;
  if (rows == 0 || cols == 0) return CTMI_OK;
  // `values` may legitimately be NULL when the tensor holds no non-zero at all
  CTMI_REQUIRE(x && bitmask && row_offsets, CTMI_ERR_VALUE, "NULL tensor pointer");
  hipStream_t st = (hipStream_t)stream;
  const int64_t pc = cdiv(cols, 8);
  const int grid = rows_grid(rows);
  if (elem_size == 1)
    hipLaunchKernelGGL(bitmask_compact_kernel<uint8_t>, grid, kBlock, 0, st, (const uint8_t*)x,
                       bitmask, row_offsets, (uint8_t*)values, rows, cols, pc);
  else if (elem_size == 2)
    hipLaunchKernelGGL(bitmask_compact_kernel<uint16_t>, grid, kBlock, 0, st, (const uint16_t*)x,
                       bitmask, row_offsets, (uint16_t*)values, rows, cols, pc);
  else
    hipLaunchKernelGGL(bitmask_compact_kernel<uint32_t>, grid, kBlock, 0, st, (const uint32_t*)x,
                       bitmask, row_offsets, (uint32_t*)values, rows, cols, pc);
  return check_launch("ctmi_bitmask_compact");
}

extern "C" int ctmi_bitmask_decompress(const void* values, int64_t nvalues, int32_t elem_size,
                                       const uint8_t* bitmask, const int64_t* row_offsets,
                                       void* out, void* tmp, int64_t rows, int64_t cols,
                                       void* stream) {
  CTMI_REQUIRE(rows >= 0 && cols >= 0, CTMI_ERR_VALUE, "negative shape");
  int rc = check_elem(elem_size);
  if (rc) return rc;
  if (rows == 0 || cols == 0) return CTMI_OK;
  CTMI_REQUIRE(bitmask && out, CTMI_ERR_VALUE, "NULL tensor pointer");
  CTMI_REQUIRE(nvalues >= 0 && (values || nvalues == 0), CTMI_ERR_VALUE, "bad values buffer");
  CTMI_REQUIRE(row_offsets || tmp, CTMI_ERR_VALUE, "row_offsets and tmp are both NULL");
  hipStream_t st = (hipStream_t)stream;
  const int64_t pc = cdiv(cols, 8);
  const int grid = rows_grid(rows);
  if (!row_offsets) {
    int64_t* counts = (int64_t*)tmp;
    int64_t* offs = counts + rows;
    hipLaunchKernelGGL(bitmask_popcount_kernel, grid, kBlock, 0, st, bitmask, counts, rows, cols, pc);
    hipLaunchKernelGGL(row_offsets_kernel, 1, 1024, 0, st, counts, offs, (int64_t*)nullptr, rows);
    row_offsets = offs;
  }
  if (elem_size == 1)
    hipLaunchKernelGGL(bitmask_scatter_kernel<uint8_t>, grid, kBlock, 0, st, (const uint8_t*)values,
                       nvalues, bitmask, row_offsets, (uint8_t*)out, rows, cols, pc);
  else if (elem_size == 2)
    hipLaunchKernelGGL(bitmask_scatter_kernel<uint16_t>, grid, kBlock, 0, st,
                       (const uint16_t*)values, nvalues, bitmask, row_offsets, (uint16_t*)out, rows, cols, pc);
  else
    hipLaunchKernelGGL(bitmask_scatter_kernel<uint32_t>, grid, kBlock, 0, st,
                       (const uint32_t*)values, nvalues, bitmask, row_offsets, (uint32_t*)out, rows, cols, pc);
  return check_launch("ctmi_bitmask_decompress");
}

// dispatch over the element types get_24_bytemasks can rank
#define CTMI_DISPATCH_24(DTYPE, ...)                                        \
  switch (DTYPE) {                                                            \
    case CTMI_BF16: { using R = uint16_t; constexpr int DT = CTMI_BF16; __VA_ARGS__; break; } \
    case CTMI_F16: { using R = uint16_t; constexpr int DT = CTMI_F16; __VA_ARGS__; break; }   \
    case CTMI_F32: { using R = uint32_t; constexpr int DT = CTMI_F32; __VA_ARGS__; break; }   \
    default: { using R = uint8_t; constexpr int DT = CTMI_I8; __VA_ARGS__; break; }          \
  }

static int check_24_dtype(int32_t dt) {
  CTMI_REQUIRE(dt == CTMI_BF16 || dt == CTMI_F16 || dt == CTMI_F32 || dt == CTMI_F8E4M3 ||
                   dt == CTMI_I8,
               CTMI_ERR_UNSUPPORTED, "2:4 masks support float16/bfloat16/float32/float8/int8");
  return CTMI_OK;
}

extern "C" int ctmi_get_24_bytemasks(const void* x, int32_t x_dtype, uint8_t* mask, int64_t numel,
                                     void* stream) {
  CTMI_REQUIRE(numel >= 0, CTMI_ERR_VALUE, "negative size");
  CTMI_REQUIRE(numel % 4 == 0, CTMI_ERR_VALUE,
               "Tensor size must be a multiple of 4 for TWO_FOUR sparsity");
  int rc = check_24_dtype(x_dtype);
  if (rc) return rc;
  if (numel == 0) return CTMI_OK;
  CTMI_REQUIRE(x && mask, CTMI_ERR_VALUE, "NULL tensor pointer");
  CTMI_REQUIRE((uintptr_t)mask % 4 == 0, CTMI_ERR_VALUE, "mask must be 4-byte aligned");
  const int64_t ng = numel / 4;
  const int grid = grid_for(ng, kBlock);
  hipStream_t st = (hipStream_t)stream;
  CTMI_DISPATCH_24(x_dtype, hipLaunchKernelGGL((bytemask24_kernel<R, DT>), grid, kBlock, 0, st,
                                                (const R*)x, mask, ng));
  return check_launch("ctmi_get_24_bytemasks");
}

extern "C" int ctmi_sparse24_compress(const void* x, int32_t x_dtype, void* values,
                                      uint8_t* bitmask, int64_t rows, int64_t cols, void* stream) {
  CTMI_REQUIRE(rows >= 0 && cols >= 0, CTMI_ERR_VALUE, "negative shape");
  CTMI_REQUIRE((rows * cols) % 4 == 0, CTMI_ERR_VALUE,
               "Tensor size must be a multiple of 4 for TWO_FOUR sparsity");
  CTMI_REQUIRE(cols % 2 == 0, CTMI_ERR_VALUE,
               "2:4 compressed values need an even number of columns");
  int rc = check_24_dtype(x_dtype);
  if (rc) return rc;
  if (rows == 0 || cols == 0) return CTMI_OK;
  CTMI_REQUIRE(x && values && bitmask, CTMI_ERR_VALUE, "NULL tensor pointer");
  hipStream_t st = (hipStream_t)stream;
  const int es = dtype_size(x_dtype);
  const int64_t n = rows * cols;
  // work item: 16 one-byte elements, or 8 wider ones
  const int per = es == 1 ? 16 : 8;
  const bool fast = cols % 8 == 0 && n % per == 0 && (uintptr_t)x % (per * es) == 0 &&
                    (uintptr_t)values % (per * es / 2) == 0;
  if (fast) {
    if (es == 1) {
      const int64_t items = n / 16;
      hipLaunchKernelGGL((sparse24_compress_kernel<uint8_t, CTMI_I8, 16>), grid_for(items, kBlock),
                         kBlock, 0, st, (const uint8_t*)x, (uint8_t*)values, bitmask, items);
    } else if (es == 2) {
      const int64_t items = n / 8;
      if (x_dtype == CTMI_BF16)
        hipLaunchKernelGGL((sparse24_compress_kernel<uint16_t, CTMI_BF16, 8>),
                           grid_for(items, kBlock), kBlock, 0, st, (const uint16_t*)x,
                           (uint16_t*)values, bitmask, items);
      else
        hipLaunchKernelGGL((sparse24_compress_kernel<uint16_t, CTMI_F16, 8>),
                           grid_for(items, kBlock), kBlock, 0, st, (const uint16_t*)x,
                           (uint16_t*)values, bitmask, items);
    } else {
      const int64_t items = n / 8;
      hipLaunchKernelGGL((sparse24_compress_kernel<uint32_t, CTMI_F32, 8>), grid_for(items, kBlock),
                         kBlock, 0, st, (const uint32_t*)x, (uint32_t*)values, bitmask, items);
    }
    return check_launch("ctmi_sparse24_compress");
  }
  const int64_t ng = n / 4;
  const int64_t pc = cdiv(cols, 8);
  CTMI_DISPATCH_24(x_dtype, hipLaunchKernelGGL((sparse24_values_kernel<R, DT>),
                                                grid_for(ng, kBlock), kBlock, 0, st, (const R*)x,
                                                (R*)values, ng));
  CTMI_DISPATCH_24(x_dtype, hipLaunchKernelGGL((sparse24_bitmask_kernel<R, DT>),
                                                grid_for(rows * pc, kBlock), kBlock, 0, st,
                                                (const R*)x, bitmask, rows, cols, pc));
  return check_launch("ctmi_sparse24_compress");
}
