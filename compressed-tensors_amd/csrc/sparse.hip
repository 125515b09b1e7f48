// Bitmask sparsity formats.
//
//   pack_bitmasks / unpack_bitmasks     utils/helpers.py:302-339
//   bitmask_compress / decompress       compressors/sparse_compressors/sparse_bitmask.py:131-169
//   get_24_bytemasks                    compressors/sparse_compressors/sparse_24_bitmask.py:227-260
//   sparse24_bitmask_compress / decompress   sparse_24_bitmask.py:162-224
//   ... of a weight's int8 / fp8 codes, fused with quantize / dequantize
//                                       model_compressors/model_compressor.py:572-604, 638-667
//
// Bit j of bitmask byte k of a row flags column 8k+j (numpy packbits,
// bitorder="little"); the last byte of a row is zero padded.  Compacted values
// are stored in row-major order of the set bits.
#include <atomic>
#include <cstddef>
#include <cstring>
#include <mutex>
#include <type_traits>
#include <unordered_map>
#include <vector>

#include "ctmi_device.h"
#include "ctmi_host.h"
#include "job_table.h"
#include "qdq_core.h"
#include "quant_fast.h"
#include "topk24_lut.h"
#include "vec_geom.h"

namespace ctmi {

static const uint8_t kTopk24LutHost[4096] = CTMI_TOPK24_LUT_INIT;
__constant__ uint8_t kTopk24LutDev[4096] = CTMI_TOPK24_LUT_INIT;

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / kWave;
// work items per lane of the 2:4 streaming kernels (measured on fp8 codes: compress
// 1 / 2 / 4 / 8 items 5.3 / 5.4 / 5.0 / 4.7 TB/s, decompress 1 / 2 / 4 items 3.1 / 4.0 / 4.2)
#ifndef CTMI_S24_U
#define CTMI_S24_U 2
#endif
constexpr int kS24U = CTMI_S24_U;  // compress
#ifndef CTMI_S24_SCATTER_U
#define CTMI_S24_SCATTER_U 4
#endif
constexpr int kS24ScatterU = CTMI_S24_SCATTER_U;  // decompress

// ------------------------------------------------------------------ block scan
// Inclusive prefix sum over the wavefront with data-parallel-primitive moves: shifts
// inside rows of 16 lanes (lanes without a source add zero), then lane 15 of rows 0
// and 2 into rows 1 and 3, then lane 31 into rows 2 and 3.  No LDS crossbar trips.
__device__ __forceinline__ int wave_inclusive_scan(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, true);   // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, true);   // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, true);   // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, true);   // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);  // row_bcast:15
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);  // row_bcast:31
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
// Rows of whole bitmask bytes make mask and bitmask flat runs: a lane turns 16 bool
// bytes (one 16-byte load) into 2 bitmask bytes and back, all loads of a workgroup
// first, whole 32-bit words at a time: a byte is set if its low 7 bits or its top bit
// are; four flags gather into four bits by shifts.
constexpr int kPackU = 4;

__global__ void __launch_bounds__(kBlock)
pack_bitmasks_flat_kernel(const uint8_t* __restrict__ mask, uint16_t* __restrict__ packed,
                          int64_t n_items) {
  constexpr int U = kPackU;
  const int64_t i0 = (int64_t)blockIdx.x * (kBlock * U) + threadIdx.x;
  Vec<uint32_t, 4> a[U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    int64_t i = i0 + k * kBlock;
    if (i >= n_items) i = n_items - 1;  // past the end: re-read, not stored
    a[k] = ldg_nt<uint32_t, 4>(reinterpret_cast<const uint32_t*>(mask) + i * 4);
  }
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t i = i0 + k * kBlock;
    uint32_t bits = 0;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const uint32_t w = a[k].v[q];
      const uint32_t nz = ((((w & 0x7F7F7F7Fu) + 0x7F7F7F7Fu) | w) >> 7) & 0x01010101u;
      bits |= ((nz | (nz >> 7) | (nz >> 14) | (nz >> 21)) & 15u) << (4 * q);
    }
    if (i < n_items) packed[i] = (uint16_t)bits;
  }
}

__global__ void __launch_bounds__(kBlock)
unpack_bitmasks_flat_kernel(const uint16_t* __restrict__ packed, uint8_t* __restrict__ mask,
                            int64_t n_items) {
  constexpr int U = kPackU;
  const int64_t i0 = (int64_t)blockIdx.x * (kBlock * U) + threadIdx.x;
  uint32_t bits[U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t i = i0 + k * kBlock;
    bits[k] = packed[i < n_items ? i : n_items - 1];
  }
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t i = i0 + k * kBlock;
    Vec<uint32_t, 4> o;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const uint32_t kq = (bits[k] >> (4 * q)) & 15u;
      o.v[q] = (kq | (kq << 7) | (kq << 14) | (kq << 21)) & 0x01010101u;
    }
    if (i < n_items) stg_nt<uint32_t, 4>(reinterpret_cast<uint32_t*>(mask) + i * 4, o);
  }
}

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
  const bool words = vec && pc % 4 == 0 && (uintptr_t)bitmask % 4 == 0;
  for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
    const R* row = x + r * cols;
    int64_t cnt = 0;
    if (vec) {
      // 4 vectors per thread and step, all loads first
      constexpr int U = 4;
      for (int64_t b0 = threadIdx.x; b0 < pc; b0 += kBlock * U) {
        Vec<R, 8> a[U];
#pragma unroll
        for (int k = 0; k < U; ++k) {
          const int64_t b = b0 + k * kBlock;
          a[k] = ldg_nt<R, 8>(row + (b < pc ? b : pc - 1) * 8);  // past the end: re-read, not used
        }
        uint32_t mine = 0;  // the lane's four bitmask bytes, byte k for vector k
#pragma unroll
        for (int k = 0; k < U; ++k) {
          const int64_t b = b0 + k * kBlock;
          if (b < pc) {
            uint32_t bits = 0;
#pragma unroll
            for (int j = 0; j < 8; ++j) bits |= (uint32_t)(((uint32_t)a[k].v[j] & nz_mask) != 0) << j;
            if (!words) bitmask[r * pc + b] = (uint8_t)bits;
            mine |= bits << (8 * k);
            cnt += __popc(bits);
          }
        }
        if (words) {
          // four neighbouring lanes hold four neighbouring bytes of each of the four
          // vectors: lane q of the four collects vector q's and stores one 32-bit word
          // (rows of whole words: the four lanes are inside the row together or not at all)
          const int q = threadIdx.x & 3, base = lane_id() & ~3;
          uint32_t word = 0;
#pragma unroll
          for (int j = 0; j < 4; ++j)
            word |= ((__shfl(mine, base + j, kWave) >> (8 * q)) & 0xffu) << (8 * j);
          const int64_t at = b0 - q + (int64_t)q * kBlock;
          if (at < pc) *reinterpret_cast<uint32_t*>(bitmask + r * pc + at) = word;
        }
      }
    } else {
      for (int64_t b = threadIdx.x; b < pc; b += kBlock) {
        uint32_t bits = 0;
        for (int j = 0; j < 8; ++j) {
          const int64_t c = b * 8 + j;
          if (c < cols) bits |= (uint32_t)(((uint32_t)row[c] & nz_mask) != 0) << j;
        }
        bitmask[r * pc + b] = (uint8_t)bits;
        cnt += __popc(bits);
      }
    }
    const int64_t t = block_sum(cnt, red);
    if (threadIdx.x == 0) counts[r] = t;
  }
}

// per-row popcount of an existing bitmask (bits at columns >= cols ignored):
// one wavefront per row, 4 bitmask bytes per lane and step when rows are whole
// words
__device__ __forceinline__ void popcount_rows(const uint8_t* __restrict__ bitmask,
                                              int64_t* __restrict__ counts, int64_t rows,
                                              int64_t cols, int64_t pc, int64_t first_row,
                                              int64_t row_stride) {
  const int lane = lane_id();
  const uint32_t tail = (cols % 8) ? ((1u << (cols % 8)) - 1u) : 0xffu;
  for (int64_t r = first_row; r < rows; r += row_stride) {
    const uint8_t* row = bitmask + r * pc;
    int cnt = 0;
    if (pc % 4 == 0 && (uintptr_t)bitmask % 4 == 0) {
      const uint32_t* w = reinterpret_cast<const uint32_t*>(row);
      const int64_t nw = pc / 4;
      const uint32_t last = 0x00ffffffu | (tail << 24);
      for (int64_t i = lane; i < nw; i += kWave) {
        uint32_t bits = w[i];
        if (i == nw - 1) bits &= last;
        cnt += __popc(bits);
      }
    } else {
      for (int64_t b = lane; b < pc; b += kWave) {
        uint32_t bits = row[b];
        if (b == pc - 1) bits &= tail;
        cnt += __popc(bits);
      }
    }
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) cnt += __shfl_xor(cnt, d, kWave);
    if (lane == 0) counts[r] = cnt;
  }
}

__global__ void __launch_bounds__(kBlock)
bitmask_popcount_kernel(const uint8_t* __restrict__ bitmask, int64_t* __restrict__ counts,
                        int64_t rows, int64_t cols, int64_t pc) {
  popcount_rows(bitmask, counts, rows, cols, pc, (int64_t)blockIdx.x * kWaves + threadIdx.x / kWave,
                (int64_t)gridDim.x * kWaves);
}

// exclusive scan of counts[rows] -> offsets[rows], total; single workgroup.  A
// wavefront takes 512 neighbouring rows per step, 64 at a time (lanes side by side:
// whole memory lines per load and store), and scans them with DPP moves; one barrier
// per step of 8192 rows puts the wavefronts behind one another.
constexpr int kScanThreads = 1024, kScanPer = 8;

__device__ __forceinline__ int64_t wave_inclusive_scan64(int64_t v) {
#define CTMI_SCAN64_STEP(ctrl, rows, bound)                                                      \
  {                                                                                              \
    const uint32_t lo = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)v, ctrl, rows, 0xf, bound); \
    const uint32_t hi = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)((uint64_t)v >> 32), ctrl, rows, 0xf, bound); \
    v += (int64_t)(((uint64_t)hi << 32) | lo);                                                   \
  }
  CTMI_SCAN64_STEP(0x111, 0xf, true)   // row_shr:1
  CTMI_SCAN64_STEP(0x112, 0xf, true)   // row_shr:2
  CTMI_SCAN64_STEP(0x114, 0xf, true)   // row_shr:4
  CTMI_SCAN64_STEP(0x118, 0xf, true)   // row_shr:8
  CTMI_SCAN64_STEP(0x142, 0xa, false)  // row_bcast:15
  CTMI_SCAN64_STEP(0x143, 0xc, false)  // row_bcast:31
#undef CTMI_SCAN64_STEP
  return v;
}

__device__ __forceinline__ int64_t wave_last64(int64_t v) {
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, kWave - 1);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)((uint64_t)v >> 32), kWave - 1);
  return (int64_t)(((uint64_t)hi << 32) | lo);
}

__device__ __forceinline__ void scan_rows(const int64_t* __restrict__ counts,
                                          int64_t* __restrict__ offsets,
                                          int64_t* __restrict__ total, int64_t rows,
                                          int64_t* wsum) {
  int64_t carry = 0;
  const int lane = lane_id(), wave = threadIdx.x / kWave;
  for (int64_t base = 0; base < rows; base += kScanThreads * kScanPer) {
    const int64_t i0 = base + (int64_t)wave * (kWave * kScanPer) + lane;
    int64_t c[kScanPer], before[kScanPer];
#pragma unroll
    for (int k = 0; k < kScanPer; ++k) {  // all loads first: no condition on the load itself
      const int64_t i = i0 + k * kWave;
      c[k] = counts[i < rows ? i : rows - 1];
    }
#pragma unroll
    for (int k = 0; k < kScanPer; ++k) c[k] = i0 + k * kWave < rows ? c[k] : 0;
    int64_t mine = 0;  // of the wavefront's rows so far
#pragma unroll
    for (int k = 0; k < kScanPer; ++k) {
      const int64_t inc = wave_inclusive_scan64(c[k]);
      before[k] = mine + inc - c[k];
      mine += wave_last64(inc);
    }
    if (lane == 0) wsum[wave] = mine;
    __syncthreads();
    int64_t woff = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < kScanThreads / kWave; ++w) {
      const int64_t sv = wsum[w];
      woff += w < wave ? sv : 0;
      tot += sv;
    }
#pragma unroll
    for (int k = 0; k < kScanPer; ++k)
      if (i0 + k * kWave < rows) offsets[i0 + k * kWave] = carry + woff + before[k];
    carry += tot;
    __syncthreads();
  }
  if (threadIdx.x == 0 && total) *total = carry;
}

__global__ void __launch_bounds__(kScanThreads)
row_offsets_kernel(const int64_t* __restrict__ counts, int64_t* __restrict__ offsets,
                   int64_t* __restrict__ total, int64_t rows) {
  __shared__ int64_t wsum[kScanThreads / kWave];
  scan_rows(counts, offsets, total, rows, wsum);
}

// ------------------------------------------------------------------ sparse-bitmask: compaction
// One workgroup per row, 2048 columns per iteration.  Survivors are first
// gathered into LDS at their rank within the iteration, then the contiguous
// run is written to HBM by the whole workgroup, so global stores are dense
// regardless of where the non-zeros sit.
// Rows of whole bitmask bytes, x aligned to 8 elements: 8192 columns per step.  A lane
// issues its four bitmask bytes and four 16-byte loads before anything else; the four
// counts ride through one workgroup scan as 16-bit fields of two words; the survivors
// are laid out in LDS with the misalignment of their destination, so that what leaves
// are aligned 16-byte stores (single elements only at the two ends).
template <typename R>
__global__ void __launch_bounds__(kBlock)
bitmask_compact_rows_kernel(const R* __restrict__ x, const uint8_t* __restrict__ bitmask,
                            const int64_t* __restrict__ row_offsets, R* __restrict__ values,
                            int64_t rows, int64_t cols, int64_t pc) {
  constexpr int U = 4;
  constexpr int VE = 16 / (int)sizeof(R);
  __shared__ uint32_t w01[kWaves], w23[kWaves];
  __shared__ __align__(16) R stage[kBlock * 8 * U + VE];
  const int tid = threadIdx.x, lane = lane_id(), wave = tid / kWave;
  for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
    const R* row = x + r * cols;
    const uint8_t* mrow = bitmask + r * pc;
    R* dst = values + row_offsets[r];
    for (int64_t b0 = 0; b0 < pc; b0 += kBlock * U) {
      uint32_t bits[U];
      Vec<R, 8> a[U];
#pragma unroll
      for (int k = 0; k < U; ++k) {
        const int64_t b = b0 + k * kBlock + tid;
        bits[k] = 0;
        if (b < pc) {
          bits[k] = mrow[b];
          a[k] = ldg_nt<R, 8>(row + b * 8);
        }
      }
      const uint32_t c01 = (uint32_t)__popc(bits[0]) | ((uint32_t)__popc(bits[1]) << 16);
      const uint32_t c23 = (uint32_t)__popc(bits[2]) | ((uint32_t)__popc(bits[3]) << 16);
      const uint32_t inc01 = (uint32_t)wave_inclusive_scan((int)c01);
      const uint32_t inc23 = (uint32_t)wave_inclusive_scan((int)c23);
      if (lane == kWave - 1) {
        w01[wave] = inc01;
        w23[wave] = inc23;
      }
      __syncthreads();
      uint32_t off01 = 0, off23 = 0, tot01 = 0, tot23 = 0;
#pragma unroll
      for (int w = 0; w < kWaves; ++w) {
        const uint32_t s01 = w01[w], s23 = w23[w];
        if (w < wave) { off01 += s01; off23 += s23; }
        tot01 += s01;
        tot23 += s23;
      }
      const uint32_t pre01 = off01 + inc01 - c01, pre23 = off23 + inc23 - c23;
      const int tot[U] = {(int)(tot01 & 0xffffu), (int)(tot01 >> 16), (int)(tot23 & 0xffffu),
                          (int)(tot23 >> 16)};
      const int pre[U] = {(int)(pre01 & 0xffffu), (int)(pre01 >> 16), (int)(pre23 & 0xffffu),
                          (int)(pre23 >> 16)};
      const int mis = (int)(((uintptr_t)dst % 16) / sizeof(R));
      int base = mis;
#pragma unroll
      for (int k = 0; k < U; ++k) {
        int at = base + pre[k];
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if ((bits[k] >> j) & 1u) stage[at++] = a[k].v[j];
        base += tot[k];
      }
      __syncthreads();
      const int end = base;         // stage[mis, end) -> dst[0, end - mis)
      R* dst_al = dst - mis;        // 16-byte aligned
      for (int e0 = tid * VE; e0 < end; e0 += kBlock * VE) {
        if (e0 >= mis && e0 + VE <= end) {
          stg<R, VE>(dst_al + e0, *reinterpret_cast<const Vec<R, VE>*>(stage + e0));
        } else {
          for (int e = e0; e < e0 + VE; ++e)
            if (e >= mis && e < end) dst_al[e] = stage[e];
        }
      }
      dst += end - mis;
      __syncthreads();
    }
  }
}

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
// One row by one workgroup, 2048 columns per step: the step's values are staged in
// LDS, every thread picks its own 8.  `src` is where the row's values start and is
// moved past them.  A bitmask with more set bits than there are values reads
// zeros, never past the end.
// `store(b, o)` takes the 8 elements that bitmask byte b of the row stands for.
template <typename R, typename Store>
__device__ __forceinline__ void scatter_row_to(const R* __restrict__ values, int64_t nvalues,
                                               const uint8_t* __restrict__ mask_row, int64_t& src,
                                               int64_t pc, uint32_t tail, int* scan_s, R* stage,
                                               Store store) {
  for (int64_t b0 = 0; b0 < pc; b0 += kBlock) {
    const int64_t b = b0 + threadIdx.x;
    uint32_t bits = 0;
    if (b < pc) {
      bits = mask_row[b];
      if (b == pc - 1) bits &= tail;
    }
    int pre, total;
    block_exclusive_scan(__popc(bits), &pre, &total, scan_s);
    for (int i = threadIdx.x; i < total; i += kBlock)
      stage[i] = (src + i < nvalues) ? values[src + i] : (R)0;
    src += total;
    __syncthreads();
    if (b < pc) {
      Vec<R, 8> o;
#pragma unroll
      for (int j = 0; j < 8; ++j) o.v[j] = ((bits >> j) & 1u) ? stage[pre++] : (R)0;
      store(b, o);
    }
    __syncthreads();
  }
}

// ... into a dense row of the same element type
template <typename R>
__device__ __forceinline__ void scatter_row(const R* __restrict__ values, int64_t nvalues,
                                            const uint8_t* __restrict__ mask_row, int64_t& src,
                                            R* __restrict__ row, int64_t cols, int64_t pc, bool vec,
                                            uint32_t tail, int* scan_s, R* stage) {
  scatter_row_to<R>(values, nvalues, mask_row, src, pc, tail, scan_s, stage,
                    [&](int64_t b, const Vec<R, 8>& o) {
                      if (vec) {
                        stg<R, 8>(row + b * 8, o);
                      } else {
                        for (int j = 0; j < 8; ++j) {
                          const int64_t c = b * 8 + j;
                          if (c < cols) row[c] = o.v[j];
                        }
                      }
                    });
}

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
    int64_t src = row_offsets[r];
    scatter_row<R>(values, nvalues, bitmask + r * pc, src, out + r * cols, cols, pc, vec, tail, scan_s,
                   stage);
  }
}

// ------------------------------------------------------------------ bitmask decompress, one wavefront per row
// For rows that are whole 16-column words (cols % 16 == 0) and 16-byte aligned
// buffers.  A lane owns 16 neighbouring columns of a 1024-column span; the
// wavefront's scan of the lanes' popcounts says where each lane's values start,
// the values of the span are copied into a wave-private patch of LDS with
// aligned 16-byte loads, and every lane picks its own out of it.  No workgroup
// barrier anywhere: LDS operations of one wavefront complete in order.  The
// row's bitmask is fetched in one go before anything depends on it.
constexpr int kScatterSpan = 1024;      // columns per wavefront and step
constexpr int kScatterMaxSteps = 16;    // rows of up to 16384 columns
template <typename R>
__global__ void __launch_bounds__(kBlock)
bitmask_scatter_wave_kernel(const R* __restrict__ values, int64_t nvalues,
                            const uint8_t* __restrict__ bitmask,
                            const int64_t* __restrict__ row_offsets, R* __restrict__ out,
                            int64_t rows, int64_t cols, int64_t pc) {
  constexpr int VE = 16 / (int)sizeof(R);  // elements per 16-byte vector
  __shared__ __align__(16) R stage_all[kWaves][kScatterSpan + 2 * VE];
  const int lane = lane_id(), wave = threadIdx.x / kWave;
  R* stage = stage_all[wave];
  for (int64_t r = (int64_t)blockIdx.x * kWaves + wave; r < rows; r += (int64_t)gridDim.x * kWaves) {
  const uint16_t* words = reinterpret_cast<const uint16_t*>(bitmask + r * pc);
  const int steps = (int)((cols + kScatterSpan - 1) / kScatterSpan);
  uint32_t bits_of[kScatterMaxSteps];
#pragma unroll
  for (int it = 0; it < kScatterMaxSteps; ++it) {
    const int64_t col = (int64_t)it * kScatterSpan + 16 * lane;
    bits_of[it] = (it < steps && col < cols) ? words[col / 16] : 0u;
  }
  int64_t src = row_offsets[r];
  R* row = out + r * cols;
#pragma unroll
  for (int it = 0; it < kScatterMaxSteps; ++it) {
    if (it >= steps) break;
    const uint32_t bits = bits_of[it];
    const int cnt = __popc(bits);
    const int inc = wave_inclusive_scan(cnt);
    const int total = __shfl(inc, kWave - 1, kWave);
    // values [src, src + total) -> stage, from the 16-byte boundary below src
    const int64_t base = src & ~(int64_t)(VE - 1);
    const int off = (int)(src - base);
    const int nvecs = (off + total + VE - 1) / VE;
    for (int i = lane; i < nvecs; i += kWave) {
      const int64_t e0 = base + (int64_t)i * VE;
      Vec<R, VE> v;
      if (e0 < nvalues) {
        // an aligned vector that starts inside the buffer never leaves its page
        v = ldg<R, VE>(values + e0);
#pragma unroll
        for (int e = 0; e < VE; ++e)
          if (e0 + e >= nvalues) v.v[e] = (R)0;  // more set bits than values: zeros
      } else {
#pragma unroll
        for (int e = 0; e < VE; ++e) v.v[e] = (R)0;
      }
      *reinterpret_cast<Vec<R, VE>*>(stage + i * VE) = v;
    }
    asm volatile("" ::: "memory");  // the reads below are of other lanes' writes
    const int64_t col = (int64_t)it * kScatterSpan + 16 * lane;
    if (col < cols) {
      int idx = off + inc - cnt;
      Vec<R, 16> o;
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const bool set = (bits >> j) & 1u;
        o.v[j] = set ? stage[idx] : (R)0;
        idx += set ? 1 : 0;
      }
#pragma unroll
      for (int h = 0; h < 16 / VE; ++h) {
        Vec<R, VE> part;
#pragma unroll
        for (int e = 0; e < VE; ++e) part.v[e] = o.v[h * VE + e];
        stg<R, VE>(row + col + h * VE, part);
      }
    }
    asm volatile("" ::: "memory");  // the next step's writes must not overtake these reads
    src += total;
  }
  }
}

template <typename R>
static bool scatter_wave_ok(const void* values, const uint8_t* bitmask, const void* out,
                            int64_t cols) {
  return cols % 16 == 0 && cols <= (int64_t)kScatterSpan * kScatterMaxSteps &&
         (uintptr_t)values % 16 == 0 && (uintptr_t)out % 16 == 0 && (uintptr_t)bitmask % 2 == 0 &&
         (cols * sizeof(R)) % 16 == 0;
}

// ------------------------------------------------------------------ bitmask decompress by tiles
// With rows of whole bitmask bytes the bitmask is one flat run of bits and the
// values one flat run in the same order, so rows do not matter.  The tensor is
// cut into tiles of kTileElems elements; a first pass counts the set bits of
// every tile (one wavefront per tile), row_offsets_kernel turns the counts into
// where each tile's values start, and the scatter then knows before it has looked
// at anything which values a tile needs: it fetches them together with the tile's
// bitmask, stages them in LDS and every lane picks its own.
constexpr int kTileElems = kBlock * 16;        // 16 elements per lane of the scatter
constexpr int kTileBytes = kTileElems / 8;     // bitmask bytes per tile

__global__ void __launch_bounds__(kBlock)
tile_popcount_kernel(const uint8_t* __restrict__ bitmask, int64_t nbytes,
                     int64_t* __restrict__ counts, int64_t ntiles) {
  const int lane = lane_id();
  const int64_t tile = (int64_t)blockIdx.x * kWaves + threadIdx.x / kWave;
  if (tile >= ntiles) return;
  int cnt = 0;
#pragma unroll
  for (int i = 0; i < kTileBytes; i += kWave * 16) {
    const int64_t b0 = tile * kTileBytes + i + lane * 16;
    if (i + lane * 16 >= kTileBytes) {
      // a tile shorter than one step of the wavefront
    } else if (b0 + 16 <= nbytes) {
      const u32x4_t q = *reinterpret_cast<const u32x4_t*>(bitmask + b0);
      cnt += __popc(q.x) + __popc(q.y) + __popc(q.z) + __popc(q.w);
    } else {
      for (int64_t b = b0; b < nbytes; ++b) cnt += __popc((uint32_t)bitmask[b]);
    }
  }
#pragma unroll
  for (int d = kWave / 2; d > 0; d >>= 1) cnt += __shfl_xor(cnt, d, kWave);
  if (lane == 0) counts[tile] = cnt;
}

// The same count for tensors of up to kGroupTiles * kMaxGroups tiles, without the
// scan kernel in between: a workgroup counts a group of kGroupTiles neighbouring
// tiles and leaves, per tile, the count of the group's earlier tiles and its own, and
// per group its total.  A scatter workgroup adds up the totals of the groups before
// its own (at most kMaxGroups numbers, resident in L2) and finds its place.  Nothing
// is handed from one workgroup to another inside a launch: the end of the count
// kernel is what makes its stores visible, and the library keeps no state of its own.
constexpr int kGroupTiles = 64;
#ifndef CTMI_SCATTER_TILES
#define CTMI_SCATTER_TILES 1
#endif
// tiles a scatter workgroup takes (8192x8192 bf16, half the bits set: 1 and 2 run alike,
// 4 is a fifth slower: the kernel is not waiting for memory latency)
constexpr int kScatterTiles = CTMI_SCATTER_TILES;
constexpr int kGroupThreads = 1024;
constexpr int kMaxGroups = 1024;
struct TileInfo {
  int32_t before;  // set bits in the group's earlier tiles
  int32_t count;   // set bits in the tile
};

__global__ void __launch_bounds__(kGroupThreads)
tile_popcount_groups_kernel(const uint8_t* __restrict__ bitmask, int64_t nbytes,
                            TileInfo* __restrict__ info, int32_t* __restrict__ group_total,
                            int64_t ntiles) {
  constexpr int kPerWave = kGroupTiles / (kGroupThreads / kWave);  // tiles per wavefront
  static_assert(kPerWave == 4 && kTileBytes == 32 * 16,
                "a wavefront reads two tiles per load, half a wavefront each");
  __shared__ int cnt_s[kGroupTiles];
  const int lane = lane_id(), wave = threadIdx.x / kWave;
  const int64_t tile0 = (int64_t)blockIdx.x * kGroupTiles;
  // The wavefront's four tiles are 2 KB in a row: two 16-byte loads per lane, both
  // issued before anything is counted (an address past the end is replaced, what it
  // brings is not used).  The counts of the two loads ride through one scan as
  // 16-bit fields; lanes 31 and 63 then hold what the four tiles add up to.
  const int64_t b0 = (tile0 + wave * kPerWave) * kTileBytes + lane * 16;
  u32x4_t q[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int64_t b = b0 + j * (kWave * 16);
    q[j] = *reinterpret_cast<const u32x4_t*>(bitmask + (b < nbytes ? b : 0));
  }
  uint32_t cnt2 = 0;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int64_t b = b0 + j * (kWave * 16);
    int c = 0;
    if (b + 16 <= nbytes) {
      c = __popc(q[j].x) + __popc(q[j].y) + __popc(q[j].z) + __popc(q[j].w);
    } else {
      for (int64_t at = b; at < nbytes; ++at) c += __popc((uint32_t)bitmask[at]);
    }
    cnt2 |= (uint32_t)c << (16 * j);
  }
  const uint32_t inc2 = (uint32_t)wave_inclusive_scan((int)cnt2);
  const uint32_t half = (uint32_t)__builtin_amdgcn_readlane((int)inc2, kWave / 2 - 1);
  const uint32_t all = (uint32_t)__builtin_amdgcn_readlane((int)inc2, kWave - 1);
  if (lane == 0) {
    cnt_s[wave * kPerWave + 0] = (int)(half & 0xffffu);
    cnt_s[wave * kPerWave + 1] = (int)((all & 0xffffu) - (half & 0xffffu));
    cnt_s[wave * kPerWave + 2] = (int)(half >> 16);
    cnt_s[wave * kPerWave + 3] = (int)((all >> 16) - (half >> 16));
  }
  __syncthreads();
  if (wave == 0) {
    const int c = cnt_s[lane];
    const int inc = wave_inclusive_scan(c);
    if (tile0 + lane < ntiles) info[tile0 + lane] = TileInfo{inc - c, c};
    if (lane == kWave - 1) group_total[blockIdx.x] = inc;
  }
}

// Set bits beyond nvalues read as zero.  GROUPED: positions from
// tile_popcount_groups_kernel (info, group_total), else from tile_popcount_kernel
// and the scan behind it (tile_counts, tile_offsets).
//
// A wavefront takes 1024 neighbouring elements of the tile, as 16-byte pieces: piece q
// of lane l is elements [q * 64 * VE + l * VE, + VE) of the stretch, so that every
// store instruction of the wavefront writes 1 KB without gaps (whole memory lines; with
// a lane's 16 elements side by side a store would leave every other 16 bytes to the
// next one, and the device moves such halves noticeably slower).
//
// A workgroup takes T neighbouring tiles (of one group) and goes through them side by
// side: bitmask bytes and values of all T are asked for before anything is waited for.
template <typename R, bool GROUPED, int T>
__global__ void __launch_bounds__(kBlock)
bitmask_scatter_tiles_kernel(const R* __restrict__ values, int64_t nvalues,
                             const uint8_t* __restrict__ bitmask,
                             const int64_t* __restrict__ tile_counts,
                             const int64_t* __restrict__ tile_offsets,
                             const TileInfo* __restrict__ info,
                             const int32_t* __restrict__ group_total, R* __restrict__ out,
                             int64_t numel, int64_t ntiles) {
  constexpr int VE = 16 / (int)sizeof(R);  // elements of a piece
  constexpr int NP = 16 / VE;              // pieces of a lane
  constexpr int P = (NP + 1) / 2;
  constexpr int kStage = kTileElems + 2 * VE + 16;
  constexpr int kRoundsIn = (kTileElems + 2 * VE) / (kBlock * VE) + 1;  // vectors a lane stages
  static_assert(kTileElems == kWaves * kWave * 16, "1024 elements per wavefront");
  static_assert(kGroupTiles % T == 0, "the tiles of a workgroup share a group");
  __shared__ int wtot[T][kWaves];
  // a tile's values, up to VE - 1 before them and room for the reads of unset
  // elements behind the last one
  __shared__ __align__(16) R stage[T][kStage];
  const int tid = threadIdx.x, lane = lane_id(), wave = tid / kWave;
  const int64_t tile0 = (int64_t)blockIdx.x * T;
  // the lane's pieces and their bits (numel is a multiple of 16: a piece is inside
  // the tensor as a whole or not at all)
  uint32_t bits[T][NP];
#pragma unroll
  for (int t = 0; t < T; ++t) {
    const int64_t elem0 = (tile0 + t) * kTileElems + wave * (kWave * 16) + lane * VE;
#pragma unroll
    for (int q = 0; q < NP; ++q) {
      const int64_t elem = elem0 + q * (kWave * VE);
      bits[t][q] = 0;
      if (elem < numel) {
        if constexpr (VE == 16) bits[t][q] = reinterpret_cast<const uint16_t*>(bitmask)[elem >> 4];
        else bits[t][q] = ((uint32_t)bitmask[elem >> 3] >> (elem & 7)) & ((1u << VE) - 1u);
      }
    }
  }
  int64_t excl[T];
  int total[T];
  if constexpr (GROUPED) {
    // set bits before the tiles' group: every wavefront adds the totals of the earlier
    // groups up by itself, four neighbouring totals a lane and round (group_total is
    // aligned to 16 bytes and readable up to the next multiple of 4 totals), 256 groups a
    // round, and no barrier.  The number of rounds is the same for the whole workgroup.
    // (a tensor on this path has at most kMaxGroups * kGroupTiles * kTileElems = 2^28 elements)
    const int group = (int)(tile0 / kGroupTiles);
    constexpr int kRounds = kMaxGroups / (4 * kWave);
    const auto counted = [&](const u32x4_t v, int first) {  // of four totals from group `first` on
      const int left = group - first;
      return (int)v.x + (left > 1 ? (int)v.y : 0) + (left > 2 ? (int)v.z : 0) + (left > 3 ? (int)v.w : 0);
    };
    int sum = 0;
    if (lane * 4 < group)
      sum = counted(*reinterpret_cast<const u32x4_t*>(group_total + lane * 4), lane * 4);
    if (group > 4 * kWave) {  // tensors beyond 2^26 elements: the other rounds, loads first
      u32x4_t part[kRounds];
#pragma unroll
      for (int k = 1; k < kRounds; ++k) {
        part[k] = u32x4_t{0, 0, 0, 0};
        if (k * 4 * kWave + lane * 4 < group)
          part[k] = *reinterpret_cast<const u32x4_t*>(group_total + k * 4 * kWave + lane * 4);
      }
#pragma unroll
      for (int k = 1; k < kRounds; ++k) sum += counted(part[k], k * 4 * kWave + lane * 4);
    }
    sum = __builtin_amdgcn_readlane(wave_inclusive_scan(sum), kWave - 1);
#pragma unroll
    for (int t = 0; t < T; ++t) {
      const TileInfo ti = tile0 + t < ntiles ? info[tile0 + t] : TileInfo{0, 0};
      excl[t] = (int64_t)sum + ti.before;
      total[t] = ti.count;
    }
  } else {
#pragma unroll
    for (int t = 0; t < T; ++t) {
      const bool in = tile0 + t < ntiles;
      excl[t] = in ? tile_offsets[tile0 + t] : 0;
      total[t] = in ? (int)tile_counts[tile0 + t] : 0;
    }
  }

  // values [excl, excl + total) -> LDS, from the 16-byte boundary below excl; lanes
  // count in elements from there, `have` of which exist.  All loads of all tiles first.
  int off[T];
  Vec<R, VE> in[T][kRoundsIn] = {};
#pragma unroll
  for (int t = 0; t < T; ++t) {
    const int64_t base = excl[t] & ~(int64_t)(VE - 1);
    off[t] = (int)(excl[t] - base);
    const int nvecs = (off[t] + total[t] + VE - 1) / VE;
    const int64_t left = nvalues - base;
    const int have = (int)(left < 0 ? 0 : left > kTileElems + 2 * VE ? kTileElems + 2 * VE : left);
    const R* from = values + base;
#pragma unroll
    for (int r = 0; r < kRoundsIn; ++r) {
      const int e0 = (r * kBlock + tid) * VE;
      // an aligned vector that starts inside the buffer never leaves its page
      if (r * kBlock + tid < nvecs && e0 < have) in[t][r] = ldg<R, VE>(from + e0);
    }
  }
#pragma unroll
  for (int t = 0; t < T; ++t) {
    const int64_t base = excl[t] & ~(int64_t)(VE - 1);
    const int nvecs = (off[t] + total[t] + VE - 1) / VE;
    const int64_t left = nvalues - base;
    const int have = (int)(left < 0 ? 0 : left > kTileElems + 2 * VE ? kTileElems + 2 * VE : left);
#pragma unroll
    for (int r = 0; r < kRoundsIn; ++r) {
      const int e0 = (r * kBlock + tid) * VE;
      if (r * kBlock + tid < nvecs) {
        Vec<R, VE> v = in[t][r];
        if (e0 + VE > have) {  // set bits beyond the values read as zero
#pragma unroll
          for (int e = 0; e < VE; ++e)
            if (e0 + e >= have) v.v[e] = (R)0;
        }
        *reinterpret_cast<Vec<R, VE>*>(&stage[t][e0]) = v;
      }
    }
  }
  // Ranks.  In a tile's order a wavefront's piece q of all lanes comes before its
  // piece q + 1.  Two pieces' counts ride through one scan as 16-bit fields.
  int first[T][NP];
#pragma unroll
  for (int t = 0; t < T; ++t) {
    int wave_total = 0;
#pragma unroll
    for (int p = 0; p < P; ++p) {
      uint32_t cnt2 = (uint32_t)__popc(bits[t][2 * p]);
      if (2 * p + 1 < NP) cnt2 |= (uint32_t)__popc(bits[t][2 * p + 1]) << 16;
      const uint32_t inc2 = (uint32_t)wave_inclusive_scan((int)cnt2);
      const uint32_t all2 = (uint32_t)__builtin_amdgcn_readlane((int)inc2, kWave - 1);
      const uint32_t below2 = inc2 - cnt2;
      first[t][2 * p] = wave_total + (int)(below2 & 0xffffu);
      wave_total += (int)(all2 & 0xffffu);
      if (2 * p + 1 < NP) {
        first[t][2 * p + 1] = wave_total + (int)(below2 >> 16);
        wave_total += (int)(all2 >> 16);
      }
    }
    if (lane == 0) wtot[t][wave] = wave_total;
  }
  __syncthreads();
  // Element j of a piece is value number popcount(bits below j) of the piece's if bit j
  // is set.  Every element is read, set or not (the place is inside the staged image
  // either way), and cleared by a mask afterwards: no branch per element.
#pragma unroll
  for (int t = 0; t < T; ++t) {
    int before = off[t];
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const int wt = wtot[t][w];
      before += w < wave ? wt : 0;
    }
    const int64_t elem0 = (tile0 + t) * kTileElems + wave * (kWave * 16) + lane * VE;
#pragma unroll
    for (int q = 0; q < NP; ++q) {
      const int64_t elem = elem0 + q * (kWave * VE);
      if (elem < numel) {
        const uint32_t mine = bits[t][q];
        const R* st = &stage[t][before + first[t][q]];
        Vec<R, VE> o;
        if constexpr (sizeof(R) == 2) {
          uint32_t w2[VE / 2];
#pragma unroll
          for (int h = 0; h < VE / 2; ++h) {
            const uint32_t lo = st[__popc(mine & ((1u << (2 * h)) - 1u))];
            const uint32_t hi = st[__popc(mine & ((1u << (2 * h + 1)) - 1u))];
            const uint32_t keep_lo = (uint32_t)((int32_t)(mine << (31 - 2 * h)) >> 31);
            const uint32_t keep_hi = (uint32_t)((int32_t)(mine << (30 - 2 * h)) >> 31);
            w2[h] = (lo | (hi << 16)) & ((keep_lo & 0xffffu) | (keep_hi & 0xffff0000u));
          }
          o = __builtin_bit_cast(Vec<R, VE>, w2);
        } else {
#pragma unroll
          for (int j = 0; j < VE; ++j) {
            const R v = st[__popc(mine & ((1u << j) - 1u))];
            const R keep = (R)(0 - (R)((mine >> j) & 1u));
            o.v[j] = v & keep;
          }
        }
        stg_nt<R, VE>(out + elem, o);
      }
    }
  }
}

// ------------------------------------------------------------------ 2:4 decompress, streaming
// In a well-formed 2:4 bitmask every group of 4 columns keeps exactly 2, so the
// values of group g are values[2g], values[2g+1] and no prefix sum over the
// bitmask is needed: a lane turns E columns' worth of mask bits and E/2 values
// into 16-byte stores.  Whether the bitmask IS well formed is only known once
// all of it has been looked at.  Every lane checks its own bits, and a workgroup
// that met a group which does not keep exactly 2 says so in a word of the launch.
// sparse24_repair_kernel, enqueued behind the streaming kernel, reads that one
// word and is done if it is zero; otherwise (a bitmask no 2:4 compressor wrote) it
// redoes the tensors named there as a general scatter.  The second kernel has to be
// a kernel of its own: its stores replace those of the first, and only the end of a
// kernel puts the first kernel's stores, which may still sit in the L2 of another
// XCD, in front of them.  (A fence per workgroup that would order them inside one
// kernel writes that L2 back every time: measured 20 times slower.)
//
// The words: kS24Slots pairs {jobs with a bad group, repair workgroups done} in
// device memory of the library, all zero between launches (a repair that found
// something puts its pair back to zero when its last workgroup is done).  A pair
// belongs to a launch from the start of its streaming kernel to the end of its repair
// kernel.  Launches on one stream run one after the other, so a stream keeps one pair
// for all its launches; every stream gets a pair of its own until kS24Slots streams
// have been seen, and only then do streams share (two launches that share a pair and
// overlap in time could take each other's verdict).
constexpr int kS24Slots = 256;
__device__ unsigned int s24_slot_state[kS24Slots][2];

static uint32_t s24_slot_of(hipStream_t st) {
  static std::mutex m;
  static std::unordered_map<hipStream_t, uint32_t> slots;
  static uint32_t next = 0;
  std::lock_guard<std::mutex> lock(m);
  auto it = slots.find(st);
  if (it != slots.end()) return it->second;
  if (slots.size() >= (1u << 16)) slots.clear();  // handles of streams long gone
  const uint32_t slot = next++ % kS24Slots;
  slots.emplace(st, slot);
  return slot;
}

// called by every thread of a streaming workgroup: `bad` goes up for job `job`
__device__ __forceinline__ void s24_report(uint32_t slot, uint32_t job, bool bad) {
  if (__syncthreads_or(bad) && threadIdx.x == 0) atomicOr(&s24_slot_state[slot][0], 1u << job);
}

// In the kernel behind: the set of jobs to redo (the same in every thread), 0 for
// well-formed bitmasks.
__device__ __forceinline__ uint32_t s24_bad_jobs(uint32_t slot) {
  return __hip_atomic_load(&s24_slot_state[slot][0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ... and once a repair workgroup is done with them: the last one clears the pair
__device__ __forceinline__ void s24_repair_done(uint32_t slot) {
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned int* st = s24_slot_state[slot];
    if (atomicAdd(&st[1], 1u) == gridDim.x - 1) {
      atomicExch(&st[0], 0u);
      atomicExch(&st[1], 0u);
    }
  }
}

template <typename R>
struct Scatter24 {
  static constexpr int E = sizeof(R) == 1 ? 16 : 8;  // columns per lane
  using MaskT = typename std::conditional<E == 16, uint16_t, uint8_t>::type;
};

// Byte selectors for v_perm_b32, 32 per element size, in LDS: entry (m, h) places the two
// survivors of a group with mask nibble m.  One-byte elements: the group's 4 output bytes
// from the pair (a, b) in the low (h = 0) or high (h = 1) half of a word of values.
// Two-byte elements: output elements 2h and 2h + 1 from the word (a, b).  The first kept
// position takes a, every later one b, a dropped one the constant zero (selector 0x0c).
template <int ES>
__device__ __forceinline__ uint32_t s24_selector(int idx) {
  const uint32_t m = (uint32_t)idx & 15u, h = (uint32_t)idx >> 4;
  uint32_t sel = 0;
  if constexpr (ES == 1) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const bool keep = (m >> q) & 1u, second = (m & ((1u << q) - 1u)) != 0;
      sel |= (keep ? 2u * h + (second ? 1u : 0u) : 0x0cu) << (8 * q);
    }
  } else {
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const uint32_t q = 2u * h + (uint32_t)e;
      const bool keep = (m >> q) & 1u, second = (m & ((1u << q) - 1u)) != 0;
      sel |= (keep ? (second ? 0x0302u : 0x0100u) : 0x0c0cu) << (16 * e);
    }
  }
  return sel;
}

struct S24Job {
  const void* values;
  const uint8_t* bitmask;
  void* out;
  int64_t nvalues, rows, cols;
};

// kernel argument (the only one: find_job_index reads its head)
struct S24Table {
  uint32_t chunk_end[kMaxJobs];  // running total of workgroups, job 0 .. j (unused: 0xFFFFFFFF)
  uint32_t n_items[kMaxJobs];
  S24Job job[kMaxJobs];
  uint32_t slot;
};
static_assert(offsetof(S24Table, chunk_end) == 0 && offsetof(S24Table, n_items) == 32, "find_job_index");

// The stacked kernels (codes AND 2:4 in one pass) for up to 8 weights per launch.  compress: src
// the dense weight, dst the values; decompress: src the values, dst the dense weight; an item is
// 8 neighbouring elements of the dense side.
struct QS24Table {  // the kernel's only argument: find_job_index reads its head
  uint32_t chunk_end[kMaxJobs];  // running total of workgroups, job 0 .. j (unused: 0xFFFFFFFF)
  uint32_t n_items[kMaxJobs];
  ChainJob job[kMaxJobs];
  uint8_t* bitmask[kMaxJobs];
  int64_t rows[kMaxJobs];        // (decompress: what the repair needs)
  float qmin, qmax;
  uint32_t slot;
};
static_assert(offsetof(QS24Table, chunk_end) == 0 && offsetof(QS24Table, n_items) == 32, "find_job_index");

// The general scatter of a whole tensor, rows dealt round-robin to the workgroups of the
// launch; where a row's values start is the number of set bits before it, which each
// workgroup counts by itself as it moves from one of its rows to the next (rows are whole
// bitmask bytes here, so the rows in between are one run of bytes).
template <typename R>
__device__ void s24_redo_job(const S24Job& job, int* scan_s, int64_t* red, R* stage) {
  const R* values = static_cast<const R*>(job.values);
  R* out = static_cast<R*>(job.out);
  const int64_t pc = job.cols / 8;
  const bool vec = (uintptr_t)out % (8 * sizeof(R)) == 0;
  int64_t src = 0, counted = 0;  // set bits in rows [0, counted)
  for (int64_t r = blockIdx.x; r < job.rows; r += gridDim.x) {
    int64_t c = 0;
    for (int64_t b = counted * pc + threadIdx.x; b < r * pc; b += kBlock)
      c += __popc((uint32_t)job.bitmask[b]);
    src += block_sum(c, red);
    scatter_row<R>(values, job.nvalues, job.bitmask + r * pc, src, out + r * job.cols, job.cols, pc,
                   vec, 0xffu, scan_s, stage);
    counted = r + 1;
  }
}

template <typename R>
__global__ void __launch_bounds__(kBlock) sparse24_scatter_kernel(S24Table t) {
  constexpr int E = Scatter24<R>::E, U = kS24ScatterU;
  constexpr int VE = 16 / (int)sizeof(R);  // elements per 16-byte access
  using MaskT = typename Scatter24<R>::MaskT;
  constexpr uint32_t kAll = E == 16 ? 0xFFFFu : 0xFFu;
  __shared__ uint32_t lut[32];
  if constexpr (sizeof(R) < 4) {
    if (threadIdx.x < 32) lut[threadIdx.x] = s24_selector<(int)sizeof(R)>((int)threadIdx.x);
    __syncthreads();
  }
  uint32_t local, n_items;
  const uint32_t j = find_job_index(blockIdx.x, &local, &n_items);
  const S24Job job = t.job[j];
  const R* __restrict__ values = static_cast<const R*>(job.values);
  R* __restrict__ out = static_cast<R*>(job.out);
  const uint32_t i0 = local * (kBlock * U) + threadIdx.x;
  MaskT m[U];
  Vec<R, E / 2> v[U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    // past the end: re-read the last item (not stored)
    uint32_t i = i0 + k * kBlock;
    if (i >= n_items) i = n_items - 1;
    m[k] = reinterpret_cast<const MaskT*>(job.bitmask)[i];
    if constexpr (sizeof(R) * (E / 2) <= 16) {
      v[k] = ldg<R, E / 2>(values + (int64_t)i * (E / 2));
    } else {
#pragma unroll
      for (int h = 0; h < E / 2 / VE; ++h) {
        const Vec<R, VE> part = ldg<R, VE>(values + (int64_t)i * (E / 2) + h * VE);
#pragma unroll
        for (int e = 0; e < VE; ++e) v[k].v[h * VE + e] = part.v[e];
      }
    }
  }
  bool bad = false;
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const uint32_t i = i0 + k * kBlock;
    const uint32_t bits = m[k];
    uint32_t n = bits - ((bits >> 1) & 0x55555555u);
    n = (n & 0x33333333u) + ((n >> 2) & 0x33333333u);  // set bits per group of 4
    bad |= i < n_items && n != (0x22222222u & kAll);
    Vec<R, E> o;
    if constexpr (sizeof(R) == 4) {
#pragma unroll
      for (int g = 0; g < E / 4; ++g) {
        const uint32_t gm = (bits >> (4 * g)) & 15u;
        const R a = v[k].v[2 * g], b = v[k].v[2 * g + 1];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const bool keep = (gm >> q) & 1u, second = (gm & ((1u << q) - 1u)) != 0;
          o.v[4 * g + q] = keep ? (second ? b : a) : (R)0;
        }
      }
    } else {
      // 16 bytes out of 8: one v_perm_b32 per output word
      const Vec<uint32_t, 2> vw = __builtin_bit_cast(Vec<uint32_t, 2>, v[k]);
      Vec<uint32_t, 4> ow;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        // one-byte elements: word w is group w, its pair in half (w & 1) of values word w / 2;
        // two-byte elements: word w is half (w & 1) of group w / 2, whose pair is values word w / 2
        const uint32_t gm = (bits >> (sizeof(R) == 1 ? 4 * w : 4 * (w / 2))) & 15u;
        ow.v[w] = __builtin_amdgcn_perm(0u, vw.v[w / 2], lut[gm + 16 * (w & 1)]);
      }
      o = __builtin_bit_cast(Vec<R, E>, ow);
    }
    if (i < n_items) {
#pragma unroll
      for (int h = 0; h < E / VE; ++h) {
        Vec<R, VE> part;
#pragma unroll
        for (int e = 0; e < VE; ++e) part.v[e] = o.v[h * VE + e];
        stg_nt<R, VE>(out + (int64_t)i * E + h * VE, part);
      }
    }
  }
  s24_report(t.slot, j, bad);
}

constexpr int kS24RepairGrid = 32;

template <typename R>
__global__ void __launch_bounds__(kBlock) sparse24_repair_kernel(S24Table t) {
  const uint32_t todo = s24_bad_jobs(t.slot);
  if (todo == 0) return;
  __shared__ int scan_s[kWaves];
  __shared__ int64_t red[kWaves];
  __shared__ R stage[kBlock * 8];
  for (int q = 0; q < kMaxJobs; ++q)
    if ((todo >> q) & 1u) s24_redo_job<R>(t.job[q], scan_s, red, stage);
  s24_repair_done(t.slot);
}

// 2:4 decompression of int8 / fp8 codes and their dequantization in one pass: what
// ModelCompressor.decompress does to a weight that is both 2:4 sparse and quantized
// (the sparse compressor first, sparse_24_bitmask.py:206-224, then dequantize on the
// dense codes, naive_quantized.py:116-140), without the dense code tensor in between:
// 1/2 + 1/8 + 2 bytes per element of a bf16 weight instead of 1 5/8 + 3.  A lane takes
// one bitmask byte and its 4 codes and stores 8 dequantized elements (one scale: rows
// are multiples of 8 elements); a pruned position holds code 0, as it does in the dense
// code tensor.  Verdicts as in sparse24_scatter_kernel.
#ifndef CTMI_S24_DQ_U
#define CTMI_S24_DQ_U 8
#endif
constexpr int kS24DqU = CTMI_S24_DQ_U;

template <typename FT, int QK, bool HAS_ZP>
__device__ __forceinline__ Vec<typename FT::raw, 8> dequant_codes8(const Vec<uint8_t, 8>& codes,
                                                                   typename FT::raw sraw,
                                                                   uint8_t zraw) {
  constexpr int kIn = QK == 0 ? kKindI8 : kKindF8;
  Vec<typename FT::raw, 8> unused_f, o;
  Vec<uint8_t, 8> unused_c;
  float z = 0.0f;
  if constexpr (HAS_ZP) z = QK == 0 ? (float)(int8_t)zraw : f8e4m3_to_f32(zraw);
  qdq_vec8<FT, kIn, kKindFloat, QK, HAS_ZP>(unused_f, codes, FT::to_f32(sraw), z, 0.0f, 0.0f, &o,
                                            &unused_c);
  return o;
}

template <typename FT, int QK, bool HAS_ZP>
__global__ void __launch_bounds__(kBlock)
sparse24_scatter_dequant_kernel(const uint8_t* __restrict__ values,
                                const uint8_t* __restrict__ bitmask,
                                const typename FT::raw* __restrict__ scale,
                                const uint8_t* __restrict__ zp, typename FT::raw* __restrict__ out,
                                int64_t n_items, VecGeom g, uint32_t slot) {
  using FR = typename FT::raw;
  constexpr int U = kS24DqU;
  __shared__ uint32_t lut[32];
  if (threadIdx.x < 32) lut[threadIdx.x] = s24_selector<1>((int)threadIdx.x);
  __syncthreads();
  const int64_t i0 = (int64_t)blockIdx.x * (kBlock * U) + threadIdx.x;
  uint8_t m[U], zraw[U];
  uint32_t v[U];
  FR sraw[U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    int64_t i = i0 + k * kBlock;
    if (i >= n_items) i = n_items - 1;  // past the end: re-read the last item (not stored)
    const uint32_t si = scale_index((uint32_t)i, g);
    m[k] = bitmask[i];
    v[k] = reinterpret_cast<const uint32_t*>(values)[i];
    sraw[k] = scale[si];
    zraw[k] = 0;
    if constexpr (HAS_ZP) zraw[k] = zp[si];
  }
  bool bad = false;
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t i = i0 + k * kBlock;
    const uint32_t bits = m[k];
    uint32_t n = bits - ((bits >> 1) & 0x55u);
    n = (n & 0x33u) + ((n >> 2) & 0x33u);  // set bits per group of 4
    bad |= i < n_items && n != 0x22u;
    Vec<uint32_t, 2> cw;  // 8 codes out of 4: one v_perm_b32 per group
#pragma unroll
    for (int q = 0; q < 2; ++q)
      cw.v[q] = __builtin_amdgcn_perm(0u, v[k], lut[((bits >> (4 * q)) & 15u) + 16 * q]);
    const Vec<uint8_t, 8> codes = __builtin_bit_cast(Vec<uint8_t, 8>, cw);
    const Vec<FR, 8> o = dequant_codes8<FT, QK, HAS_ZP>(codes, sraw[k], zraw[k]);
    if (i < n_items) stg_nt<FR, 8>(out + i * 8, o);
  }
  s24_report(slot, 0, bad);
}

// ... and what sparse24_repair_kernel is to sparse24_scatter_kernel: nothing for a 2:4
// bitmask, otherwise the general scatter of the codes, dequantized as they are placed.
template <typename FT, int QK, bool HAS_ZP>
__global__ void __launch_bounds__(kBlock)
sparse24_repair_dequant_kernel(const uint8_t* __restrict__ values, int64_t nvalues,
                               const uint8_t* __restrict__ bitmask,
                               const typename FT::raw* __restrict__ scale,
                               const uint8_t* __restrict__ zp, typename FT::raw* __restrict__ out,
                               int64_t rows, int64_t pc, VecGeom g, uint32_t slot) {
  using FR = typename FT::raw;
  if (s24_bad_jobs(slot) == 0) return;
  __shared__ int scan_s[kWaves];
  __shared__ int64_t red[kWaves];
  __shared__ uint8_t stage[kBlock * 8];
  int64_t src = 0, counted = 0;  // set bits in rows [0, counted)
  for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
    int64_t c = 0;
    for (int64_t b = counted * pc + threadIdx.x; b < r * pc; b += kBlock) c += __popc((uint32_t)bitmask[b]);
    src += block_sum(c, red);
    scatter_row_to<uint8_t>(values, nvalues, bitmask + r * pc, src, pc, 0xffu, scan_s, stage,
                            [&](int64_t b, const Vec<uint8_t, 8>& codes) {
                              const int64_t i = r * pc + b;
                              const uint32_t si = scale_index((uint32_t)i, g);
                              uint8_t zraw = 0;
                              if constexpr (HAS_ZP) zraw = zp[si];
                              stg<FR, 8>(out + i * 8,
                                         dequant_codes8<FT, QK, HAS_ZP>(codes, scale[si], zraw));
                            });
    counted = r + 1;
  }
  s24_repair_done(slot);
}

// sparse24_scatter_dequant_kernel / sparse24_repair_dequant_kernel for the weights of a
// QS24Table: a workgroup finds its weight in the table's head, a malformed bitmask sets the
// weight's bit in the launch's verdict word, the kernel behind redoes the weights named there.
template <typename FT, int QK, bool HAS_ZP, bool FLAT>
__global__ void __launch_bounds__(kBlock) sparse24_scatter_dequant_chain_kernel(const QS24Table t) {
  using FR = typename FT::raw;
  constexpr int U = kS24DqU;
  __shared__ uint32_t lut[32];
  if (threadIdx.x < 32) lut[threadIdx.x] = s24_selector<1>((int)threadIdx.x);
  __syncthreads();
  uint32_t local, n_items;
  const uint32_t ji = find_job_index(blockIdx.x, &local, &n_items);
  const ChainJob job = t.job[ji];
  const uint8_t* __restrict__ bitmask = t.bitmask[ji];
  const uint8_t* __restrict__ values = static_cast<const uint8_t*>(job.src);
  const FR* __restrict__ scale = static_cast<const FR*>(job.scale);
  const uint8_t* __restrict__ zp = reinterpret_cast<const uint8_t*>(job.zp);
  FR* __restrict__ out = static_cast<FR*>(job.dst);
  const uint32_t i0 = local * (kBlock * U) + threadIdx.x;
  uint8_t m[U], zraw[U];
  uint32_t v[U];
  FR sraw[U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    uint32_t i = i0 + k * kBlock;
    if (i >= n_items) i = n_items - 1;  // past the end: re-read the last item (not stored)
    const uint32_t si = chain_scale_index<FLAT>(i, job);
    m[k] = bitmask[i];
    v[k] = reinterpret_cast<const uint32_t*>(values)[i];
    sraw[k] = scale[si];
    zraw[k] = 0;
    if constexpr (HAS_ZP) zraw[k] = zp[si];
  }
  bool bad = false;
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const uint32_t i = i0 + k * kBlock;
    const uint32_t bits = m[k];
    uint32_t n = bits - ((bits >> 1) & 0x55u);
    n = (n & 0x33u) + ((n >> 2) & 0x33u);  // set bits per group of 4
    bad |= i < n_items && n != 0x22u;
    Vec<uint32_t, 2> cw;  // 8 codes out of 4: one v_perm_b32 per group
#pragma unroll
    for (int q = 0; q < 2; ++q)
      cw.v[q] = __builtin_amdgcn_perm(0u, v[k], lut[((bits >> (4 * q)) & 15u) + 16 * q]);
    const Vec<uint8_t, 8> codes = __builtin_bit_cast(Vec<uint8_t, 8>, cw);
    const Vec<FR, 8> o = dequant_codes8<FT, QK, HAS_ZP>(codes, sraw[k], zraw[k]);
    if (i < n_items) stg_nt<FR, 8>(out + (int64_t)i * 8, o);
  }
  s24_report(t.slot, ji, bad);
}

template <typename FT, int QK, bool HAS_ZP, bool FLAT>
__global__ void __launch_bounds__(kBlock) sparse24_repair_dequant_chain_kernel(const QS24Table t) {
  using FR = typename FT::raw;
  const uint32_t todo = s24_bad_jobs(t.slot);
  if (todo == 0) return;
  __shared__ int scan_s[kWaves];
  __shared__ int64_t red[kWaves];
  __shared__ uint8_t stage[kBlock * 8];
  for (int q = 0; q < kMaxJobs; ++q) {
    if (!((todo >> q) & 1u)) continue;
    const ChainJob job = t.job[q];
    const uint8_t* bitmask = t.bitmask[q];
    const uint8_t* values = static_cast<const uint8_t*>(job.src);
    const FR* scale = static_cast<const FR*>(job.scale);
    const uint8_t* zp = reinterpret_cast<const uint8_t*>(job.zp);
    FR* out = static_cast<FR*>(job.dst);
    const int64_t rows = t.rows[q], pc = (int64_t)t.n_items[q] / rows, nvalues = (int64_t)t.n_items[q] * 4;
    int64_t src = 0, counted = 0;  // set bits in rows [0, counted)
    for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
      int64_t c = 0;
      for (int64_t b = counted * pc + threadIdx.x; b < r * pc; b += kBlock) c += __popc((uint32_t)bitmask[b]);
      src += block_sum(c, red);
      scatter_row_to<uint8_t>(values, nvalues, bitmask + r * pc, src, pc, 0xffu, scan_s, stage,
                              [&](int64_t b, const Vec<uint8_t, 8>& codes) {
                                const int64_t i = r * pc + b;
                                const uint32_t si = chain_scale_index<FLAT>((uint32_t)i, job);
                                uint8_t zraw = 0;
                                if constexpr (HAS_ZP) zraw = zp[si];
                                stg<FR, 8>(out + i * 8,
                                           dequant_codes8<FT, QK, HAS_ZP>(codes, scale[si], zraw));
                              });
      counted = r + 1;
    }
  }
  s24_repair_done(t.slot);
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

// Keep masks of the N/4 groups of one work item (group q in bits [4q, 4q+4)).
// A group with exactly two keys above zero (what a 2:4-pruned tensor holds
// nearly everywhere) keeps those two whatever order torch.topk gives the rest;
// only when some lane of the wavefront meets another kind of group are the ties
// resolved through the comparison table (read from memory then: no per-workgroup
// copy of it for the common case).
template <typename R, int DT, int N>
__device__ __forceinline__ uint32_t keep_masks24(const Vec<R, N>& a) {
  constexpr bool kBytes = sizeof(R) == 1;  // int8 and float8 tensors, ranked through their int8 view
  static_assert(kBytes == (DT == CTMI_I8), "one-byte elements are ranked as int8");
  uint32_t keep = 0;
  bool clear = true;
  if constexpr (kBytes) {
    // a group is one 32-bit word: which of its bytes are neither 0x00 nor 0x80 (abs(-128)
    // stays -128 in int8 and ranks below zero), and the four flags gathered into four bits
    const Vec<uint32_t, N / 4> w = __builtin_bit_cast(Vec<uint32_t, N / 4>, a);
#pragma unroll
    for (int q = 0; q < N / 4; ++q) {
      const uint32_t t = w.v[q] & 0x7F7F7F7Fu;
      const uint32_t nz = ((t + 0x7F7F7F7Fu) >> 7) & 0x01010101u;
      clear &= __popc(nz) == 2;
      keep |= ((nz | (nz >> 7) | (nz >> 14) | (nz >> 21)) & 15u) << (4 * q);
    }
    if (wave_all(clear)) return keep;
  }
  uint32_t keys[N];
#pragma unroll
  for (int i = 0; i < N; ++i) keys[i] = key24<DT>(a.v[i]);
  if constexpr (!kBytes) {
#pragma unroll
    for (int q = 0; q < N / 4; ++q) {
      uint32_t pos = 0;
#pragma unroll
      for (int j = 0; j < 4; ++j) pos |= (keys[4 * q + j] != 0 ? 1u : 0u) << j;
      clear &= __popc(pos) == 2;
      keep |= pos << (4 * q);
    }
    if (wave_all(clear)) return keep;
  }
  keep = 0;
#pragma unroll
  for (int q = 0; q < N / 4; ++q)
    keep |= keep24(keys[4 * q], keys[4 * q + 1], keys[4 * q + 2], keys[4 * q + 3], kTopk24LutDev)
            << (4 * q);
  return keep;
}

// get_24_bytemasks: one bool per element; work item = 16 elements (numel % 16 == 0)
template <typename R, int DT>
__global__ void __launch_bounds__(kBlock)
bytemask24_vec_kernel(const R* __restrict__ x, uint8_t* __restrict__ mask, int64_t nitems) {
  constexpr int N = 16, U = 2;
  const int64_t i0 = (int64_t)blockIdx.x * (kBlock * U) + threadIdx.x;
  Vec<R, N> a[U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    int64_t i = i0 + k * kBlock;
    if (i >= nitems) i = nitems - 1;  // re-read, not stored
    if constexpr (sizeof(R) * N == 16) {
      a[k] = ldg_nt<R, N>(x + i * N);
    } else {
#pragma unroll
      for (int h = 0; h < (int)(sizeof(R) * N / 16); ++h) {
        constexpr int PER = 16 / sizeof(R);
        const Vec<R, PER> part = ldg_nt<R, PER>(x + i * N + h * PER);
#pragma unroll
        for (int j = 0; j < PER; ++j) a[k].v[h * PER + j] = part.v[j];
      }
    }
  }
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t i = i0 + k * kBlock;
    const uint32_t keep = keep_masks24<R, DT, N>(a[k]);
    Vec<uint32_t, N / 4> o;  // four bool bytes per group
#pragma unroll
    for (int q = 0; q < N / 4; ++q) {
      const uint32_t kq = (keep >> (4 * q)) & 15u;
      o.v[q] = (kq | (kq << 7) | (kq << 14) | (kq << 21)) & 0x01010101u;
    }
    if (i < nitems) stg_nt<uint32_t, N / 4>(reinterpret_cast<uint32_t*>(mask + i * N), o);
  }
}

template <typename R, int DT>
__global__ void __launch_bounds__(kBlock)
bytemask24_kernel(const R* __restrict__ x, uint8_t* __restrict__ mask, int64_t ngroups) {
  for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < ngroups;
       g += (int64_t)gridDim.x * blockDim.x) {
    const R* p = x + g * 4;
    const uint32_t keep = keep24(key24<DT>(p[0]), key24<DT>(p[1]), key24<DT>(p[2]),
                                 key24<DT>(p[3]), kTopk24LutDev);
    uint32_t w = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) w |= ((keep >> j) & 1u) << (8 * j);
    *reinterpret_cast<uint32_t*>(mask + g * 4) = w;
  }
}

// Fused 2:4 compress, cols % 8 == 0.  Work item = N elements (N/4 groups):
// one 16-byte load, N/2 survivors stored as one vector, N/8 bitmask bytes.
// One workgroup per chunk of items, every load issued before the first use.
// item i (N neighbouring elements): the 2 survivors of every group of 4, in column
// order, and the item's bitmask bytes
template <typename R, int DT, int N>
__device__ __forceinline__ void store_survivors24_any(const Vec<R, N>& a, R* __restrict__ values,
                                                      uint8_t* __restrict__ bitmask, int64_t i,
                                                      bool keep_item) {
  const uint32_t keep_all = keep_masks24<R, DT, N>(a);
  Vec<R, N / 2> o;
  Vec<uint8_t, N / 8> m;
#pragma unroll
  for (int q = 0; q < N / 4; ++q) {
    const uint32_t keep = (keep_all >> (4 * q)) & 15u;
    // the two survivors in column order: the lower one is element 0, 1 or 2,
    // the upper one element 1, 2 or 3
    const R e0 = a.v[4 * q], e1 = a.v[4 * q + 1], e2 = a.v[4 * q + 2], e3 = a.v[4 * q + 3];
    o.v[2 * q] = (keep & 1u) ? e0 : ((keep & 2u) ? e1 : e2);
    o.v[2 * q + 1] = (keep & 8u) ? e3 : ((keep & 4u) ? e2 : e1);
  }
#pragma unroll
  for (int bq = 0; bq < N / 8; ++bq) m.v[bq] = (uint8_t)((keep_all >> (8 * bq)) & 0xffu);
  if (keep_item) {
    stg_nt<R, N / 2>(values + i * (N / 2), o);
    stg_nt<uint8_t, N / 8>(bitmask + i * (N / 8), m);
  }
}

// One-byte elements (int8 and float8 tensors), four groups or two to a lane: a group is
// one 32-bit word, and the survivors of two groups are picked by one byte permute.
template <int N>
__device__ __forceinline__ void store_survivors24_bytes(const Vec<uint8_t, N>& a,
                                                        uint8_t* __restrict__ values,
                                                        uint8_t* __restrict__ bitmask, int64_t i,
                                                        bool keep_item) {
  constexpr int G = N / 4;
  static_assert(G % 2 == 0, "pairs of groups");
  const uint32_t keep_all = keep_masks24<uint8_t, CTMI_I8, N>(a);  // two bits set in every group
  const Vec<uint32_t, G> w = __builtin_bit_cast(Vec<uint32_t, G>, a);
  Vec<uint32_t, G / 2> o;
#pragma unroll
  for (int p = 0; p < G / 2; ++p) {
    const uint32_t k0 = (keep_all >> (8 * p)) & 15u, k1 = (keep_all >> (8 * p + 4)) & 15u;
    // byte numbers of the lower and the upper survivor of either group, in the 8 bytes
    // {second word, first word}
    const uint32_t sel = (uint32_t)__builtin_ctz(k0) | ((31u - (uint32_t)__clz(k0)) << 8) |
                         ((4u + (uint32_t)__builtin_ctz(k1)) << 16) |
                         ((35u - (uint32_t)__clz(k1)) << 24);
    o.v[p] = __builtin_amdgcn_perm(w.v[2 * p + 1], w.v[2 * p], sel);
  }
  Vec<uint8_t, N / 8> m;
#pragma unroll
  for (int bq = 0; bq < N / 8; ++bq) m.v[bq] = (uint8_t)((keep_all >> (8 * bq)) & 0xffu);
  if (keep_item) {
    stg_nt<uint32_t, G / 2>(reinterpret_cast<uint32_t*>(values + i * (N / 2)), o);
    stg_nt<uint8_t, N / 8>(bitmask + i * (N / 8), m);
  }
}

template <typename R, int DT, int N>
__device__ __forceinline__ void store_survivors24(const Vec<R, N>& a, R* __restrict__ values,
                                                  uint8_t* __restrict__ bitmask, int64_t i,
                                                  bool keep_item) {
  if constexpr (sizeof(R) == 1 && DT == CTMI_I8 && N % 8 == 0)
    store_survivors24_bytes<N>(a, values, bitmask, i, keep_item);
  else
    store_survivors24_any<R, DT, N>(a, values, bitmask, i, keep_item);
}

template <typename R, int DT, int N>
__global__ void __launch_bounds__(kBlock)
sparse24_compress_kernel(const R* __restrict__ x, R* __restrict__ values,
                         uint8_t* __restrict__ bitmask, int64_t nitems) {
  constexpr int U = kS24U;
  const int64_t i0 = (int64_t)blockIdx.x * (kBlock * U) + threadIdx.x;
  Vec<R, N> a[U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t i = i0 + k * kBlock;
    a[k] = ldg<R, N>(x + (i < nitems ? i : nitems - 1) * N);  // past the end: re-read, not stored
  }
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t i = i0 + k * kBlock;
    store_survivors24<R, DT, N>(a[k], values, bitmask, i, i < nitems);
  }
}

// the same for up to kMaxJobs tensors of one dtype
struct S24CompressJob {
  const void* x;
  void* values;
  uint8_t* bitmask;
};
struct S24CompressTable {  // the kernel's only argument: find_job_index reads its head
  uint32_t chunk_end[kMaxJobs];
  uint32_t n_items[kMaxJobs];
  S24CompressJob job[kMaxJobs];
};
static_assert(offsetof(S24CompressTable, n_items) == 32, "find_job_index");

template <typename R, int DT, int N>
__global__ void __launch_bounds__(kBlock) sparse24_compress_chain_kernel(S24CompressTable t) {
  constexpr int U = kS24U;
  uint32_t local, nitems;
  const S24CompressJob job = t.job[find_job_index(blockIdx.x, &local, &nitems)];
  const R* __restrict__ x = static_cast<const R*>(job.x);
  const int64_t i0 = (int64_t)local * (kBlock * U) + threadIdx.x;
  Vec<R, N> a[U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t i = i0 + k * kBlock;
    a[k] = ldg<R, N>(x + (i < nitems ? i : nitems - 1) * N);  // past the end: re-read, not stored
  }
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t i = i0 + k * kBlock;
    store_survivors24<R, DT, N>(a[k], static_cast<R*>(job.values), job.bitmask, i, i < nitems);
  }
}

// Quantization to fp8 / int8 codes and 2:4 compression of the codes in one pass: what
// ModelCompressor.compress does to a weight that is both quantized (float- / int- /
// naive-quantized, naive_quantized.py:79-114) and 2:4 sparse (sparse_24_bitmask.py:
// 162-203), without the dense code tensor in between: 2 + 1/2 + 1/8 bytes per element
// instead of 3 + 1 5/8.  A lane quantizes 8 neighbouring elements (one 16-byte load,
// one scale: rows are multiples of 8 elements) and keeps 2 of every 4 codes by the rule
// of get_24_bytemasks on the codes' int8 view.
template <typename FT, int QK, bool HAS_ZP>
__global__ void __launch_bounds__(kBlock)
quant_sparse24_compress_kernel(const typename FT::raw* __restrict__ x,
                               const typename FT::raw* __restrict__ scale,
                               const uint8_t* __restrict__ zp, uint8_t* __restrict__ values,
                               uint8_t* __restrict__ bitmask, int64_t nitems, VecGeom g, float qmin,
                               float qmax) {
  using FR = typename FT::raw;
  constexpr int U = 4;
  constexpr int kOut = QK == 0 ? kKindI8 : kKindF8;
  const int64_t i0 = (int64_t)blockIdx.x * (kBlock * U) + threadIdx.x;
  Vec<FR, 8> a[U];
  FR sraw[U];
  uint8_t zraw[U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t i = i0 + k * kBlock;
    const int64_t at = i < nitems ? i : nitems - 1;  // past the end: re-read, not stored
    const uint32_t si = scale_index((uint32_t)at, g);
    a[k] = ldg_nt<FR, 8>(x + at * 8);
    sraw[k] = scale[si];
    if constexpr (HAS_ZP) zraw[k] = zp[si];
  }
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t i = i0 + k * kBlock;
    Vec<FR, 8> unused_f;
    Vec<uint8_t, 8> codes, unused_c;
    float z = 0.0f;  // the zero point as the reference adds it (zero_point.to(x.dtype))
    if constexpr (HAS_ZP) z = QK == 0 ? (float)(int8_t)zraw[k] : f8e4m3_to_f32(zraw[k]);
    qdq_vec8<FT, kKindFloat, kOut, QK, HAS_ZP>(a[k], unused_c, FT::to_f32(sraw[k]), z, qmin, qmax,
                                               &unused_f, &codes);
    store_survivors24<uint8_t, CTMI_I8, 8>(codes, values, bitmask, i, i < nitems);
  }
}

// ... for the weights of a QS24Table
template <typename FT, int QK, bool HAS_ZP, bool FLAT>
__global__ void __launch_bounds__(kBlock) quant_sparse24_compress_chain_kernel(const QS24Table t) {
  using FR = typename FT::raw;
  constexpr int U = 4;
  constexpr int kOut = QK == 0 ? kKindI8 : kKindF8;
  uint32_t local, nitems;
  const uint32_t ji = find_job_index(blockIdx.x, &local, &nitems);
  const ChainJob job = t.job[ji];
  uint8_t* __restrict__ bitmask = t.bitmask[ji];
  const FR* __restrict__ x = static_cast<const FR*>(job.src);
  const FR* __restrict__ scale = static_cast<const FR*>(job.scale);
  const uint8_t* __restrict__ zp = reinterpret_cast<const uint8_t*>(job.zp);
  uint8_t* __restrict__ values = static_cast<uint8_t*>(job.dst);
  const uint32_t i0 = local * (kBlock * U) + threadIdx.x;
  Vec<FR, 8> a[U];
  FR sraw[U];
  uint8_t zraw[U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const uint32_t i = i0 + k * kBlock;
    const uint32_t at = i < nitems ? i : nitems - 1;  // past the end: re-read, not stored
    const uint32_t si = chain_scale_index<FLAT>(at, job);
    a[k] = ldg_nt<FR, 8>(x + (int64_t)at * 8);
    sraw[k] = scale[si];
    if constexpr (HAS_ZP) zraw[k] = zp[si];
  }
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const uint32_t i = i0 + k * kBlock;
    Vec<FR, 8> unused_f;
    Vec<uint8_t, 8> codes, unused_c;
    float z = 0.0f;  // the zero point as the reference adds it (zero_point.to(x.dtype))
    if constexpr (HAS_ZP) z = QK == 0 ? (float)(int8_t)zraw[k] : f8e4m3_to_f32(zraw[k]);
    qdq_vec8<FT, kKindFloat, kOut, QK, HAS_ZP>(a[k], unused_c, FT::to_f32(sraw[k]), z, t.qmin, t.qmax,
                                               &unused_f, &codes);
    store_survivors24<uint8_t, CTMI_I8, 8>(codes, values, bitmask, (int64_t)i, i < nitems);
  }
}

// Any shape with numel % 4 == 0 (groups may straddle rows): survivors per group.
template <typename R, int DT>
__global__ void __launch_bounds__(kBlock)
sparse24_values_kernel(const R* __restrict__ x, R* __restrict__ values, int64_t ngroups) {
  for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < ngroups;
       g += (int64_t)gridDim.x * blockDim.x) {
    const R* p = x + g * 4;
    const uint32_t keep = keep24(key24<DT>(p[0]), key24<DT>(p[1]), key24<DT>(p[2]),
                                 key24<DT>(p[3]), kTopk24LutDev);
    values[2 * g] = p[__ffs(keep) - 1];
    values[2 * g + 1] = p[31 - __clz(keep)];
  }
}

// ... and the row-structured bitmask for that case: one thread per bitmask byte
template <typename R, int DT>
__global__ void __launch_bounds__(kBlock)
sparse24_bitmask_kernel(const R* __restrict__ x, uint8_t* __restrict__ bitmask, int64_t rows,
                        int64_t cols, int64_t pc) {
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
                                   key24<DT>(p[3]), kTopk24LutDev);
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
  const int64_t numel = rows * cols;
  if (cols % 8 == 0 && numel % 16 == 0 && (uintptr_t)mask % 16 == 0 && (uintptr_t)packed % 2 == 0 &&
      numel / 16 < (1ll << 40)) {
    const int64_t n_items = numel / 16;
    hipLaunchKernelGGL(pack_bitmasks_flat_kernel, (unsigned)cdiv(n_items, kBlock * kPackU), kBlock, 0,
                       (hipStream_t)stream, mask, (uint16_t*)packed, n_items);
    return check_launch("ctmi_pack_bitmasks");
  }
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
  const int64_t numel = rows * cols;
  if (cols % 8 == 0 && numel % 16 == 0 && (uintptr_t)mask % 16 == 0 && (uintptr_t)packed % 2 == 0 &&
      numel / 16 < (1ll << 40)) {
    const int64_t n_items = numel / 16;
    hipLaunchKernelGGL(unpack_bitmasks_flat_kernel, (unsigned)cdiv(n_items, kBlock * kPackU), kBlock,
                       0, (hipStream_t)stream, (const uint16_t*)packed, mask, n_items);
    return check_launch("ctmi_unpack_bitmasks");
  }
  hipLaunchKernelGGL(unpack_bitmasks_kernel, grid_for(rows * pc, kBlock), kBlock, 0,
                     (hipStream_t)stream, packed, mask, rows, cols, pc);
  return check_launch("ctmi_unpack_bitmasks");
}

// per-row counts and offsets for the row kernels, per-tile ones for the tile kernels
extern "C" int64_t ctmi_bitmask_tmp_bytes(int64_t rows, int64_t cols) {
  const int64_t r = rows < 1 ? 1 : rows, c = cols < 1 ? 1 : cols;
  return 16 * r + 16 * cdiv(r * c, kTileElems) + 32;
}

// what the general kernels need (the 2:4 streaming kernel needs none)
extern "C" int64_t ctmi_sparse24_tmp_bytes(int64_t rows, int64_t cols, int32_t elem_size) {
  (void)elem_size;
  return ctmi_bitmask_tmp_bytes(rows, cols);
}

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
  hipLaunchKernelGGL(row_offsets_kernel, 1, kScanThreads, 0, st, counts, row_offsets, total_nnz, rows);
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
  const bool whole = cols % 8 == 0 && (uintptr_t)x % (8 * (size_t)elem_size) == 0 &&
                     (uintptr_t)values % (size_t)elem_size == 0;
#define CTMI_COMPACT(R)                                                                          \
  if (whole)                                                                                     \
    hipLaunchKernelGGL(bitmask_compact_rows_kernel<R>, grid, kBlock, 0, st, (const R*)x, bitmask, \
                       row_offsets, (R*)values, rows, cols, pc);                                 \
  else                                                                                           \
    hipLaunchKernelGGL(bitmask_compact_kernel<R>, grid, kBlock, 0, st, (const R*)x, bitmask,     \
                       row_offsets, (R*)values, rows, cols, pc)
  if (elem_size == 1) { CTMI_COMPACT(uint8_t); }
  else if (elem_size == 2) { CTMI_COMPACT(uint16_t); }
  else { CTMI_COMPACT(uint32_t); }
#undef CTMI_COMPACT
  return check_launch("ctmi_bitmask_compact");
}

// argument checks of the scatter entry points (no HIP call)
static int scatter_check(const void* values, int64_t nvalues, int32_t elem_size,
                         const uint8_t* bitmask, void* out, int64_t rows, int64_t cols) {
  CTMI_REQUIRE(rows >= 0 && cols >= 0, CTMI_ERR_VALUE, "negative shape");
  int rc = check_elem(elem_size);
  if (rc) return rc;
  if (rows == 0 || cols == 0) return CTMI_OK;
  CTMI_REQUIRE(bitmask && out, CTMI_ERR_VALUE, "NULL tensor pointer");
  CTMI_REQUIRE(nvalues >= 0 && (values || nvalues == 0), CTMI_ERR_VALUE, "bad values buffer");
  return CTMI_OK;
}

// what sparse24_scatter_kernel needs of a tensor: half as many values as elements, rows of
// whole bitmask bytes, whole work items, aligned accesses
static bool s24_streamable(const void* values, int64_t nvalues, int32_t elem_size,
                           const uint8_t* bitmask, const void* out, int64_t rows, int64_t cols) {
  const int64_t numel = rows * cols;
  const int e24 = elem_size == 1 ? 16 : 8;
  return nvalues * 2 == numel && cols % 8 == 0 && numel % e24 == 0 && (uintptr_t)out % 16 == 0 &&
         (uintptr_t)values % 16 == 0 && (uintptr_t)bitmask % (e24 / 8) == 0 &&
         numel / e24 < (1ll << 31);
}

// up to kMaxJobs streamable tensors of one element size in one launch
static void s24_launch(const S24Job* jobs, int n, int32_t elem_size, hipStream_t st) {
  S24Table t;
  const int e24 = elem_size == 1 ? 16 : 8;
  uint32_t total = 0;
  for (int k = 0; k < kMaxJobs; ++k) {
    if (k < n) {
      t.job[k] = jobs[k];
      t.n_items[k] = (uint32_t)(jobs[k].rows * jobs[k].cols / e24);
      total += (uint32_t)cdiv((int64_t)t.n_items[k], kBlock * kS24ScatterU);
      t.chunk_end[k] = total;
    } else {
      t.job[k] = S24Job{nullptr, nullptr, nullptr, 0, 0, 0};
      t.n_items[k] = 0;
      t.chunk_end[k] = 0xFFFFFFFFu;
    }
  }
  t.slot = s24_slot_of(st);
#define CTMI_24(R)                                                                \
  hipLaunchKernelGGL(sparse24_scatter_kernel<R>, total, kBlock, 0, st, t);        \
  hipLaunchKernelGGL(sparse24_repair_kernel<R>, kS24RepairGrid, kBlock, 0, st, t)
  if (elem_size == 1) { CTMI_24(uint8_t); }
  else if (elem_size == 2) { CTMI_24(uint16_t); }
  else { CTMI_24(uint32_t); }
#undef CTMI_24
}

static int scatter_entry(const void* values, int64_t nvalues, int32_t elem_size,
                         const uint8_t* bitmask, const int64_t* row_offsets, void* out, void* tmp,
                         int64_t rows, int64_t cols, void* stream, bool try_24, const char* what) {
  int rc = scatter_check(values, nvalues, elem_size, bitmask, out, rows, cols);
  if (rc) return rc;
  if (rows == 0 || cols == 0) return CTMI_OK;
  CTMI_REQUIRE(row_offsets || tmp, CTMI_ERR_VALUE, "row_offsets and tmp are both NULL");
  hipStream_t st = (hipStream_t)stream;
  const int64_t pc = cdiv(cols, 8);
  const int64_t numel = rows * cols;
  // exactly half as many values as elements, rows of whole bitmask bytes: the 2:4
  // streaming kernel (which also copes with a bitmask that turns out not to be 2:4)
  if (try_24 && s24_streamable(values, nvalues, elem_size, bitmask, out, rows, cols)) {
    S24Job job{values, bitmask, out, nvalues, rows, cols};
    s24_launch(&job, 1, elem_size, st);
    return check_launch(what);
  }
  if (tmp && cols % 8 == 0 && numel % 16 == 0 && (uintptr_t)out % 16 == 0 &&
      (uintptr_t)values % 16 == 0 && (uintptr_t)bitmask % 16 == 0 && (uintptr_t)tmp % 8 == 0 &&
      cdiv(numel, kTileElems) < (1ll << 31)) {
    // positions from the bitmask alone, as in the reference (sparse_bitmask.py:152-169)
    const int64_t ntiles = cdiv(numel, kTileElems);
    const int64_t ngroups = cdiv(ntiles, kGroupTiles);
    int64_t* counts = nullptr;
    int64_t* offs = nullptr;
    TileInfo* info = nullptr;
    int32_t* totals = nullptr;
    const bool grouped = ngroups <= kMaxGroups;
    if (grouped) {
      info = (TileInfo*)tmp;
      // set bits of each group, from the next 16-byte boundary (the scatter kernel reads
      // four totals per load); ctmi_bitmask_tmp_bytes leaves room for that and for the
      // round-up of the last four
      totals = (int32_t*)(((uintptr_t)(info + ntiles) + 15) & ~(uintptr_t)15);
      hipLaunchKernelGGL(tile_popcount_groups_kernel, (unsigned)ngroups, kGroupThreads, 0, st,
                         bitmask, rows * pc, info, totals, ntiles);
    } else {
      counts = (int64_t*)tmp;
      offs = counts + ntiles;
      hipLaunchKernelGGL(tile_popcount_kernel, (unsigned)cdiv(ntiles, kWaves), kBlock, 0, st,
                         bitmask, rows * pc, counts, ntiles);
      hipLaunchKernelGGL(row_offsets_kernel, 1, kScanThreads, 0, st, counts, offs,
                         (int64_t*)nullptr, ntiles);
    }
#define CTMI_TILES(R)                                                                              \
  if (grouped)                                                                                     \
    hipLaunchKernelGGL((bitmask_scatter_tiles_kernel<R, true, kScatterTiles>),                     \
                       (unsigned)cdiv(ntiles, kScatterTiles), kBlock, 0, st, (const R*)values,     \
                       nvalues, bitmask, counts, offs, info, totals, (R*)out, numel, ntiles);      \
  else                                                                                             \
    hipLaunchKernelGGL((bitmask_scatter_tiles_kernel<R, false, kScatterTiles>),                    \
                       (unsigned)cdiv(ntiles, kScatterTiles), kBlock, 0, st, (const R*)values,     \
                       nvalues, bitmask, counts, offs, info, totals, (R*)out, numel, ntiles)
    if (elem_size == 1) { CTMI_TILES(uint8_t); }
    else if (elem_size == 2) { CTMI_TILES(uint16_t); }
    else { CTMI_TILES(uint32_t); }
#undef CTMI_TILES
    return check_launch(what);
  }
  // any other shape: per-row counts, their prefix, one wavefront or workgroup per row
  const int grid = rows_grid(rows);
  if (!row_offsets) {
    int64_t* counts = (int64_t*)tmp;
    int64_t* offs = counts + rows;
    int64_t pop_grid = cdiv(rows, kWaves);
    if (pop_grid > (1 << 20)) pop_grid = 1 << 20;
    hipLaunchKernelGGL(bitmask_popcount_kernel, (unsigned)pop_grid, kBlock, 0, st, bitmask, counts,
                       rows, cols, pc);
    hipLaunchKernelGGL(row_offsets_kernel, 1, kScanThreads, 0, st, counts, offs, (int64_t*)nullptr,
                       rows);
    row_offsets = offs;
  }
#define CTMI_SCATTER(R)                                                                           \
  if (scatter_wave_ok<R>(values, bitmask, out, cols))                                             \
    hipLaunchKernelGGL(bitmask_scatter_wave_kernel<R>, (unsigned)wave_grid, kBlock, 0, st,        \
                       (const R*)values, nvalues, bitmask, row_offsets, (R*)out, rows, cols, pc); \
  else                                                                                            \
    hipLaunchKernelGGL(bitmask_scatter_kernel<R>, grid, kBlock, 0, st, (const R*)values, nvalues, \
                       bitmask, row_offsets, (R*)out, rows, cols, pc)
  int64_t wave_grid = cdiv(rows, kWaves);
  if (wave_grid > (1 << 24)) wave_grid = 1 << 24;
  if (elem_size == 1) { CTMI_SCATTER(uint8_t); }
  else if (elem_size == 2) { CTMI_SCATTER(uint16_t); }
  else { CTMI_SCATTER(uint32_t); }
#undef CTMI_SCATTER
  return check_launch(what);
}

extern "C" int ctmi_bitmask_decompress(const void* values, int64_t nvalues, int32_t elem_size,
                                       const uint8_t* bitmask, const int64_t* row_offsets,
                                       void* out, void* tmp, int64_t rows, int64_t cols,
                                       void* stream) {
  return scatter_entry(values, nvalues, elem_size, bitmask, row_offsets, out, tmp, rows, cols,
                       stream, false, "ctmi_bitmask_decompress");
}

// ---- ctmi_bitmask_decompress for callers that cannot allocate: the scratch of the
// scatter kernels (per-tile set-bit counts and group totals, or per-row counts and
// offsets) lives in this file-scope device array instead of a caller's buffer.
// Every GPU holds its own copy at its own address; host code reaches it only
// through the address hipGetSymbolAddress returns for the current device.
constexpr int64_t kStaticScratchBytes = 4ll << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxScratchDevices = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kMaxScratchDevices];  // per device, filled on first use

// device address of `scratch` on the current device
static int static_scratch(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return set_error(CTMI_ERR_HIP, "hipGetDevice: %s", hipGetErrorString(e));
  CTMI_REQUIRE(dev >= 0 && dev < kMaxScratchDevices, CTMI_ERR_UNSUPPORTED,
               "device index %d is beyond the %d devices the static scratch table holds", dev,
               kMaxScratchDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr)
      return set_error(CTMI_ERR_HIP, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return CTMI_OK;
}

extern "C" int64_t ctmi_bitmask_decompress_static_max_bytes(void) { return kStaticScratchBytes; }

extern "C" int ctmi_bitmask_decompress_static(const void* values, int64_t nvalues,
                                              int32_t elem_size, const uint8_t* bitmask, void* out,
                                              int64_t rows, int64_t cols, void* stream) {
  int rc = scatter_check(values, nvalues, elem_size, bitmask, out, rows, cols);
  if (rc) return rc;
  if (rows == 0 || cols == 0) return CTMI_OK;
  const int64_t need = ctmi_bitmask_tmp_bytes(rows, cols);
  CTMI_REQUIRE(need <= kStaticScratchBytes, CTMI_ERR_VALUE,
               "a [%lld, %lld] tensor needs %lld bytes of scratch, the static buffer holds %lld: "
               "use ctmi_bitmask_decompress with a caller-owned buffer",
               (long long)rows, (long long)cols, (long long)need, (long long)kStaticScratchBytes);
  void* tmp = nullptr;
  rc = static_scratch(&tmp);
  if (rc) return rc;
  // the kernels write every scratch word they later read (counts of all tiles or rows
  // of THIS call), so what an earlier call left behind needs no clearing
  return scatter_entry(values, nvalues, elem_size, bitmask, nullptr, out, tmp, rows, cols, stream,
                       false, "ctmi_bitmask_decompress_static");
}

extern "C" int ctmi_sparse24_decompress(const void* values, int64_t nvalues, int32_t elem_size,
                                        const uint8_t* bitmask, void* out, void* tmp, int64_t rows,
                                        int64_t cols, void* stream) {
  CTMI_REQUIRE(tmp != nullptr || rows == 0 || cols == 0, CTMI_ERR_VALUE, "tmp is NULL");
  return scatter_entry(values, nvalues, elem_size, bitmask, nullptr, out, tmp, rows, cols, stream,
                       true, "ctmi_sparse24_decompress");
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
  if (numel % 16 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)mask % 16 == 0) {
    const int64_t items = numel / 16;
    CTMI_DISPATCH_24(x_dtype, hipLaunchKernelGGL((bytemask24_vec_kernel<R, DT>),
                                                  (unsigned)cdiv(items, kBlock * 2), kBlock, 0, st,
                                                  (const R*)x, mask, items));
    return check_launch("ctmi_get_24_bytemasks");
  }
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
      hipLaunchKernelGGL((sparse24_compress_kernel<uint8_t, CTMI_I8, 16>), (unsigned)cdiv(items, kBlock * kS24U),
                         kBlock, 0, st, (const uint8_t*)x, (uint8_t*)values, bitmask, items);
    } else if (es == 2) {
      const int64_t items = n / 8;
      if (x_dtype == CTMI_BF16)
        hipLaunchKernelGGL((sparse24_compress_kernel<uint16_t, CTMI_BF16, 8>),
                           (unsigned)cdiv(items, kBlock * kS24U), kBlock, 0, st, (const uint16_t*)x,
                           (uint16_t*)values, bitmask, items);
      else
        hipLaunchKernelGGL((sparse24_compress_kernel<uint16_t, CTMI_F16, 8>),
                           (unsigned)cdiv(items, kBlock * kS24U), kBlock, 0, st, (const uint16_t*)x,
                           (uint16_t*)values, bitmask, items);
    } else {
      const int64_t items = n / 8;
      hipLaunchKernelGGL((sparse24_compress_kernel<uint32_t, CTMI_F32, 8>),
                         (unsigned)cdiv(items, kBlock * kS24U), kBlock, 0, st, (const uint32_t*)x,
                         (uint32_t*)values, bitmask, items);
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

extern "C" int ctmi_sparse24_compress_many(const ctmi_sparse24_job* jobs, int64_t n_jobs,
                                           int32_t x_dtype, void* stream) {
  CTMI_REQUIRE(n_jobs >= 0 && (jobs || n_jobs == 0), CTMI_ERR_VALUE, "bad job list");
  int rc = check_24_dtype(x_dtype);
  if (rc) return rc;
  const int es = dtype_size(x_dtype);
  const int per = es == 1 ? 16 : 8;  // elements per work item
  // everything is checked before anything is enqueued
  for (int64_t i = 0; i < n_jobs; ++i) {
    const ctmi_sparse24_job& j = jobs[i];
    CTMI_REQUIRE(j.rows >= 0 && j.cols >= 0, CTMI_ERR_VALUE, "job %lld: negative shape", (long long)i);
    if (j.rows == 0 || j.cols == 0) continue;
    CTMI_REQUIRE(j.dense && j.values && j.bitmask, CTMI_ERR_VALUE, "job %lld: NULL tensor pointer",
                 (long long)i);
    const int64_t n = j.rows * j.cols;
    CTMI_REQUIRE(j.cols % 8 == 0 && n % per == 0 && (uintptr_t)j.dense % (per * es) == 0 &&
                     (uintptr_t)j.values % (per * es / 2) == 0 && n / per < (1ll << 31),
                 CTMI_ERR_UNSUPPORTED,
                 "job %lld: the multi-tensor call takes rows of whole bitmask bytes and aligned "
                 "tensors; use ctmi_sparse24_compress for this one", (long long)i);
  }
  hipStream_t st = (hipStream_t)stream;
  S24CompressTable t;
  int filled = 0;
  uint32_t total = 0;
  bool any = false;
  auto flush = [&]() {
    for (int k = filled; k < kMaxJobs; ++k) {
      t.chunk_end[k] = 0xFFFFFFFFu;
      t.n_items[k] = 0;
      t.job[k] = S24CompressJob{nullptr, nullptr, nullptr};
    }
    if (es == 1)
      hipLaunchKernelGGL((sparse24_compress_chain_kernel<uint8_t, CTMI_I8, 16>), total, kBlock, 0, st, t);
    else if (x_dtype == CTMI_BF16)
      hipLaunchKernelGGL((sparse24_compress_chain_kernel<uint16_t, CTMI_BF16, 8>), total, kBlock, 0, st, t);
    else if (es == 2)
      hipLaunchKernelGGL((sparse24_compress_chain_kernel<uint16_t, CTMI_F16, 8>), total, kBlock, 0, st, t);
    else
      hipLaunchKernelGGL((sparse24_compress_chain_kernel<uint32_t, CTMI_F32, 8>), total, kBlock, 0, st, t);
    filled = 0;
    total = 0;
  };
  for (int64_t i = 0; i < n_jobs; ++i) {
    const ctmi_sparse24_job& j = jobs[i];
    if (j.rows == 0 || j.cols == 0) continue;
    any = true;
    t.job[filled] = S24CompressJob{j.dense, j.values, j.bitmask};
    t.n_items[filled] = (uint32_t)(j.rows * j.cols / per);
    total += (uint32_t)cdiv((int64_t)t.n_items[filled], kBlock * kS24U);
    t.chunk_end[filled] = total;
    if (++filled == kMaxJobs) flush();
  }
  if (!any) return CTMI_OK;
  if (filled) flush();
  return check_launch("ctmi_sparse24_compress_many");
}

extern "C" int ctmi_sparse24_decompress_many(const ctmi_sparse24_job* jobs, int64_t n_jobs,
                                             int32_t elem_size, void* stream) {
  CTMI_REQUIRE(n_jobs >= 0 && (jobs || n_jobs == 0), CTMI_ERR_VALUE, "bad job list");
  int rc = check_elem(elem_size);
  if (rc) return rc;
  for (int64_t i = 0; i < n_jobs; ++i) {
    const ctmi_sparse24_job& j = jobs[i];
    rc = scatter_check(j.values, j.nvalues, elem_size, j.bitmask, j.dense, j.rows, j.cols);
    if (rc) return rc;
    if (j.rows == 0 || j.cols == 0) continue;
    CTMI_REQUIRE(s24_streamable(j.values, j.nvalues, elem_size, j.bitmask, j.dense, j.rows, j.cols),
                 CTMI_ERR_UNSUPPORTED,
                 "job %lld: the multi-tensor call takes tensors with rows * cols / 2 values, rows "
                 "of whole bitmask bytes and aligned buffers; use ctmi_sparse24_decompress for "
                 "this one", (long long)i);
  }
  hipStream_t st = (hipStream_t)stream;
  S24Job batch[kMaxJobs];
  int filled = 0;
  bool any = false;
  for (int64_t i = 0; i < n_jobs; ++i) {
    const ctmi_sparse24_job& j = jobs[i];
    if (j.rows == 0 || j.cols == 0) continue;
    any = true;
    batch[filled] = S24Job{j.values, j.bitmask, j.dense, j.nvalues, j.rows, j.cols};
    if (++filled == kMaxJobs) {
      s24_launch(batch, filled, elem_size, st);
      filled = 0;
    }
  }
  if (!any) return CTMI_OK;
  if (filled) s24_launch(batch, filled, elem_size, st);
  return check_launch("ctmi_sparse24_decompress_many");
}

extern "C" int ctmi_quantize_sparse24_compress_supported(int32_t x_dtype, int64_t rows, int64_t cols,
                                                         const ctmi_qparams* qp) {
  if (!qp || rows < 1 || cols < 1 || cols % 8) return 0;
  if (x_dtype != CTMI_BF16 && x_dtype != CTMI_F16 && x_dtype != CTMI_F32) return 0;
  if (qp->scale_dtype != x_dtype || qp->global_scale || qp->col_group) return 0;
  if (qp->zero_point &&
      qp->zp_dtype != (qp->qtype == CTMI_QTYPE_FLOAT ? CTMI_F8E4M3 : CTMI_I8))
    return 0;
  const bool codes8 = (qp->qtype == CTMI_QTYPE_FLOAT && qp->num_bits == 8) ||
                      (qp->qtype == CTMI_QTYPE_INT && qp->num_bits <= 8);
  if (!codes8) return 0;
  VecGeom g;
  return vec_geometry(qp, rows, cols, &g) ? 1 : 0;
}

extern "C" int ctmi_quantize_sparse24_compress(const void* x, int32_t x_dtype, void* values,
                                               uint8_t* bitmask, int64_t rows, int64_t cols,
                                               const ctmi_qparams* qp, void* stream) {
  CTMI_REQUIRE(rows >= 0 && cols >= 0, CTMI_ERR_VALUE, "negative shape");
  int rc = check_qparams(qp, rows, cols);
  if (rc) return rc;
  if (rows == 0 || cols == 0) return CTMI_OK;
  CTMI_REQUIRE(ctmi_quantize_sparse24_compress_supported(x_dtype, rows, cols, qp),
               CTMI_ERR_UNSUPPORTED,
               "no fused kernel for this layout: quantize, then compress the codes");
  CTMI_REQUIRE(x && values && bitmask, CTMI_ERR_VALUE, "NULL tensor pointer");
  CTMI_REQUIRE((uintptr_t)x % (8 * dtype_size(x_dtype)) == 0 && (uintptr_t)values % 4 == 0,
               CTMI_ERR_VALUE, "tensors must be aligned to 8 elements");
  VecGeom g;
  vec_geometry(qp, rows, cols, &g);
  float qmin, qmax;
  rc = quant_range(qp->qtype, qp->num_bits, &qmin, &qmax);
  if (rc) return rc;
  const int64_t items = rows * cols / 8;
  const unsigned grid = (unsigned)cdiv(items, kBlock * 4);
  hipStream_t st = (hipStream_t)stream;
  const uint8_t* zp = (const uint8_t*)qp->zero_point;
#define CTMI_QS24_K(FT, RAW, QK, HZ)                                                             \
  hipLaunchKernelGGL((quant_sparse24_compress_kernel<FT, QK, HZ>), grid, kBlock, 0, st,           \
                     (const RAW*)x, (const RAW*)qp->scale, zp, (uint8_t*)values, bitmask, items,  \
                     g, qmin, qmax)
#define CTMI_QS24(FT, RAW)                                                       \
  if (qp->qtype == CTMI_QTYPE_INT) {                                             \
    if (zp) CTMI_QS24_K(FT, RAW, 0, true); else CTMI_QS24_K(FT, RAW, 0, false);  \
  } else {                                                                       \
    if (zp) CTMI_QS24_K(FT, RAW, 1, true); else CTMI_QS24_K(FT, RAW, 1, false);  \
  }
  if (x_dtype == CTMI_BF16) { CTMI_QS24(BF16, uint16_t); }
  else if (x_dtype == CTMI_F16) { CTMI_QS24(F16, uint16_t); }
  else { CTMI_QS24(F32, float); }
#undef CTMI_QS24_K
#undef CTMI_QS24
  return check_launch("ctmi_quantize_sparse24_compress");
}

// the layouts of ctmi_quantize_sparse24_compress, read the other way; how the codes are
// decoded follows from their dtype, not from the quantization arguments (dequantize
// infers those from the scale's shape, forward.py:107-138)
extern "C" int ctmi_sparse24_decompress_dequantize_supported(int32_t values_dtype,
                                                             int32_t out_dtype, int64_t rows,
                                                             int64_t cols, const ctmi_qparams* qp) {
  if (!qp || rows < 1 || cols < 1 || cols % 8) return 0;
  if (values_dtype != CTMI_I8 && values_dtype != CTMI_F8E4M3) return 0;
  if (out_dtype != CTMI_BF16 && out_dtype != CTMI_F16 && out_dtype != CTMI_F32) return 0;
  if (qp->scale_dtype != out_dtype || qp->global_scale || qp->col_group) return 0;
  if (qp->zero_point && qp->zp_dtype != values_dtype) return 0;
  VecGeom g;
  return vec_geometry(qp, rows, cols, &g) ? 1 : 0;
}

extern "C" int64_t ctmi_sparse24_dequantize_tmp_bytes(int64_t rows, int64_t cols) {
  (void)rows;
  (void)cols;
  return 0;  // the verdicts of the streaming workgroups live in the library's own counters
}

extern "C" int ctmi_sparse24_decompress_dequantize(const void* values, int64_t nvalues,
                                                   int32_t values_dtype, const uint8_t* bitmask,
                                                   void* out,
                                                   int32_t out_dtype, void* tmp, int64_t rows,
                                                   int64_t cols, const ctmi_qparams* qp,
                                                   void* stream) {
  CTMI_REQUIRE(rows >= 0 && cols >= 0, CTMI_ERR_VALUE, "negative shape");
  int rc = check_qparams(qp, rows, cols);
  if (rc) return rc;
  if (rows == 0 || cols == 0) return CTMI_OK;
  CTMI_REQUIRE(ctmi_sparse24_decompress_dequantize_supported(values_dtype, out_dtype, rows, cols, qp),
               CTMI_ERR_UNSUPPORTED,
               "no fused kernel for this layout: decompress the codes, then dequantize");
  (void)tmp;  // no scratch is used any more; the argument stays for callers built against it
  CTMI_REQUIRE(values && bitmask && out, CTMI_ERR_VALUE, "NULL tensor pointer");
  CTMI_REQUIRE(nvalues * 2 == rows * cols, CTMI_ERR_VALUE,
               "a 2:4 tensor of %lld x %lld elements has %lld values, got %lld", (long long)rows,
               (long long)cols, (long long)(rows * cols / 2), (long long)nvalues);
  CTMI_REQUIRE((uintptr_t)out % (8 * dtype_size(out_dtype)) == 0 && (uintptr_t)values % 4 == 0,
               CTMI_ERR_VALUE, "tensors must be aligned to 8 elements");
  VecGeom g;
  vec_geometry(qp, rows, cols, &g);
  const int64_t items = rows * cols / 8;
  const unsigned grid = (unsigned)cdiv(items, kBlock * kS24DqU);
  hipStream_t st = (hipStream_t)stream;
  const uint8_t* zp = (const uint8_t*)qp->zero_point;
  const uint32_t slot = s24_slot_of(st);
#define CTMI_S24DQ_K(FT, RAW, QK, HZ)                                                             \
  hipLaunchKernelGGL((sparse24_scatter_dequant_kernel<FT, QK, HZ>), grid, kBlock, 0, st,          \
                     (const uint8_t*)values, bitmask, (const RAW*)qp->scale, zp, (RAW*)out, items, \
                     g, slot);                                                                     \
  hipLaunchKernelGGL((sparse24_repair_dequant_kernel<FT, QK, HZ>), kS24RepairGrid, kBlock, 0, st, \
                     (const uint8_t*)values, nvalues, bitmask, (const RAW*)qp->scale, zp,          \
                     (RAW*)out, rows, cols / 8, g, slot)
#define CTMI_S24DQ(FT, RAW)                                                          \
  if (values_dtype == CTMI_I8) {                                                     \
    if (zp) { CTMI_S24DQ_K(FT, RAW, 0, true); } else { CTMI_S24DQ_K(FT, RAW, 0, false); } \
  } else {                                                                           \
    if (zp) { CTMI_S24DQ_K(FT, RAW, 1, true); } else { CTMI_S24DQ_K(FT, RAW, 1, false); } \
  }
  if (out_dtype == CTMI_BF16) { CTMI_S24DQ(BF16, uint16_t); }
  else if (out_dtype == CTMI_F16) { CTMI_S24DQ(F16, uint16_t); }
  else { CTMI_S24DQ(F32, float); }
#undef CTMI_S24DQ_K
#undef CTMI_S24DQ
  return check_launch("ctmi_sparse24_decompress_dequantize");
}

// ---- the stacked entry points for a list of weights
namespace ctmi {
namespace {

struct StackedKey {
  int sd, qk;
  bool has_zp, flat;
  float qmin, qmax;
  bool operator==(const StackedKey& o) const {
    return sd == o.sd && qk == o.qk && has_zp == o.has_zp && flat == o.flat && qmin == o.qmin &&
           qmax == o.qmax;
  }
};

struct StackedPlan {
  StackedKey key;
  VecJob job;
  uint8_t* bitmask;
  int64_t rows;
};

template <bool COMPRESS, typename FT, int QK>
void launch_stacked_chain2(const StackedKey& k, const QS24Table& t, unsigned grid, hipStream_t st) {
#define CTMI_ST(ZP, FLAT)                                                                              \
  if constexpr (COMPRESS) {                                                                            \
    hipLaunchKernelGGL((quant_sparse24_compress_chain_kernel<FT, QK, ZP, FLAT>), grid, kBlock, 0, st, t); \
  } else {                                                                                             \
    hipLaunchKernelGGL((sparse24_scatter_dequant_chain_kernel<FT, QK, ZP, FLAT>), grid, kBlock, 0, st, t); \
    hipLaunchKernelGGL((sparse24_repair_dequant_chain_kernel<FT, QK, ZP, FLAT>), kS24RepairGrid, kBlock, 0, \
                       st, t);                                                                         \
  }
  if (k.has_zp) { if (k.flat) { CTMI_ST(true, true) } else { CTMI_ST(true, false) } }
  else { if (k.flat) { CTMI_ST(false, true) } else { CTMI_ST(false, false) } }
#undef CTMI_ST
}

template <bool COMPRESS>
void launch_stacked_chain(const StackedKey& k, const QS24Table& t, unsigned grid, hipStream_t st) {
#define CTMI_ST1(FT)                                                        \
  if (k.qk == 0) launch_stacked_chain2<COMPRESS, FT, 0>(k, t, grid, st);    \
  else launch_stacked_chain2<COMPRESS, FT, 1>(k, t, grid, st)
  if (k.sd == CTMI_BF16) { CTMI_ST1(BF16); }
  else if (k.sd == CTMI_F16) { CTMI_ST1(F16); }
  else { CTMI_ST1(F32); }
#undef CTMI_ST1
}

// weights that share a kernel instance (dtype, code kind, zero points, scale numbering,
// quantization range) into common launches, 8 per launch
template <bool COMPRESS>
void run_stacked(std::vector<StackedPlan>& plans, hipStream_t st) {
  constexpr int per_chunk = kBlock * (COMPRESS ? 4 : kS24DqU);
  std::vector<char> done(plans.size(), 0);
  for (size_t i = 0; i < plans.size(); ++i) {
    if (done[i]) continue;
    const StackedKey key = plans[i].key;
    QS24Table t;
    std::memset(&t, 0, sizeof(t));
    int n = 0;
    uint64_t chunks = 0;
    auto reset = [&]() {
      n = 0;
      chunks = 0;
      for (int k = 0; k < kMaxJobs; ++k) t.chunk_end[k] = 0xFFFFFFFFu;
    };
    reset();
    t.qmin = key.qmin;
    t.qmax = key.qmax;
    auto flush = [&]() {
      if (n == 0) return;
      if (!COMPRESS) t.slot = s24_slot_of(st);
      launch_stacked_chain<COMPRESS>(key, t, (unsigned)chunks, st);
      reset();
    };
    for (size_t j = i; j < plans.size(); ++j) {
      if (done[j] || !(plans[j].key == key)) continue;
      const uint64_t c = (uint64_t)cdiv(plans[j].job.g.nvec, per_chunk);
      if (n == kMaxJobs || chunks + c >= (1ull << 31)) flush();
      t.job[n] = make_chain_job(plans[j].job);
      t.n_items[n] = plans[j].job.g.nvec;
      t.bitmask[n] = plans[j].bitmask;
      t.rows[n] = plans[j].rows;
      chunks += c;
      t.chunk_end[n] = (uint32_t)chunks;
      ++n;
      done[j] = 1;
    }
    flush();
  }
}

}  // namespace
}  // namespace ctmi

extern "C" int ctmi_quantize_sparse24_compress_many(const ctmi_stacked24_job* jobs, int64_t n,
                                                    void* stream) {
  CTMI_REQUIRE(n >= 0 && (jobs || n == 0), CTMI_ERR_VALUE, "bad job list");
  std::vector<StackedPlan> plans;
  plans.reserve((size_t)n);
  for (int64_t i = 0; i < n; ++i) {  // every job is looked at before anything is enqueued
    const ctmi_stacked24_job& j = jobs[i];
    CTMI_REQUIRE(j.rows >= 0 && j.cols >= 0, CTMI_ERR_VALUE, "negative shape");
    int rc = check_qparams(&j.qp, j.rows, j.cols);
    if (rc) return rc;
    if (j.rows == 0 || j.cols == 0) continue;
    CTMI_REQUIRE(ctmi_quantize_sparse24_compress_supported(j.dense_dtype, j.rows, j.cols, &j.qp),
                 CTMI_ERR_UNSUPPORTED,
                 "job %lld: no fused kernel for this layout: quantize, then compress the codes",
                 (long long)i);
    CTMI_REQUIRE(j.dense && j.values && j.bitmask, CTMI_ERR_VALUE, "NULL tensor pointer");
    CTMI_REQUIRE((uintptr_t)j.dense % (8 * dtype_size(j.dense_dtype)) == 0 && (uintptr_t)j.values % 4 == 0,
                 CTMI_ERR_VALUE, "tensors must be aligned to 8 elements");
    CTMI_REQUIRE(j.rows * j.cols / 8 < (1ll << 31), CTMI_ERR_UNSUPPORTED, "job %lld: tensor too large",
                 (long long)i);
    StackedPlan p;
    vec_geometry(&j.qp, j.rows, j.cols, &p.job.g);
    float qmin, qmax;
    rc = quant_range(j.qp.qtype, j.qp.num_bits, &qmin, &qmax);
    if (rc) return rc;
    p.key = StackedKey{j.dense_dtype, j.qp.qtype == CTMI_QTYPE_INT ? 0 : 1, j.qp.zero_point != nullptr,
                       flat_geometry(p.job.g), qmin, qmax};
    p.job.src = j.dense;
    p.job.dst = j.values;
    p.job.scale = j.qp.scale;
    p.job.zp = (const int8_t*)j.qp.zero_point;
    p.bitmask = j.bitmask;
    p.rows = j.rows;
    plans.push_back(p);
  }
  if (plans.empty()) return CTMI_OK;  // nothing to enqueue
  run_stacked<true>(plans, (hipStream_t)stream);
  return check_launch("ctmi_quantize_sparse24_compress_many");
}

extern "C" int ctmi_sparse24_decompress_dequantize_many(const ctmi_stacked24_job* jobs, int64_t n,
                                                        void* stream) {
  CTMI_REQUIRE(n >= 0 && (jobs || n == 0), CTMI_ERR_VALUE, "bad job list");
  std::vector<StackedPlan> plans;
  plans.reserve((size_t)n);
  for (int64_t i = 0; i < n; ++i) {
    const ctmi_stacked24_job& j = jobs[i];
    CTMI_REQUIRE(j.rows >= 0 && j.cols >= 0, CTMI_ERR_VALUE, "negative shape");
    int rc = check_qparams(&j.qp, j.rows, j.cols);
    if (rc) return rc;
    if (j.rows == 0 || j.cols == 0) continue;
    CTMI_REQUIRE(ctmi_sparse24_decompress_dequantize_supported(j.values_dtype, j.dense_dtype, j.rows,
                                                               j.cols, &j.qp),
                 CTMI_ERR_UNSUPPORTED,
                 "job %lld: no fused kernel for this layout: decompress the codes, then dequantize",
                 (long long)i);
    CTMI_REQUIRE(j.dense && j.values && j.bitmask, CTMI_ERR_VALUE, "NULL tensor pointer");
    CTMI_REQUIRE((uintptr_t)j.dense % (8 * dtype_size(j.dense_dtype)) == 0 && (uintptr_t)j.values % 4 == 0,
                 CTMI_ERR_VALUE, "tensors must be aligned to 8 elements");
    CTMI_REQUIRE(j.rows * j.cols / 8 < (1ll << 31), CTMI_ERR_UNSUPPORTED, "job %lld: tensor too large",
                 (long long)i);
    StackedPlan p;
    vec_geometry(&j.qp, j.rows, j.cols, &p.job.g);
    p.key = StackedKey{j.dense_dtype, j.values_dtype == CTMI_I8 ? 0 : 1, j.qp.zero_point != nullptr,
                       flat_geometry(p.job.g), 0.0f, 0.0f};
    p.job.src = j.values;
    p.job.dst = const_cast<void*>(j.dense);
    p.job.scale = j.qp.scale;
    p.job.zp = (const int8_t*)j.qp.zero_point;
    p.bitmask = j.bitmask;
    p.rows = j.rows;
    plans.push_back(p);
  }
  if (plans.empty()) return CTMI_OK;
  run_stacked<false>(plans, (hipStream_t)stream);
  return check_launch("ctmi_sparse24_decompress_dequantize_many");
}
