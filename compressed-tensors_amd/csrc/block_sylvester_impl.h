// Transforms W = diag(sign_in) * (Ma (x) Sylvester(64)) * diag(sign_out) * scale on runs of
// K * 64 bfloat16 (or float16) elements, K <= 224: the reference's Hadamard matrices of size K * 2^m
//
//   random_hadamard_matrix, _matmul_hadU        transform/utils/hadamard.py:65-163
//   HadamardTransform.forward                   transform/factory/hadamard.py:104-121
//
// (K from its table of known matrices: 12, 20, 28 ... 224; 14336 = 224 * 64 is the size in
// front of Llama-3's down projections).  A run is a K x 64 matrix X (element 64 i + j) and
//     y = vec(Ma^T X S),      S = Sylvester(64).
// The product with Ma takes bfloat16 inputs and a matrix of +-1, so it is exact as ONE product
// on the matrix cores (v_mfma_f32_32x32x16_bf16, fp32 accumulation); the factor S then needs no
// matrix at all: it is six butterfly stages on the fp32 accumulators.  Nothing is split into
// bfloat16 terms, which is what made the two-product kernel three times as expensive.
//
// Per run a wavefront computes D[j][i'] = sum_i X[i][j] Ma[i][i'] with j on the M side:
//   A operand  X^T: lane (c, g) holds X[16 ks + 8 g + e][32 mt + c], e = 0..7: picked as single
//              16-bit elements out of an image of 32 rows of X in LDS (the run streams through
//              it, 4.5 KB at a time, loaded as whole 128-byte lines)
//   B operand  Ma: lane (c, g) holds Ma[16 ks + 8 g + e][32 nt + c] = 16 bytes of row 32 nt + c
//              of Ma^T; all fragments of Ma sit in LDS in the lanes' own order (K = 224: 98 KB,
//              shared by the four wavefronts of the workgroup) and one read serves both M tiles
//   D          acc[mt][nt][4 b + r] = D[32 mt + 8 b + 4 g + r][32 nt + c]
// The butterflies over j: the stage over mt adds and subtracts whole accumulator tiles; one
// exchange between the lane halves (v_permlane32_swap) pairs the two values of the stage over
// g in one lane; the other four stages are within a lane's 16 values.  Afterwards lane (c, h)
// holds, for every nt, the 32 neighbouring outputs y[64 (32 nt + c) + 32 h ...]: they go
// through the LDS image once more so that the stores are whole lines again.
//
// One wavefront per SIMD for K > 128: the accumulators are 32 NT registers a lane and the next
// run, prefetched whole, another 16 NT.
#pragma once
#include <utility>

#include "ctmi_device.h"
#include "ctmi_host.h"
#include "quant_fast.h"
#include "fwht.h"

namespace ctmi {

struct BsTable {
  const void* x[kFwhtMaxJobs];
  void* out[kFwhtMaxJobs];
  int64_t end[kFwhtMaxJobs];  // running total of runs, job 0 .. j (unused: INT64_MAX)
  int64_t total;
};

// The kernels are compiled in four translation units (bfloat16 / float16 tensors, Sylvester
// factors of 32 ... 128 / of 4 ... 16), one entry point each.
#define CTMI_BS_ENTRY(name)                                                                      \
  int name(const BsTable& tab, int inner, const uint16_t* ma_t, int k, const float* sign_in,     \
           const float* sign_out, float scale, hipStream_t st)
CTMI_BS_ENTRY(bs_wide_bf16);
CTMI_BS_ENTRY(bs_narrow_bf16);
CTMI_BS_ENTRY(bs_wide_f16);
CTMI_BS_ENTRY(bs_narrow_f16);

namespace {

typedef __bf16 bs_bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 bs_f16x8_t __attribute__((ext_vector_type(8)));
typedef float bs_f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t bs_u32x4 __attribute__((ext_vector_type(4)));

constexpr int kBsWaves = 4;
constexpr int kBsThreads = kBsWaves * kWave;
constexpr int kBsPitch = 36;                    // dwords between the rows of an image (64 bf16 + 16 bytes)
constexpr int kBsImage = 32 * kBsPitch;         // dwords of an image of 32 rows
constexpr int kBsRing = kBsImage;               // per wavefront


// A wavefront's run number is the same in all its lanes, which the compiler cannot see: said
// outright, the search and the table reads behind it are scalar instructions.  (As vector
// loads they would also make every prefetch wait for all loads in flight.)
__device__ __forceinline__ int64_t bs_uniform(int64_t v) {
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)v >> 32));
  return (int64_t)(((uint64_t)hi << 32) | lo);
}

__device__ __forceinline__ int bs_job(const BsTable& t, int64_t run, int64_t* local) {
  run = bs_uniform(run);
  int j = 0;
  int64_t first = 0;
#pragma unroll
  for (int i = 0; i < kFwhtMaxJobs - 1; ++i) {
    const bool past = run >= t.end[i];
    j = past ? i + 1 : j;
    first = past ? t.end[i] : first;
  }
  *local = run - first;
  return j;
}

// Where run number `run` (its own in every lane) of n elements begins, in the inputs or (OUT)
// the outputs: the table's entries picked by comparisons, no indexed read of the table.
template <bool OUT>
__device__ __forceinline__ uint16_t* bs_lane_run(const BsTable& t, int64_t run, int64_t n) {
  int64_t first = 0;
  const void* base = OUT ? t.out[0] : t.x[0];
#pragma unroll
  for (int i = 0; i < kFwhtMaxJobs - 1; ++i) {
    const bool past = run >= t.end[i];
    first = past ? t.end[i] : first;
    base = past ? (OUT ? t.out[i + 1] : t.x[i + 1]) : base;
  }
  return static_cast<uint16_t*>(const_cast<void*>(base)) + (run - first) * n;
}

// fragments of Ma, the sign masks (SIGNS != 0), one image per wavefront
constexpr size_t bs_lds_bytes(int nt, int ch, int signs) {
  return ((size_t)2 * ch * nt * kWave * 4 + (signs ? (size_t)(signs == 1 ? ch : nt) * 4 * kWave * 4 : 0) +
          (size_t)kBsWaves * kBsRing) * sizeof(uint32_t);
}

// One product on the matrix cores: bfloat16 operands, or (HALF) float16 ones
template <bool HALF>
__device__ __forceinline__ bs_f32x16_t bs_mma(const bs_u32x4& a, const bs_u32x4& b, const bs_f32x16_t& c) {
  if constexpr (HALF)
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(bs_f16x8_t, a),
                                                  __builtin_bit_cast(bs_f16x8_t, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bs_bf16x8_t, a),
                                                   __builtin_bit_cast(bs_bf16x8_t, b), c, 0, 0, 0);
}

// The fragments of Ma into LDS, zero beyond K: fragment (ks, nt), lane (c, g) holds
// Ma[16 ks + 8 g + e][first_col + 32 nt + c], e = 0..7 (CH chunks of 32 rows of Ma, NT tiles of
// 32 of its columns from first_col on).  Eight at a time per wavefront, loads first: one
// after the other they would cost the launch as many memory round trips as there are
// fragments.
template <int NT, bool HALF, int CH = NT>
__device__ __forceinline__ void bs_load_fragments(const uint16_t* __restrict__ ma_t, int k_dim,
                                                  bs_u32x4* ma_frag, uint32_t wave, uint32_t l,
                                                  int first_col = 0) {
  constexpr int KS = 2 * CH;
  const uint32_t c = l & 31u, g = l >> 5;
  const bool ma_vectors = k_dim % 8 == 0 && (uintptr_t)ma_t % 16 == 0;  // 16-byte pieces of whole rows
  for (int f0 = 0; f0 < KS * NT; f0 += kBsWaves * 8) {
    bs_u32x4 w[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int f = f0 + u * kBsWaves + (int)wave;
      const int ks = f / NT, nt = f % NT;
      const int col = first_col + 32 * nt + (int)c, i0 = 16 * ks + 8 * (int)g;  // Ma[i0 + e][col] = ma_t[col][i0 + e]
      w[u] = bs_u32x4{0u, 0u, 0u, 0u};
      if (f < KS * NT && col < k_dim) {
        if (ma_vectors) {
          if (i0 < k_dim) w[u] = __builtin_bit_cast(bs_u32x4, ldg<uint16_t, 8>(ma_t + (int64_t)col * k_dim + i0));
        } else {
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            const int i = i0 + 2 * d;
            const uint32_t lo = i < k_dim ? ma_t[(int64_t)col * k_dim + i] : 0u;
            const uint32_t hi = i + 1 < k_dim ? ma_t[(int64_t)col * k_dim + i + 1] : 0u;
            w[u][d] = lo | (hi << 16);
          }
        }
      }
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int f = f0 + u * kBsWaves + (int)wave;
      if constexpr (HALF) {
#pragma unroll
        for (int d = 0; d < 4; ++d)
          w[u][d] = (uint32_t)f32_to_f16(bf16_lo(w[u][d])) | ((uint32_t)f32_to_f16(bf16_hi(w[u][d])) << 16);
      }
      if (f < KS * NT) ma_frag[f * kWave + l] = w[u];
    }
  }
}

// NT: column tiles of 32 that cover K (K <= 32 NT); SIGNS: 0 none, 1 sign_in, 2 sign_out;
// HALF: float16 tensors (the matrix arrives in bfloat16 and converts exactly: entries +-1);
// PAIR (RUNS != 1): runs of K * 2^log_inner elements, 2^log_inner = 64 / RUNS = 32, 16 or 8 (Ma (x) Sylvester(32),
// e.g. 7168 = 224 * 32, 3584 = 224 * 16, 1792 = 224 * 8), two, four or eight at a time: the
// 64 columns of the image are 32 (16, 8) of one run beside those of the next, and the
// butterfly stages over the column bits that tell the runs apart are left out (the stage over
// the M tiles always; 16: the one 16 columns apart as well; 8: and the one 8 apart).  A lane
// loads and stores the run its piece of a row lies in; where the tensors end inside a unit
// the missing runs are read as the last one once more and not stored.
// RUNS: runs side by side in the image: 1, 2, 4, 8, 16 for Sylvester(64), (32), (16), (8), (4).
// With 16 (768 = 192 * 4, 896 = 224 * 4) a lane's 8 columns are the rows of two runs: two
// 8-byte loads and stores, and the stage between the lane halves only exchanges.
// CH: chunks of 32 rows of X (= of Ma) a run has; NT tiles of 32 output rows from row out_first
// on are computed.  CH = NT and out_first = 0 for K <= 224; for K up to 256 the accumulators of
// all eight tiles do not fit beside a run held ahead, and two launches compute four tiles each
// (CH = 8, NT = 4, out_first = 0 and 128: the run is read twice).
template <int NT, int SIGNS, bool HALF, int RUNS, int CH = NT>
__global__ void __launch_bounds__(kBsThreads, 1)
block_sylvester64_kernel(BsTable tab, const uint16_t* __restrict__ ma_t, int k_dim,
                         const float* __restrict__ signs, float scale, int out_first) {
  constexpr int KS = 2 * CH;  // steps of 16 over the contracted index
  if constexpr (CH == NT) out_first = 0;
  constexpr bool PAIR = RUNS != 1;
  constexpr int log_inner = RUNS == 1 ? 6 : RUNS == 2 ? 5 : RUNS == 4 ? 4 : RUNS == 8 ? 3 : 2;
  constexpr bool TWO = RUNS == 16;  // a lane's 8 columns are the rows of two runs of 4 columns
  constexpr int unit_runs = RUNS;
  extern __shared__ __attribute__((aligned(16))) uint32_t bs_lds[];
  bs_u32x4* ma_frag = reinterpret_cast<bs_u32x4*>(bs_lds);                    // [KS * NT][64]
  bs_u32x4* flip = ma_frag + KS * NT * kWave;                                 // [CH or NT][4][64] (SIGNS 1 or 2)
  constexpr int SIGN_TILES = SIGNS == 1 ? CH : NT;
  const uint32_t l = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const uint32_t c = l & 31u, g = l >> 5;
  uint32_t* image = bs_lds + (KS * NT + (SIGNS ? SIGN_TILES * 4 : 0)) * kWave * 4 + wave * kBsRing;
  const int64_t n = (int64_t)k_dim << log_inner;
  // the lane's 8 columns inside a row of a run, and that run's place in the unit (TWO: the
  // first of its two runs)
  const uint32_t piece = TWO ? 0u : 8 * (l & ((1u << (TWO ? 0 : log_inner - 3)) - 1u));
  const uint32_t my_run = TWO ? 2 * (l & 7u) : PAIR ? (l & 7u) >> (TWO ? 0 : log_inner - 3) : 0u;

  bs_load_fragments<NT, HALF, CH>(ma_t, k_dim, ma_frag, wave, l, out_first);
  // Sign masks of the vectors a lane loads (SIGNS == 1: vector q of chunk ch is row
  // 32 ch + l / 8 + 8 q, columns 8 (l % 8) ...) or stores (SIGNS == 2: the same positions with
  // the tile nt in place of the chunk): the same for the four wavefronts, read at each use
  if constexpr (SIGNS != 0) {
    for (int f = (int)wave; f < SIGN_TILES * 4; f += kBsWaves) {
      const int row = (SIGNS == 2 ? out_first : 0) + 32 * (f >> 2) + (int)(l >> 3) + 8 * (f & 3);
      bs_u32x4 m = {0u, 0u, 0u, 0u};
      if (row < k_dim) {
        if constexpr (TWO) {  // both runs: the row's four signs
          const Vec<uint32_t, 4> s4 = ldg<uint32_t, 4>(reinterpret_cast<const uint32_t*>(signs) + 4 * row);
#pragma unroll
          for (int d = 0; d < 2; ++d)
            m[d] = m[d + 2] = ((s4.v[2 * d] >> 16) & 0x8000u) | (s4.v[2 * d + 1] & 0x80000000u);
        } else {
          const Vec<uint32_t, 8> s8 = ldg<uint32_t, 8>(reinterpret_cast<const uint32_t*>(signs) + (row << log_inner) + piece);
#pragma unroll
          for (int d = 0; d < 4; ++d) m[d] = ((s8.v[2 * d] >> 16) & 0x8000u) | (s8.v[2 * d + 1] & 0x80000000u);
        }
      }
      flip[f * kWave + l] = m;
    }
  }
  __syncthreads();

  // selector that puts the 16-bit element of column c out of two dwords (columns c & ~1, c | 1
  // of two neighbouring rows) side by side
  const uint32_t pick = (c & 1u) ? 0x07060302u : 0x05040100u;

  // A run is NT chunks of 32 rows of X, 4 vectors a lane each; rows beyond K read as zeros.
  // All of the next run is in flight while this one is worked on: with one wavefront per SIMD
  // nothing else hides the latency of memory.
  // No branch around the loads (a load under a condition makes the compiler wait for it on
  // the spot): a run beyond the last reads the last again, a row beyond K reads row K - 1 and
  // is replaced by zeros when it is used.
  bs_u32x4 in[CH][4];
  // where the lane's run of unit u begins (a unit: one run, two neighbouring ones looked up
  // with scalar instructions, or four / eight looked up by every lane for itself);
  // table reads once per unit, not per chunk
  auto run_start = [&](int64_t u, int second = 0) {
    if constexpr (RUNS > 2) {
      return (const uint16_t*)bs_lane_run<false>(
          tab, min(unit_runs * u + (int64_t)my_run + second, tab.total - 1), n);
    } else if constexpr (PAIR) {
      int64_t la, lb;
      const int64_t ra = min(2 * u, tab.total - 1), rb = min(2 * u + 1, tab.total - 1);
      const int ja = bs_job(tab, ra, &la), jb = bs_job(tab, rb, &lb);
      const uint16_t* a = static_cast<const uint16_t*>(tab.x[ja]) + la * n;
      const uint16_t* b = static_cast<const uint16_t*>(tab.x[jb]) + lb * n;
      return my_run ? b : a;
    } else {
      const int64_t r = u < tab.total ? u : tab.total - 1;
      int64_t local;
      const int j = bs_job(tab, r, &local);
      return static_cast<const uint16_t*>(tab.x[j]) + local * n;
    }
  };
  auto fetch = [&](const uint16_t* __restrict__ xr, const uint16_t* __restrict__ xr2, int ch) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int row = 32 * ch + (int)(l >> 3) + 8 * q;
      const int at = ((row < k_dim ? row : k_dim - 1) << log_inner) + piece;
      if constexpr (TWO) {
        const Vec<uint32_t, 2> a = __builtin_bit_cast(Vec<uint32_t, 2>, ldg_nt<uint16_t, 4>(xr + at));
        const Vec<uint32_t, 2> b = __builtin_bit_cast(Vec<uint32_t, 2>, ldg_nt<uint16_t, 4>(xr2 + at));
        in[ch][q] = bs_u32x4{a.v[0], a.v[1], b.v[0], b.v[1]};
      } else {
        in[ch][q] = __builtin_bit_cast(bs_u32x4, ldg_nt<uint16_t, 8>(xr + at));
      }
    }
  };
  const int64_t units = PAIR ? (tab.total + unit_runs - 1) / unit_runs : tab.total;

  auto pack2 = [](float lo, float hi) -> uint32_t {
    if constexpr (HALF) return (uint32_t)f32_to_f16(lo) | ((uint32_t)f32_to_f16(hi) << 16);
    else return pack_bf16x2(lo, hi);
  };
  const int64_t step = (int64_t)gridDim.x * kBsWaves;
  int64_t run = (int64_t)blockIdx.x * kBsWaves + wave;
  {
    const uint16_t* first = run_start(run);
    const uint16_t* first2 = TWO ? run_start(run, 1) : first;
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) fetch(first, first2, ch);
  }
  for (; run < units; run += step) {
    const uint16_t* next = run_start(run + step);
    const uint16_t* next2 = TWO ? run_start(run + step, 1) : next;
    bs_f32x16_t acc[2][NT];
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mt][nt][i] = 0.0f;
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) {
      // (LDS reads grouped ahead of the LDS writes they do not depend on: the compiler keeps
      // accesses of the one shared array in program order, and every read that sits behind
      // a write costs the wavefront a round trip of its own)
      bs_u32x4 fl[SIGNS == 1 ? 4 : 1];
      if constexpr (SIGNS == 1) {
#pragma unroll
        for (int q = 0; q < 4; ++q) fl[q] = flip[(ch * 4 + q) * kWave + l];
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        bs_u32x4 w = in[ch][q];
        if (32 * ch + (int)(l >> 3) + 8 * q >= k_dim) w = bs_u32x4{0u, 0u, 0u, 0u};
        if constexpr (SIGNS == 1) w ^= fl[q];
        *reinterpret_cast<bs_u32x4*>(&image[((l >> 3) + 8 * q) * kBsPitch + 4 * (l & 7u)]) = w;
      }
      fetch(next, next2, ch);
      // A operands of both steps and both M tiles: rows 16 ks2 + 8 g + e of the image,
      // column 32 mt + c
      bs_u32x4 a2[2][2];
#pragma unroll
      for (int ks2 = 0; ks2 < 2; ++ks2)
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            const uint32_t* p = &image[(16 * ks2 + 8 * g + 2 * d) * kBsPitch + 16 * mt + (c >> 1)];
            a2[ks2][mt][d] = __builtin_amdgcn_perm(p[kBsPitch], p[0], pick);
          }
#pragma unroll
      for (int ks2 = 0; ks2 < 2; ++ks2) {
        const int ks = 2 * ch + ks2;
        const bs_u32x4* a = a2[ks2];
        // Up to 4 tiles: all fragments of Ma for this step first, one LDS latency per step
        // instead of one per pair of tiles (with 7 tiles the registers do not reach)
        if constexpr (NT <= 4) {
          bs_u32x4 bq[NT];
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) bq[nt] = ma_frag[(ks * NT + nt) * kWave + l];
          asm volatile("" ::: "memory");
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) {
            acc[0][nt] = bs_mma<HALF>(a[0], bq[nt], acc[0][nt]);
            acc[1][nt] = bs_mma<HALF>(a[1], bq[nt], acc[1][nt]);
          }
        } else {
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) {
            const bs_u32x4 b = ma_frag[(ks * NT + nt) * kWave + l];
            acc[0][nt] = bs_mma<HALF>(a[0], b, acc[0][nt]);
            acc[1][nt] = bs_mma<HALF>(a[1], b, acc[1][nt]);
          }
        }
      }
    }
    // butterflies over j = 32 mt + 8 b + 4 g + r
    uint16_t* __restrict__ yr;
    bool stored = true;  // PAIR: a run past the last tensor is not
    uint16_t* __restrict__ yr2 = nullptr;  // TWO: the lane's second run
    bool stored2 = false;
    if constexpr (RUNS > 2) {
      const int64_t mine = unit_runs * run + (int64_t)my_run;
      yr = bs_lane_run<true>(tab, min(mine, tab.total - 1), n);
      stored = mine < tab.total;
      if constexpr (TWO) {
        yr2 = bs_lane_run<true>(tab, min(mine + 1, tab.total - 1), n);
        stored2 = mine + 1 < tab.total;
      }
    } else if constexpr (PAIR) {
      int64_t la, lb;
      const int64_t rb = 2 * run + 1 < tab.total ? 2 * run + 1 : 2 * run;
      const int ja = bs_job(tab, 2 * run, &la), jb = bs_job(tab, rb, &lb);
      uint16_t* a = static_cast<uint16_t*>(tab.out[ja]) + la * n;
      uint16_t* b = static_cast<uint16_t*>(tab.out[jb]) + lb * n;
      yr = my_run ? b : a;
      stored = !my_run || 2 * run + 1 < tab.total;
    } else {
      int64_t local;
      const int j = bs_job(tab, run, &local);
      yr = static_cast<uint16_t*>(tab.out[j]) + local * n;
    }
    const uint32_t h = g;  // after the exchange: lane half h holds j = 32 h ... (PAIR: other runs than half 1 - h)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      float u[2][16];  // u[x][4 b + r] = value at j = 32 h + 8 b + 4 x + r
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        // stage over mt (PAIR: the two tiles are two runs and stay apart)
        const float s = PAIR ? acc[0][nt][v] : acc[0][nt][v] + acc[1][nt][v];
        const float t = PAIR ? acc[1][nt][v] : acc[0][nt][v] - acc[1][nt][v];
        const auto pr = __builtin_amdgcn_permlane32_swap(__float_as_uint(s), __float_as_uint(t), false, false);
        const float lower = __uint_as_float(pr[0]), upper = __uint_as_float(pr[1]);  // g = 0, g = 1
        u[0][v] = TWO ? lower : lower + upper;  // (TWO: columns 4 apart belong to two runs)
        u[1][v] = TWO ? upper : lower - upper;
      }
#pragma unroll
      for (int x = 0; x < 2; ++x)
#pragma unroll
        for (int st = 1; st < 16; st <<= 1) {
          // value 4 b + r sits at column 8 b + 4 x + r: st = 4 pairs columns 8 apart, st = 8 16 apart
          if (PAIR && ((st == 8 && log_inner < 5) || (st == 4 && log_inner < 4))) continue;
#pragma unroll
          for (int v = 0; v < 16; ++v)
            if ((v & st) == 0) {
              const float p = u[x][v], m = u[x][v + st];
              u[x][v] = p + m;
              u[x][v + st] = p - m;
            }
        }
      // row c of this tile, 32 outputs from column 32 h: 8 b + 4 x + r -> four vectors of 8
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        bs_u32x4 w;
        w[0] = pack2(u[0][4 * b] * scale, u[0][4 * b + 1] * scale);
        w[1] = pack2(u[0][4 * b + 2] * scale, u[0][4 * b + 3] * scale);
        w[2] = pack2(u[1][4 * b] * scale, u[1][4 * b + 1] * scale);
        w[3] = pack2(u[1][4 * b + 2] * scale, u[1][4 * b + 3] * scale);
        *reinterpret_cast<bs_u32x4*>(&image[c * kBsPitch + 16 * h + 4 * b]) = w;
      }
      bs_u32x4 fo[SIGNS == 2 ? 4 : 1];
      if constexpr (SIGNS == 2) {
#pragma unroll
        for (int q = 0; q < 4; ++q) fo[q] = flip[(nt * 4 + q) * kWave + l];
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int row = out_first + 32 * nt + (int)(l >> 3) + 8 * q;
        bs_u32x4 w = *reinterpret_cast<const bs_u32x4*>(&image[((l >> 3) + 8 * q) * kBsPitch + 4 * (l & 7u)]);
        if constexpr (SIGNS == 2) w ^= fo[q];
        if constexpr (TWO) {
          if (row < k_dim && stored)
            stg_nt<uint16_t, 4>(yr + 4 * row, __builtin_bit_cast(Vec<uint16_t, 4>, Vec<uint32_t, 2>{{w[0], w[1]}}));
          if (row < k_dim && stored2)
            stg_nt<uint16_t, 4>(yr2 + 4 * row, __builtin_bit_cast(Vec<uint16_t, 4>, Vec<uint32_t, 2>{{w[2], w[3]}}));
        } else if (row < k_dim && stored) {
          stg_nt<uint16_t, 8>(yr + (row << log_inner) + piece, __builtin_bit_cast(Vec<uint16_t, 8>, w));
        }
      }
    }
  }
}

// ---------------------------------------------------------------- Ma (x) Sylvester(128)
// Runs of K * 128 elements (28672 = 224 * 128).  Sylvester(128) = Sylvester(2) (x) Sylvester(64):
// a row of the run is two halves of 64 columns, each half goes through the product with Ma
// like a run of the kernel above, and the stage over the halves is one more addition and
// subtraction of accumulator tiles in front of the other six.  Four M tiles of accumulators
// for all of Ma's column tiles do not fit a wavefront, so the order is turned round: first
// all A operands of the run (both halves, 32 NT registers), then one output tile of Ma after
// the other, each with its four accumulator tiles, its butterflies and its stores; one read
// of a fragment of Ma serves four products.  No run is held ahead.
// Sign masks: one word per lane and vector in LDS (bit 15 - d / 31 - d for the two elements
// of dword d), expanded by a shift and a mask at each use: whole masks would not fit.
constexpr size_t bs128_lds_bytes(int nt, bool signs) {
  return ((size_t)2 * nt * nt * kWave * 4 + (signs ? (size_t)2 * nt * 4 * kWave : 0) +
          (size_t)kBsWaves * kBsRing) * sizeof(uint32_t);
}

template <int NT, int SIGNS, bool HALF>
__global__ void __launch_bounds__(kBsThreads, 1)
block_sylvester128_kernel(BsTable tab, const uint16_t* __restrict__ ma_t, int k_dim,
                          const float* __restrict__ signs, float scale) {
  constexpr int KS = 2 * NT;
  extern __shared__ __attribute__((aligned(16))) uint32_t bs_lds[];
  bs_u32x4* ma_frag = reinterpret_cast<bs_u32x4*>(bs_lds);   // [KS * NT][64]
  uint32_t* flipc = bs_lds + KS * NT * kWave * 4;            // [2][NT * 4][64] (SIGNS != 0)
  const uint32_t l = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const uint32_t c = l & 31u, g = l >> 5;
  uint32_t* image = bs_lds + KS * NT * kWave * 4 + (SIGNS ? 2 * NT * 4 * kWave : 0) + wave * kBsRing;
  const int64_t n = (int64_t)k_dim * 128;
  bs_load_fragments<NT, HALF>(ma_t, k_dim, ma_frag, wave, l);
  if constexpr (SIGNS != 0) {
    for (int f = (int)wave; f < 2 * NT * 4; f += kBsWaves) {
      const int hf = f / (NT * 4), rest = f % (NT * 4);
      const int row = 32 * (rest >> 2) + (int)(l >> 3) + 8 * (rest & 3);
      uint32_t m = 0;
      if (row < k_dim) {
        const Vec<uint32_t, 8> s8 = ldg<uint32_t, 8>(reinterpret_cast<const uint32_t*>(signs) + 128 * row +
                                                     64 * hf + 8 * (l & 7u));
#pragma unroll
        for (int d = 0; d < 4; ++d)
          m |= ((s8.v[2 * d] >> 31) << (15 - d)) | ((s8.v[2 * d + 1] >> 31) << (31 - d));
      }
      flipc[f * kWave + l] = m;
    }
  }
  __syncthreads();
  const uint32_t pick = (c & 1u) ? 0x07060302u : 0x05040100u;
  auto pack2 = [](float lo, float hi) -> uint32_t {
    if constexpr (HALF) return (uint32_t)f32_to_f16(lo) | ((uint32_t)f32_to_f16(hi) << 16);
    else return pack_bf16x2(lo, hi);
  };
  auto flip_of = [&](int hf, int tile, int q) {  // the lane's mask for vector q of a chunk / tile
    const uint32_t m = flipc[((hf * NT + tile) * 4 + q) * kWave + l];
    bs_u32x4 w;
#pragma unroll
    for (int d = 0; d < 4; ++d) w[d] = (m << d) & 0x80008000u;
    return w;
  };
  const int64_t step = (int64_t)gridDim.x * kBsWaves;
  for (int64_t run = (int64_t)blockIdx.x * kBsWaves + wave; run < tab.total; run += step) {
    int64_t local;
    const int j = bs_job(tab, run, &local);
    const uint16_t* __restrict__ xr = static_cast<const uint16_t*>(tab.x[j]) + local * n;
    uint16_t* __restrict__ yr = static_cast<uint16_t*>(tab.out[j]) + local * n;
    // ---- the A operands of both halves: aop[hf][ks][mt]
    bs_u32x4 aop[2][KS][2];
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      bs_u32x4 in[NT][4];
#pragma unroll
      for (int ch = 0; ch < NT; ++ch)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int row = 32 * ch + (int)(l >> 3) + 8 * q;
          in[ch][q] = __builtin_bit_cast(
              bs_u32x4, ldg_nt<uint16_t, 8>(xr + 128 * (row < k_dim ? row : k_dim - 1) + 64 * hf + 8 * (l & 7u)));
        }
#pragma unroll
      for (int ch = 0; ch < NT; ++ch) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          bs_u32x4 w = in[ch][q];
          if (32 * ch + (int)(l >> 3) + 8 * q >= k_dim) w = bs_u32x4{0u, 0u, 0u, 0u};
          if constexpr (SIGNS == 1) w ^= flip_of(hf, ch, q);
          *reinterpret_cast<bs_u32x4*>(&image[((l >> 3) + 8 * q) * kBsPitch + 4 * (l & 7u)]) = w;
        }
#pragma unroll
        for (int ks2 = 0; ks2 < 2; ++ks2)
#pragma unroll
          for (int mt = 0; mt < 2; ++mt)
#pragma unroll
            for (int d = 0; d < 4; ++d) {
              const uint32_t* p = &image[(16 * ks2 + 8 * g + 2 * d) * kBsPitch + 16 * mt + (c >> 1)];
              aop[hf][2 * ch + ks2][mt][d] = __builtin_amdgcn_perm(p[kBsPitch], p[0], pick);
            }
      }
    }
    // ---- one output tile of Ma after the other
    const uint32_t h = g;  // after the exchange: lane half h holds columns 32 h ... of its half
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      bs_f32x16_t acc[2][2];
#pragma unroll
      for (int hf = 0; hf < 2; ++hf)
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[hf][mt][i] = 0.0f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const bs_u32x4 b = ma_frag[(ks * NT + nt) * kWave + l];
#pragma unroll
        for (int hf = 0; hf < 2; ++hf)
#pragma unroll
          for (int mt = 0; mt < 2; ++mt) acc[hf][mt] = bs_mma<HALF>(aop[hf][ks][mt], b, acc[hf][mt]);
      }
#pragma unroll
      for (int oh = 0; oh < 2; ++oh) {  // output half: sum (0) or difference (1) of the input halves
        float u[2][16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const float y0 = oh == 0 ? acc[0][0][v] + acc[1][0][v] : acc[0][0][v] - acc[1][0][v];  // stage over the halves
          const float y1 = oh == 0 ? acc[0][1][v] + acc[1][1][v] : acc[0][1][v] - acc[1][1][v];
          const float s = y0 + y1, t = y0 - y1;  // stage over mt
          const auto pr = __builtin_amdgcn_permlane32_swap(__float_as_uint(s), __float_as_uint(t), false, false);
          const float lower = __uint_as_float(pr[0]), upper = __uint_as_float(pr[1]);  // g = 0, g = 1
          u[0][v] = lower + upper;
          u[1][v] = lower - upper;
        }
#pragma unroll
        for (int x = 0; x < 2; ++x)
#pragma unroll
          for (int st = 1; st < 16; st <<= 1)
#pragma unroll
            for (int v = 0; v < 16; ++v)
              if ((v & st) == 0) {
                const float p = u[x][v], m = u[x][v + st];
                u[x][v] = p + m;
                u[x][v + st] = p - m;
              }
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          bs_u32x4 w;
          w[0] = pack2(u[0][4 * b] * scale, u[0][4 * b + 1] * scale);
          w[1] = pack2(u[0][4 * b + 2] * scale, u[0][4 * b + 3] * scale);
          w[2] = pack2(u[1][4 * b] * scale, u[1][4 * b + 1] * scale);
          w[3] = pack2(u[1][4 * b + 2] * scale, u[1][4 * b + 3] * scale);
          *reinterpret_cast<bs_u32x4*>(&image[c * kBsPitch + 16 * h + 4 * b]) = w;
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int row = 32 * nt + (int)(l >> 3) + 8 * q;
          bs_u32x4 w = *reinterpret_cast<const bs_u32x4*>(&image[((l >> 3) + 8 * q) * kBsPitch + 4 * (l & 7u)]);
          if constexpr (SIGNS == 2) w ^= flip_of(oh, nt, q);
          if (row < k_dim)
            stg_nt<uint16_t, 8>(yr + 128 * row + 64 * oh + 8 * (l & 7u), __builtin_bit_cast(Vec<uint16_t, 8>, w));
        }
      }
    }
  }
}

template <int NT, int SIGNS, bool HALF>
int launch_bs128_variant(const BsTable& tab, const uint16_t* ma_t, int k, const float* signs, float scale,
                         hipStream_t st) {
  auto kern = block_sylvester128_kernel<NT, SIGNS, HALF>;
  constexpr size_t lds = bs128_lds_bytes(NT, SIGNS != 0);
  if (lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return set_error(CTMI_ERR_HIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  }
  static int per_cu = 0;
  int dev = 0, cus = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e == hipSuccess && per_cu == 0) {
    int n = 0;
    e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kern, kBsThreads, lds);
    per_cu = n > 0 ? n : 1;
  }
  if (e != hipSuccess) return set_error(CTMI_ERR_HIP, "device query: %s", hipGetErrorString(e));
  const int64_t wgs = cdiv(tab.total, kBsWaves);
  const int64_t cap = (int64_t)(cus > 0 ? cus : 256) * per_cu;
  const int64_t each = cdiv(wgs, cap);
  const unsigned grid = (unsigned)cdiv(wgs, each);
  hipLaunchKernelGGL(kern, grid, kBsThreads, lds, st, tab, ma_t, k, signs, scale);
  return CTMI_OK;
}

template <int NT, bool HALF>
int launch_bs128(const BsTable& tab, const uint16_t* ma_t, int k, const float* sign_in,
                 const float* sign_out, float scale, hipStream_t st) {
  if (sign_in) return launch_bs128_variant<NT, 1, HALF>(tab, ma_t, k, sign_in, scale, st);
  if (sign_out) return launch_bs128_variant<NT, 2, HALF>(tab, ma_t, k, sign_out, scale, st);
  return launch_bs128_variant<NT, 0, HALF>(tab, ma_t, k, nullptr, scale, st);
}

template <int NT, int SIGNS, bool HALF, int RUNS, int CH = NT>
int launch_bs_variant(const BsTable& tab, const uint16_t* ma_t, int k, const float* signs, float scale,
                      hipStream_t st) {
  auto kern = block_sylvester64_kernel<NT, SIGNS, HALF, RUNS, CH>;
  constexpr size_t lds = bs_lds_bytes(NT, CH, SIGNS);
  if (lds > 48 * 1024) {
    // the attribute belongs to the kernel as loaded on one device; setting it again is cheap
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return set_error(CTMI_ERR_HIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  }
  // as many workgroups as are resident together (one per compute unit for K > 128, where a
  // wavefront fills a SIMD's registers); every wavefront takes runs in turn
  static int per_cu = 0;  // the same on every device of one process (one architecture)
  int dev = 0, cus = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e == hipSuccess && per_cu == 0) {
    int n = 0;
    e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kern, kBsThreads, lds);
    per_cu = n > 0 ? n : 1;
  }
  if (e != hipSuccess) return set_error(CTMI_ERR_HIP, "device query: %s", hipGetErrorString(e));
  const int64_t wgs = cdiv(cdiv(tab.total, (int64_t)RUNS), kBsWaves);
  const int64_t cap = (int64_t)(cus > 0 ? cus : 256) * per_cu;
  const int64_t each = cdiv(wgs, cap);  // runs per wavefront, the same for all
  const unsigned grid = (unsigned)cdiv(wgs, each);
  // CH > NT: the output tiles in turn, NT at a time
  for (int first = 0; first < 32 * CH && first < k; first += 32 * NT)
    hipLaunchKernelGGL(kern, grid, kBsThreads, lds, st, tab, ma_t, k, signs, scale, first);
  return CTMI_OK;
}

template <int NT, bool HALF, int RUNS, int CH = NT>
int launch_bs_dtype(const BsTable& tab, const uint16_t* ma_t, int k, const float* sign_in,
                    const float* sign_out, float scale, hipStream_t st) {
  if (sign_in) return launch_bs_variant<NT, 1, HALF, RUNS, CH>(tab, ma_t, k, sign_in, scale, st);
  if (sign_out) return launch_bs_variant<NT, 2, HALF, RUNS, CH>(tab, ma_t, k, sign_out, scale, st);
  return launch_bs_variant<NT, 0, HALF, RUNS, CH>(tab, ma_t, k, nullptr, scale, st);
}

// by the size of the block: tiles of 32 that cover it
template <bool HALF, int RUNS>
int bs_by_block(const BsTable& tab, const uint16_t* ma_t, int k, const float* sign_in,
                const float* sign_out, float scale, hipStream_t st) {
  if (k <= 32) return launch_bs_dtype<1, HALF, RUNS>(tab, ma_t, k, sign_in, sign_out, scale, st);
  if (k <= 64) return launch_bs_dtype<2, HALF, RUNS>(tab, ma_t, k, sign_in, sign_out, scale, st);
  if (k <= 128) return launch_bs_dtype<4, HALF, RUNS>(tab, ma_t, k, sign_in, sign_out, scale, st);
  // (the reference's largest-block rule gives blocks of 132 ... 256 rows: a tile count of their own each)
  if (k <= 160) return launch_bs_dtype<5, HALF, RUNS>(tab, ma_t, k, sign_in, sign_out, scale, st);
  if (k <= 192) return launch_bs_dtype<6, HALF, RUNS>(tab, ma_t, k, sign_in, sign_out, scale, st);
  if (k <= 224) return launch_bs_dtype<7, HALF, RUNS>(tab, ma_t, k, sign_in, sign_out, scale, st);
  return launch_bs_dtype<4, HALF, RUNS, 8>(tab, ma_t, k, sign_in, sign_out, scale, st);
}

// Sylvester factors of 128, 64 and 32 ...
template <bool HALF>
int bs_wide(const BsTable& tab, int inner, const uint16_t* ma_t, int k, const float* sign_in,
            const float* sign_out, float scale, hipStream_t st) {
  if (inner == 128) {
    if (k <= 32) return launch_bs128<1, HALF>(tab, ma_t, k, sign_in, sign_out, scale, st);
    if (k <= 64) return launch_bs128<2, HALF>(tab, ma_t, k, sign_in, sign_out, scale, st);
    if (k <= 128) return launch_bs128<4, HALF>(tab, ma_t, k, sign_in, sign_out, scale, st);
    if (k <= 160) return launch_bs128<5, HALF>(tab, ma_t, k, sign_in, sign_out, scale, st);
    if (k <= 192) return launch_bs128<6, HALF>(tab, ma_t, k, sign_in, sign_out, scale, st);
    return launch_bs128<7, HALF>(tab, ma_t, k, sign_in, sign_out, scale, st);
  }
  if (inner == 64) return bs_by_block<HALF, 1>(tab, ma_t, k, sign_in, sign_out, scale, st);
  return bs_by_block<HALF, 2>(tab, ma_t, k, sign_in, sign_out, scale, st);
}

// ... and of 16, 8 and 4
template <bool HALF>
int bs_narrow(const BsTable& tab, int inner, const uint16_t* ma_t, int k, const float* sign_in,
              const float* sign_out, float scale, hipStream_t st) {
  if (inner == 16) return bs_by_block<HALF, 4>(tab, ma_t, k, sign_in, sign_out, scale, st);
  if (inner == 8) return bs_by_block<HALF, 8>(tab, ma_t, k, sign_in, sign_out, scale, st);
  return bs_by_block<HALF, 16>(tab, ma_t, k, sign_in, sign_out, scale, st);
}

}  // namespace
}  // namespace ctmi
