// Hadamard transform apply on the matrix cores.
//
//   apply_transform_weight / _multihead_matmul   transform/utils/matrix.py:65-171
//   HadamardTransform.forward                    transform/factory/hadamard.py:104-121
//
// The reference multiplies by an explicit n x n matrix (fp32 online, fp64 when
// fused into weights) and divides by sqrt(n).  Here the matrix is taken in
// factored form  W = diag(s_in) * (Ma (x) Mb) * diag(s_out)  with Ma (a x a) and
// Mb (b x b) small +-1 matrices (Sylvester blocks for Hadamard transforms; a = 1
// for block sizes up to 128).  Viewing each length-n run of the last dimension
// as an a x b matrix X,
//        x * (Ma (x) Mb)  =  vec( Ma^T * X * Mb ),
// two small dense products that run on bf16 MFMA (v_mfma_f32_16x16x32_bf16)
// out of LDS.  +-1 is exact in bf16 and inputs are split into bf16 terms that
// sum to the input exactly (1 term for bf16, 2 for fp16, 3 for fp32), so stage
// 1 accumulates exact products in fp32.  The fp32 intermediate is split three
// ways (24 significant bits) before stage 2.  Results differ from the
// reference only by fp32 summation order: within one ulp of the output dtype.
//
// Tile = S sub-rows of b elements = one contiguous span of memory, staged
// through LDS in both directions so that every HBM access is a full 16-byte
// lane access on consecutive addresses.
#include <atomic>
#include "ctmi_device.h"
#include "ctmi_host.h"
#include "fwht.h"
#include "qparams.h"
#include "quant_core.h"
#include "quant_fast.h"

namespace ctmi {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

constexpr int kHadThreads = 256;
constexpr int kHadWaves = kHadThreads / kWave;
#ifndef CTMI_HAD_ROWS_THREADS
#define CTMI_HAD_ROWS_THREADS 512  // the matrix set-up of hadamard_rows_kernel is shared by a workgroup
#endif
constexpr int kRowsThreads = CTMI_HAD_ROWS_THREADS;
constexpr int kRowsWaves = kRowsThreads / kWave;
#ifndef CTMI_HAD_KRON_THREADS
#define CTMI_HAD_KRON_THREADS 256  // measured: 512 is 4 % slower at 64 x 64
#endif
constexpr int kKronThreads = CTMI_HAD_KRON_THREADS;
constexpr int kKronWaves = kKronThreads / kWave;
#ifndef CTMI_HQP_GROUPS
#define CTMI_HQP_GROUPS 1  // groups of 16 sub-rows a wavefront takes at a time
#endif
#ifndef CTMI_HQP_TUNING
#define CTMI_HQP_TUNING 1024, 1  // fused rotation + quantization kernel: threads, workgroups per CU
#endif
constexpr int kHqpTuning[] = {CTMI_HQP_TUNING};
constexpr int kHqpThreads = kHqpTuning[0];
constexpr int kHqpWaves = kHqpThreads / kWave;
#define CTMI_HQP_WG_PER_CU kHqpTuning[1]
#ifndef CTMI_HAD_KRON_WAVES
#define CTMI_HAD_KRON_WAVES 2  // waves per SIMD the kernel for 64 x 64 is built for (measured best)
#endif

// Up to kHadMaxJobs tensors for one launch of a kernel whose workgroups stay for the
// whole launch (the matrix set-up is then paid once for all of them).  A unit is
// what a wavefront takes at a time: 16 sub-rows, or a data row.
constexpr int kHadMaxJobs = 8;
struct HadJobs {
  const void* x[kHadMaxJobs];
  void* out[kHadMaxJobs];
  void* scale[kHadMaxJobs];    // fused rotation + quantization only
  void* rotated[kHadMaxJobs];  // fused rotation + quantization only
  int64_t end[kHadMaxJobs];    // running total of units, job 0 .. j (unused: INT64_MAX)
  int64_t n_sub[kHadMaxJobs];  // sub-rows of job j
};

// the job of a unit and the unit's number within that job (all wave-uniform); launches
// of a single tensor skip the search and the indexed loads behind it
template <bool MANY>
__device__ __forceinline__ int had_job(const HadJobs& t, int64_t unit, int64_t* local) {
  if constexpr (!MANY) {
    *local = unit;
    return 0;
  }
  {
    // a wavefront's unit is the same in all its lanes, which the compiler cannot see: said
    // outright, the search and the table reads behind it are scalar instructions (as vector
    // loads they make the wavefront wait for every load it has in flight)
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)unit);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)unit >> 32));
    unit = (int64_t)(((uint64_t)hi << 32) | lo);
  }
  int j = 0;
  int64_t first = 0;
#pragma unroll
  for (int i = 0; i < kHadMaxJobs - 1; ++i) {
    const bool past = unit >= t.end[i];
    j = past ? i + 1 : j;
    first = past ? t.end[i] : first;
  }
  *local = unit - first;
  return j;
}

struct HadArgs {
  const void* x;
  void* out;
  const uint16_t* mbt;   // Mb^T, [b][b] bf16
  const uint16_t* mat;   // Ma^T, [a][a] bf16 (a > 1)
  const float* s_in;     // [n] or NULL
  const float* s_out;    // [n] or NULL
  int64_t n_sub;         // number of sub-rows (numel / b)
  float sqrt_n;
};

template <int A, int B, typename IO>
struct HadCfg {
  static constexpr int NS = IO::id == CTMI_BF16 ? 1 : (IO::id == CTMI_F16 ? 2 : 3);
  static constexpr int S = A > 64 ? A : 64;  // sub-rows per tile, a multiple of A
  static constexpr int XP = B + 8;           // padded row pitch (elements): conflict-free 16-byte reads
  static constexpr int TP = S + 8;
  static constexpr int AP = A + 8;
  static constexpr int OP = B + 16 / (int)sizeof(typename IO::raw);
  static constexpr size_t xs_bytes = (size_t)NS * S * XP * 2;
  static constexpr size_t mbt_bytes = (size_t)B * XP * 2;
  static constexpr size_t mat_bytes = A > 1 ? (size_t)A * AP * 2 : 0;
  static constexpr size_t tt_bytes = A > 1 ? (size_t)3 * B * TP * 2 : 0;
  static constexpr size_t os_bytes = (size_t)S * OP * sizeof(typename IO::raw);
  static constexpr size_t lds_bytes = xs_bytes + mbt_bytes + mat_bytes + tt_bytes + os_bytes;
};

// split an fp32 value into bf16 terms that add up to it (exactly when the
// value has at most 8 * NS significant bits)
template <int NS>
__device__ __forceinline__ void split_bf16(float v, uint16_t* parts) {
  float rest = v;
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    const uint16_t h = f32_to_bf16(rest);
    parts[s] = h;
    rest -= bf16_to_f32(h);
  }
}

template <int A, int B, typename IO>
__global__ void __launch_bounds__(kHadThreads) hadamard_mfma_kernel(HadArgs a) {
  using C = HadCfg<A, B, IO>;
  using R = typename IO::raw;
  constexpr int NS = C::NS, S = C::S, XP = C::XP, TP = C::TP, AP = C::AP, OP = C::OP;
  constexpr int N = A * B;
  constexpr int VE = 16 / (int)sizeof(R);  // elements per 16-byte global access
  extern __shared__ __align__(16) unsigned char lds[];
  uint16_t* Xs = reinterpret_cast<uint16_t*>(lds);
  uint16_t* Mbt = reinterpret_cast<uint16_t*>(lds + C::xs_bytes);
  uint16_t* Mat = reinterpret_cast<uint16_t*>(lds + C::xs_bytes + C::mbt_bytes);
  uint16_t* Tt = reinterpret_cast<uint16_t*>(lds + C::xs_bytes + C::mbt_bytes + C::mat_bytes);
  R* Os = reinterpret_cast<R*>(lds + C::xs_bytes + C::mbt_bytes + C::mat_bytes + C::tt_bytes);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, lq = lane >> 4;

  // ---- the small matrices, once per workgroup
  for (int i = tid; i < B * B / 8; i += kHadThreads) {
    const int r = (i * 8) / B, c = (i * 8) % B;
    *reinterpret_cast<uint4*>(&Mbt[r * XP + c]) = *reinterpret_cast<const uint4*>(&a.mbt[r * B + c]);
  }
  if constexpr (A > 1) {
    for (int i = tid; i < A * A / 8; i += kHadThreads) {
      const int r = (i * 8) / A, c = (i * 8) % A;
      *reinterpret_cast<uint4*>(&Mat[r * AP + c]) = *reinterpret_cast<const uint4*>(&a.mat[r * A + c]);
    }
  }

  const int64_t n_tiles = (a.n_sub + S - 1) / S;
  for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
    const int64_t sub0 = tile * S;
    const R* src = reinterpret_cast<const R*>(a.x) + sub0 * B;
    R* dst = reinterpret_cast<R*>(a.out) + sub0 * B;
    const int64_t live = (a.n_sub - sub0 < S ? a.n_sub - sub0 : S) * B;  // elements in this tile

    __syncthreads();  // previous tile fully written out before Xs / Os are reused
    // ---- global -> LDS, with the input signs and the bf16 split
    for (int e = tid * VE; e < S * B; e += kHadThreads * VE) {
      Vec<R, VE> v;
      if (e < live) {
        v = ldg_nt<R, VE>(src + e);
      } else {
#pragma unroll
        for (int j = 0; j < VE; ++j) v.v[j] = IO::from_f32(0.0f);
      }
      const int row = e / B, col = e % B;
      const int pos = e % N;  // a tile starts on a multiple of N elements
#pragma unroll
      for (int j = 0; j < VE; ++j) {
        float f = IO::to_f32(v.v[j]);
        if (a.s_in) f *= a.s_in[pos + j];
        uint16_t parts[NS];
        split_bf16<NS>(f, parts);
#pragma unroll
        for (int s = 0; s < NS; ++s) Xs[(s * S + row) * XP + col + j] = parts[s];
      }
    }
    __syncthreads();

    // ---- stage 1: T = X * Mb  (per 16 x 16 output tile: K = B in steps of 32)
    for (int mt = wave; mt < S / 16; mt += kHadWaves) {
#pragma unroll
      for (int nt = 0; nt < B / 16; ++nt) {
        f32x4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int ks = 0; ks < B / 32; ++ks) {
          const bf16x8_t hf =
              *reinterpret_cast<const bf16x8_t*>(&Mbt[(nt * 16 + l16) * XP + ks * 32 + 8 * lq]);
#pragma unroll
          for (int s = 0; s < NS; ++s) {
            const bf16x8_t xf = *reinterpret_cast<const bf16x8_t*>(
                &Xs[(s * S + mt * 16 + l16) * XP + ks * 32 + 8 * lq]);
            if constexpr (A == 1) {
              // D^T = Mb^T * X^T: lane holds 4 neighbouring output columns of one sub-row
              acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(hf, xf, acc, 0, 0, 0);
            } else {
              // D = X * Mb: lane holds 4 neighbouring sub-rows of one column
              acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xf, hf, acc, 0, 0, 0);
            }
          }
        }
        if constexpr (A == 1) {
          const int row = mt * 16 + l16, col = nt * 16 + 4 * lq;
          Vec<R, 4> o;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            float v = acc[r] / a.sqrt_n;
            if (a.s_out) v *= a.s_out[col + r];
            o.v[r] = IO::from_f32(v);
          }
          *reinterpret_cast<Vec<R, 4>*>(&Os[row * OP + col]) = o;
        } else {
          const int col = nt * 16 + l16, row = mt * 16 + 4 * lq;
          Vec<uint16_t, 4> p[3];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            uint16_t parts[3];
            split_bf16<3>(acc[r], parts);
            p[0].v[r] = parts[0];
            p[1].v[r] = parts[1];
            p[2].v[r] = parts[2];
          }
#pragma unroll
          for (int s = 0; s < 3; ++s)
            *reinterpret_cast<Vec<uint16_t, 4>*>(&Tt[(s * B + col) * TP + row]) = p[s];
        }
      }
    }

    if constexpr (A > 1) {
      __syncthreads();
      // ---- stage 2: Y = Ma^T * T per data row; computed as Y^T = T^T * Ma so that a
      // lane ends up with 4 neighbouring columns of one output sub-row
      constexpr int MT = B / 16, NT = A / 16, PER_ROW = MT * NT;
      for (int q = wave; q < (S / A) * PER_ROW; q += kHadWaves) {
        const int d = q / PER_ROW, mt = (q % PER_ROW) / NT, nt = q % NT;
        f32x4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int ks = 0; ks < A / 32; ++ks) {
          const bf16x8_t mf =
              *reinterpret_cast<const bf16x8_t*>(&Mat[(nt * 16 + l16) * AP + ks * 32 + 8 * lq]);
#pragma unroll
          for (int s = 0; s < 3; ++s) {
            const bf16x8_t tf = *reinterpret_cast<const bf16x8_t*>(
                &Tt[(s * B + mt * 16 + l16) * TP + d * A + ks * 32 + 8 * lq]);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(tf, mf, acc, 0, 0, 0);
          }
        }
        const int i = nt * 16 + l16;           // output sub-row inside the data row
        const int col = mt * 16 + 4 * lq;
        Vec<R, 4> o;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float v = acc[r] / a.sqrt_n;
          if (a.s_out) v *= a.s_out[i * B + col + r];
          o.v[r] = IO::from_f32(v);
        }
        *reinterpret_cast<Vec<R, 4>*>(&Os[(d * A + i) * OP + col]) = o;
      }
    }
    __syncthreads();

    // ---- LDS -> global
    for (int e = tid * VE; e < S * B; e += kHadThreads * VE) {
      if (e < live) {
        const int row = e / B, col = e % B;
        stg_nt<R, VE>(dst + e, *reinterpret_cast<const Vec<R, VE>*>(&Os[row * OP + col]));
      }
    }
  }
}

// ---------------------------------------------------------------- block sizes up to 128, bf16 / float16
// One wavefront owns 16 sub-rows at a time and never talks to another wave.  The 16
// sub-rows are one stretch of memory; the wavefront loads and stores it lanes side by
// side, whole memory lines per instruction, and passes it through an image in LDS of
// its own on the way to the operand layout and back (the operand layout itself asks a
// lane group for half a line per instruction and the other half with the next; read
// and written that way the kernel was 7 % slower at 128, 20 % at 64).  Accesses are
// plain ones: streaming loads cost 2 %, streaming stores 5-10 %.
// With D^T = Mb^T * X^T on v_mfma_f32_16x16x32_bf16 the operand layouts line up
// with memory on both sides:
//   B operand (X^T): lane (i + 16 q) holds X[row i][32 ks + 8 q .. + 8], one
//                    16-byte global load;
//   A operand:       rows of Mb^T, fetched once per wave and kept in registers
//                    for every tile the wave handles, with the signs folded in
//                    (row c times sign_out[c], column k times sign_in[k]);
//   D^T:             lane (i + 16 jq) holds 4 output columns of row i.  Which 4
//                    is a matter of labelling the rows of the A operand: tiles
//                    2p and 2p+1 are given the columns 32 p + 8 jq + {0..3} and
//                    + {4..7}, so a lane ends up with 8 neighbouring outputs,
//                    one 16-byte global store.
// Sign vectors are used as signs: their entries must be +1 or -1.
template <int B, bool HALF, bool MANY>
__global__ void __launch_bounds__(kRowsThreads)
hadamard_rows_kernel(HadJobs jobs, int64_t n_full, int ragged_sub,
                     const uint16_t* __restrict__ mbt, const float* __restrict__ s_in,
                     const float* __restrict__ s_out, float inv_sqrt_n) {
  constexpr int KS = B / 32;  // k steps
  constexpr int NP = B / 32;  // pairs of 16-column output tiles
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // uniform: loop control stays scalar
  const int l16 = lane & 15, lq = lane >> 4;
  // HALF: float16 tensors on v_mfma_f32_16x16x32_f16; the matrix arrives in bfloat16
  // and converts to float16 exactly (more significand bits, entries of order 1)
  using frag_t = typename std::conditional<HALF, f16x8_t, bf16x8_t>::type;

  // The matrix fragments are the same in every wave of the workgroup: each wave
  // fetches a quarter of them, and all pick up the whole set from LDS.
  __shared__ u32x4_t frag_lds[2 * NP * KS][kWave];
  for (int f = wave; f < 2 * NP * KS; f += kRowsWaves) {
    const int nt = f / KS, ks = f % KS;
    const int col = 32 * (nt / 2) + 8 * (l16 / 4) + 4 * (nt % 2) + (l16 % 4);
    u32x4_t m = *reinterpret_cast<const u32x4_t*>(mbt + col * B + 32 * ks + 8 * lq);
    if constexpr (HALF) {
#pragma unroll
      for (int w = 0; w < 4; ++w)
        m[w] = (uint32_t)f32_to_f16(bf16_lo(m[w])) | ((uint32_t)f32_to_f16(bf16_hi(m[w])) << 16);
    }
    frag_lds[f][lane] = m;
  }
  __syncthreads();
  frag_t mb[2 * NP][KS];
#pragma unroll
  for (int nt = 0; nt < 2 * NP; ++nt)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      mb[nt][ks] = __builtin_bit_cast(frag_t, frag_lds[nt * KS + ks][lane]);
  if (s_in || s_out) {
    // Sign bits, XORed into the fragments (bit 15 of each half word).  An absent
    // vector reads the matrix instead (any valid address) and is masked out: no
    // branches, so these loads overlap too.
    const uint32_t* pin = reinterpret_cast<const uint32_t*>(s_in ? (const void*)s_in : (const void*)mbt);
    const uint32_t* pout = reinterpret_cast<const uint32_t*>(s_out ? (const void*)s_out : (const void*)mbt);
    const uint32_t use_in = s_in ? 1u : 0u, use_out = s_out ? 0x80008000u : 0u;
    uint32_t raw_in[KS][8], raw_out[2 * NP];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int e = 0; e < 8; ++e) raw_in[ks][e] = pin[32 * ks + 8 * lq + e];
#pragma unroll
    for (int nt = 0; nt < 2 * NP; ++nt)
      raw_out[nt] = pout[32 * (nt / 2) + 8 * (l16 / 4) + 4 * (nt % 2) + (l16 % 4)];
#pragma unroll
    for (int nt = 0; nt < 2 * NP; ++nt) {
      const uint32_t fo = (raw_out[nt] >> 31) * use_out;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        Vec<uint32_t, 4> m = __builtin_bit_cast(Vec<uint32_t, 4>, mb[nt][ks]);
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const uint32_t lo = (raw_in[ks][2 * w] >> 31) & use_in, hi = (raw_in[ks][2 * w + 1] >> 31) & use_in;
          m.v[w] ^= ((lo << 15) | (hi << 31)) ^ fo;
        }
        mb[nt][ks] = __builtin_bit_cast(frag_t, m);
      }
    }
  }

  // n_full: whole groups of 16 sub-rows, over all jobs
  const int64_t stride = (int64_t)gridDim.x * kRowsWaves;
  const int64_t first = (int64_t)blockIdx.x * kRowsWaves + wave;

  auto pack2 = [&](float lo, float hi) -> uint32_t {
    if constexpr (HALF) return (uint32_t)f32_to_f16(lo) | ((uint32_t)f32_to_f16(hi) << 16);
    else return pack_bf16x2(lo, hi);
  };
  auto transform_rows = [&](const frag_t* xf, uint16_t* dst, bool keep) {
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      f32x4_t a0 = {0.0f, 0.0f, 0.0f, 0.0f}, a1 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        if constexpr (HALF) {
          a0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(mb[2 * p][ks], xf[ks], a0, 0, 0, 0);
          a1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(mb[2 * p + 1][ks], xf[ks], a1, 0, 0, 0);
        } else {
          a0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(mb[2 * p][ks], xf[ks], a0, 0, 0, 0);
          a1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(mb[2 * p + 1][ks], xf[ks], a1, 0, 0, 0);
        }
      }
      Vec<uint32_t, 4> o;
      o.v[0] = pack2(a0[0] * inv_sqrt_n, a0[1] * inv_sqrt_n);
      o.v[1] = pack2(a0[2] * inv_sqrt_n, a0[3] * inv_sqrt_n);
      o.v[2] = pack2(a1[0] * inv_sqrt_n, a1[1] * inv_sqrt_n);
      o.v[3] = pack2(a1[2] * inv_sqrt_n, a1[3] * inv_sqrt_n);
      if (keep) stg<uint16_t, 8>(dst + 32 * p, __builtin_bit_cast(Vec<uint16_t, 8>, o));
    }
  };
  // A group of 16 sub-rows is one stretch of 32 B bytes in memory.  It is loaded and
  // stored as such, lanes side by side (every instruction whole memory lines), and
  // turned into the operand layout and back in an image of the group in LDS that
  // belongs to the wavefront alone: no barrier.  Sub-rows are 16 bytes further apart
  // than they are long, so that the 16 lanes that read one column of pieces hit
  // different banks.
  constexpr int kPitch = (2 * B + 16) / 4;  // dwords between sub-rows of the image
  constexpr int kPieces = B / 8;            // 16-byte pieces of a sub-row
  __shared__ __attribute__((aligned(16))) uint32_t image_lds[kRowsWaves][16 * kPitch];
  uint32_t* const img = image_lds[wave];
  // piece j of the stretch, and the piece of sub-row l16 at columns 32 t + 8 lq
  auto linear_at = [&](int j) { return (j / kPieces) * kPitch + (j % kPieces) * 4; };
  auto operand_at = [&](int t) { return l16 * kPitch + 16 * t + 4 * lq; };
  // Loads are never conditional (a group past the end re-reads the last whole one)
  // and the stores of whole groups are not either: with a fixed number of memory
  // operations per step the waits can say exactly how many newer operations may
  // still be in flight.  Where the group's outputs go is looked up together with
  // where its inputs are.
  auto load_block = [&](int64_t grp, u32x4_t* raw, uint16_t** dst) {
    if (grp >= n_full) grp = n_full - 1;
    int64_t local;
    const int j = had_job<MANY>(jobs, grp, &local);
    const int64_t at = local * 16 * B + lane * 8;
    const uint16_t* src = static_cast<const uint16_t*>(jobs.x[j]) + at;
    *dst = static_cast<uint16_t*>(jobs.out[j]) + at;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      raw[ks] = __builtin_bit_cast(u32x4_t, ldg<uint16_t, 8>(src + 512 * ks));
  };
  if (first < n_full) {
    u32x4_t raw[KS];
    uint16_t *dst, *dst_next;
    int64_t g = first;
    load_block(g, raw, &dst);
    // The first group is handled ahead of the loop so that the loop is entered with
    // the same operations in flight as on its back edge (a group's loads, then a
    // group's stores): the wait for the loads then leaves the stores in flight.
    auto step = [&]() {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        *reinterpret_cast<u32x4_t*>(&img[linear_at(ks * kWave + lane)]) = raw[ks];
      load_block(g + stride, raw, &dst_next);
      frag_t xf[KS];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        xf[ks] = __builtin_bit_cast(frag_t, *reinterpret_cast<const u32x4_t*>(&img[operand_at(ks)]));
#pragma unroll
      for (int p = 0; p < NP; ++p) {
        f32x4_t a0 = {0.0f, 0.0f, 0.0f, 0.0f}, a1 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          if constexpr (HALF) {
            a0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(mb[2 * p][ks], xf[ks], a0, 0, 0, 0);
            a1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(mb[2 * p + 1][ks], xf[ks], a1, 0, 0, 0);
          } else {
            a0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(mb[2 * p][ks], xf[ks], a0, 0, 0, 0);
            a1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(mb[2 * p + 1][ks], xf[ks], a1, 0, 0, 0);
          }
        }
        u32x4_t o;
        o[0] = pack2(a0[0] * inv_sqrt_n, a0[1] * inv_sqrt_n);
        o[1] = pack2(a0[2] * inv_sqrt_n, a0[3] * inv_sqrt_n);
        o[2] = pack2(a1[0] * inv_sqrt_n, a1[1] * inv_sqrt_n);
        o[3] = pack2(a1[2] * inv_sqrt_n, a1[3] * inv_sqrt_n);
        *reinterpret_cast<u32x4_t*>(&img[operand_at(p)]) = o;
      }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const u32x4_t r = *reinterpret_cast<const u32x4_t*>(&img[linear_at(ks * kWave + lane)]);
        stg<uint16_t, 8>(dst + 512 * ks, __builtin_bit_cast(Vec<uint16_t, 8>, r));
      }
      dst = dst_next;
      g += stride;
    };
    step();
    while (g < n_full) step();
  }
  // the ragged last group (fewer than 16 sub-rows; single tensors only), by the wave
  // whose turn it is
  if (ragged_sub != 0 && n_full % stride == first) {
    const int64_t n_sub = n_full * 16 + ragged_sub;
    const uint16_t* x = static_cast<const uint16_t*>(jobs.x[0]);
    uint16_t* out = static_cast<uint16_t*>(jobs.out[0]);
    int64_t row = n_full * 16 + l16;
    const bool keep = row < n_sub;
    if (!keep) row = n_sub - 1;
    frag_t xt[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      xt[ks] = __builtin_bit_cast(frag_t, ldg<uint16_t, 8>(x + row * B + 8 * lq + 32 * ks));
    transform_rows(xt, out + row * B + 8 * lq, keep);
  }
}

static void clear_jobs(HadJobs* t) {
  for (int k = 0; k < kHadMaxJobs; ++k) {
    t->x[k] = nullptr;
    t->out[k] = t->scale[k] = t->rotated[k] = nullptr;
    t->end[k] = INT64_MAX;
    t->n_sub[k] = 0;
  }
}

// jobs: whole groups of 16 sub-rows per tensor, except that a single tensor may end
// in a ragged group
template <int B, bool HALF>
static int launch_had_rows_jobs(const HadJobs& jobs, int n_jobs, const HadArgs& a, hipStream_t st) {
  const int64_t n_full = n_jobs == 1 ? jobs.n_sub[0] / 16 : jobs.end[n_jobs - 1];
  const int ragged = n_jobs == 1 ? (int)(jobs.n_sub[0] % 16) : 0;
  const int64_t wgs = cdiv(n_full + (ragged ? 1 : 0), kRowsWaves);
  // a wave keeps the matrix in registers: give it several groups to use it on
  // (as many wavefronts as fit on the chip at once: 8 per CU at 128, where a wave
  // needs some 190 registers, more below)
  const int64_t cap = 256 * (B == 32 ? 16 : 8) / kRowsWaves;
  const unsigned grid = (unsigned)(wgs < cap ? wgs : cap);
  if (n_jobs == 1)
    hipLaunchKernelGGL((hadamard_rows_kernel<B, HALF, false>), grid, kRowsThreads, 0, st, jobs, n_full,
                       ragged, a.mbt, a.s_in, a.s_out, 1.0f / a.sqrt_n);
  else
    hipLaunchKernelGGL((hadamard_rows_kernel<B, HALF, true>), grid, kRowsThreads, 0, st, jobs, n_full,
                       ragged, a.mbt, a.s_in, a.s_out, 1.0f / a.sqrt_n);
  return CTMI_OK;
}

// ---------------------------------------------------------------- rotation + int4 group quantization + packing
// hadamard_rows_kernel with the rest of the W4A16 pipeline in its epilogue, for
// group size == block size B: the rotated sub-row (rounded to bf16, as the
// stand-alone transform stores it) IS one quantization group, so its min / max,
// calculate_qparams (helpers.py:67-146, symmetric), _quantize (forward.py:455-487)
// and pack_to_int32 (pack_quantized.py:186-246) follow in registers.  The bits are
// those of the three separate steps; the rotated tensor never goes to memory
// (unless `rotated` asks for it).  A sub-row's 128 outputs sit in the 4 lanes
// l16 + 16 q; they agree on min / max through two lane exchanges.
#ifndef CTMI_HQP_LOAD
#define CTMI_HQP_LOAD ldg
#endif
#ifndef CTMI_HQP_STORE
#define CTMI_HQP_STORE stg
#endif
#ifndef CTMI_HQP_MIN_WAVES
#define CTMI_HQP_MIN_WAVES 4  // wavefronts per SIMD the kernel is compiled for
#endif
template <int B, bool MANY>
__global__ void __launch_bounds__(kHqpThreads, CTMI_HQP_MIN_WAVES)
hadamard_quant_pack_kernel(HadJobs jobs, int64_t n_groups, const uint16_t* __restrict__ mbt,
                           const float* __restrict__ s_in, const float* __restrict__ s_out,
                           float inv_sqrt_n, QpCfg cfg) {
  constexpr int KS = B / 32, NP = B / 32;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int l16 = lane & 15, lq = lane >> 4;

  // The matrix fragments stay in LDS, in the lanes' own layout, and are read at
  // each use (16 bytes per lane, conflict free): with the epilogue's registers on
  // top of 128 for the matrix only one wavefront per SIMD would fit, and it is
  // the number of wavefronts in flight that hides the memory latency here.
  __shared__ u32x4_t frag_lds[2 * NP * KS][kWave];
  __shared__ __align__(16) int32_t swap_lds[kHqpWaves][16][16];
  for (int f = wave; f < 2 * NP * KS; f += kHqpWaves) {
    const int nt = f / KS, ks = f % KS;
    const int col = 32 * (nt / 2) + 8 * (l16 / 4) + 4 * (nt % 2) + (l16 % 4);
    u32x4_t m = *reinterpret_cast<const u32x4_t*>(mbt + col * B + 32 * ks + 8 * lq);
    if (s_in || s_out) {
      const uint32_t fo = s_out ? ((f2u(s_out[col]) >> 31) * 0x80008000u) : 0u;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const int k0 = 32 * ks + 8 * lq + 2 * w;
        const uint32_t lo = s_in ? (f2u(s_in[k0]) >> 31) : 0u, hi = s_in ? (f2u(s_in[k0 + 1]) >> 31) : 0u;
        m[w] ^= ((lo << 15) | (hi << 31)) ^ fo;
      }
    }
    frag_lds[f][lane] = m;
  }
  __syncthreads();

  // n_groups: groups of 16 sub-rows over all jobs (a job's last one may be ragged)
  const int64_t stride = (int64_t)gridDim.x * kHqpWaves;
  // where a group's sub-rows are and go, and its loads
  struct Place {
    int j;
    int64_t row;
    bool keep;
  };
  auto place_of = [&](int64_t g) {
    if (g >= n_groups) g = n_groups - 1;  // past the end: the last group again, nothing stored
    int64_t local;
    Place pl;
    pl.j = had_job<MANY>(jobs, g, &local);
    pl.row = local * 16 + l16;
    pl.keep = pl.row < jobs.n_sub[pl.j];
    if (!pl.keep) pl.row = jobs.n_sub[pl.j] - 1;  // ragged last group: the last sub-row again
    return pl;
  };
  auto fetch = [&](const Place& pl, bf16x8_t* xf) {
    const uint16_t* src = static_cast<const uint16_t*>(jobs.x[pl.j]) + pl.row * B + 8 * lq;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      xf[ks] = __builtin_bit_cast(bf16x8_t, CTMI_HQP_LOAD<uint16_t, 8>(src + 32 * ks));
  };
  // A wavefront takes G groups at a time (neighbours in memory): every fragment of the matrix
  // it reads from LDS then serves G products.
  constexpr int G = CTMI_HQP_GROUPS;
  for (int64_t g = ((int64_t)blockIdx.x * kHqpWaves + wave) * G; g < n_groups; g += stride * G) {
    Place here[G];
    bf16x8_t xf[G][KS];
#pragma unroll
    for (int t = 0; t < G; ++t) {
      here[t] = place_of(g + t);
      here[t].keep = here[t].keep && g + t < n_groups;
      fetch(here[t], xf[t]);
    }
    Vec<uint32_t, 4> o[G][NP];  // the rotated sub-rows in bf16: columns 32 p + 8 lq .. + 8
    // A symmetric scale only needs max |x| of the group (min(min,0) and max(max,0)
    // enter through their magnitudes, helpers.py:87-104).  Magnitudes of bf16
    // values order like their bit patterns, a NaN above everything: the maximum is
    // taken on the packed 16-bit halves, two elements per instruction.
    typedef uint16_t u16x2_t __attribute__((ext_vector_type(2)));
    u16x2_t top[G];
#pragma unroll
    for (int t = 0; t < G; ++t) top[t] = u16x2_t{0, 0};
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      f32x4_t a0[G], a1[G];
#pragma unroll
      for (int t = 0; t < G; ++t) a0[t] = a1[t] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
      // keeps the compiler from hoisting these (loop-invariant) LDS reads out of
      // the loop, back into 128 registers
      asm volatile("" ::: "memory");
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const bf16x8_t m0 = __builtin_bit_cast(bf16x8_t, frag_lds[(2 * p) * KS + ks][lane]);
        const bf16x8_t m1 = __builtin_bit_cast(bf16x8_t, frag_lds[(2 * p + 1) * KS + ks][lane]);
#pragma unroll
        for (int t = 0; t < G; ++t) {
          a0[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(m0, xf[t][ks], a0[t], 0, 0, 0);
          a1[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(m1, xf[t][ks], a1[t], 0, 0, 0);
        }
      }
#ifdef CTMI_HQP_DIAG_NOMFMA
#pragma unroll
      for (int t = 0; t < G; ++t) {
        o[t][p] = __builtin_bit_cast(Vec<uint32_t, 4>, xf[t][p]);
#pragma unroll
        for (int w = 0; w < 4; ++w)
          top[t] = __builtin_elementwise_max(top[t], __builtin_bit_cast(u16x2_t, o[t][p].v[w] & 0x7FFF7FFFu));
      }
      continue;
#endif
#pragma unroll
      for (int t = 0; t < G; ++t) {
        o[t][p].v[0] = pack_bf16x2(a0[t][0] * inv_sqrt_n, a0[t][1] * inv_sqrt_n);
        o[t][p].v[1] = pack_bf16x2(a0[t][2] * inv_sqrt_n, a0[t][3] * inv_sqrt_n);
        o[t][p].v[2] = pack_bf16x2(a1[t][0] * inv_sqrt_n, a1[t][1] * inv_sqrt_n);
        o[t][p].v[3] = pack_bf16x2(a1[t][2] * inv_sqrt_n, a1[t][3] * inv_sqrt_n);
#pragma unroll
        for (int w = 0; w < 4; ++w)
          top[t] = __builtin_elementwise_max(top[t], __builtin_bit_cast(u16x2_t, o[t][p].v[w] & 0x7FFF7FFFu));
      }
    }
#pragma unroll
    for (int t = 0; t < G; ++t) {
      const int j = here[t].j;
      int32_t* packed = static_cast<int32_t*>(jobs.out[j]);
      uint16_t* scale = static_cast<uint16_t*>(jobs.scale[j]);
      uint16_t* rotated = static_cast<uint16_t*>(jobs.rotated[j]);
      const int64_t row = here[t].row;
      const bool keep = here[t].keep;
      uint32_t mag = top[t].x > top[t].y ? top[t].x : top[t].y;
#pragma unroll
      for (int d = 16; d < 64; d <<= 1) {
        const uint32_t other = (uint32_t)__shfl_xor((int)mag, d, kWave);
        mag = other > mag ? other : mag;
      }
      // calculate_qparams, symmetric, in bf16 (helpers.py:101-122); 7.5 is a bf16 value: the
      // product with its reciprocal rounds to the same bf16 as the quotient
      const float sv = symmetric_scale<BF16>(bf16_to_f32((uint16_t)mag), mag > 0x7F80u, cfg.sym_div);
      // Packed word 4 p + lq of the sub-row comes out of lane (l16, lq) for pair p.
      // The 4 lanes of a sub-row swap words through a wave-private patch of LDS so
      // that each stores NP neighbouring words (16 bytes at B = 128) instead of NP
      // single ones 16 bytes apart.
      int32_t* swap = &swap_lds[wave][l16][0];
#pragma unroll
      for (int p = 0; p < NP; ++p) {
#ifdef CTMI_HQP_DIAG_NOQUANT
        Vec<int32_t, 1> w;
        w.v[0] = (int32_t)(o[t][p].v[0] ^ o[t][p].v[1] ^ o[t][p].v[2] ^ o[t][p].v[3]) + (int32_t)__float_as_uint(sv);
#else
        const Vec<int32_t, 1> w = quant_pack8<BF16, BF16, 4, false>(
            __builtin_bit_cast(Vec<uint16_t, 8>, o[t][p]), sv, 0.0f, cfg.bit_min, cfg.bit_max);
#endif
        swap[4 * p + lq] = w.v[0];
        if (rotated && keep)
          stg<uint16_t, 8>(rotated + row * B + 32 * p + 8 * lq, __builtin_bit_cast(Vec<uint16_t, 8>, o[t][p]));
      }
      asm volatile("" ::: "memory");  // the reads below are of other lanes' words
      if (keep) {
        if (lq == 0) scale[row] = f32_to_bf16(sv);
        if (lq < NP) {
          Vec<int32_t, 4> out4;
#pragma unroll
          for (int j4 = 0; j4 < 4; ++j4) out4.v[j4] = swap[4 * lq + j4];
          CTMI_HQP_STORE<int32_t, 4>(packed + row * (B / 8) + 4 * lq, out4);
        }
      }
      asm volatile("" ::: "memory");  // the next group's words must not overtake these reads
    }
  }
}

// ---------------------------------------------------------------- the same for Sylvester's matrix of 128
// hadamard_quant_pack_kernel for the matrix the reference uses at this size (Sylvester's H_128,
// with or without sign vectors; transform/utils/hadamard.py:65-100), with no matrix in memory:
// H[k][c] = (-1)^popcount(k & c) splits, for the operand layout above (k = 32 ks + 8 q + e,
// c = 32 p + 8 (m / 4) + 4 b + m % 4 for row m of tile 2 p + b), into
//     (-1)^popcount(ks & p)  *  (-1)^(popcount(q & (m / 4)) + popcount(e & (4 b + m % 4))):
// two fragments (b = 0, 1) a lane keeps in 8 registers serve all 32 products, and the sign
// in front goes to the other operand (the sub-rows, negated once per group).  Sign vectors are
// applied as sign-bit masks to the inputs and to the rounded outputs.  Without a matrix to set
// up, a workgroup takes one chunk of sub-rows and exits (no loop over the tensor, no barrier),
// like the streaming kernels of the other formats.
#ifndef CTMI_SQP_GROUPS
#define CTMI_SQP_GROUPS 2  // groups of 16 sub-rows a wavefront takes
#endif
#ifndef CTMI_SQP_FP32_MAX
#define CTMI_SQP_FP32_MAX 1  // max |x| on the fp32 values (one instruction per two) or on the packed bf16 ones
#endif
#ifndef CTMI_SQP_NEG_FRAG
#define CTMI_SQP_NEG_FRAG 0  // the sign in front of a product on the fragment (1) or on the sub-rows (0)
#endif
#ifndef CTMI_SQP_IMAGE
#define CTMI_SQP_IMAGE 1  // whole groups are loaded as stretches of memory and reordered in LDS
#endif
#ifndef CTMI_SQP_LOAD
#define CTMI_SQP_LOAD ldg_nt
#endif
#ifndef CTMI_SQP_STORE
#define CTMI_SQP_STORE stg_nt
#endif
constexpr int kSqpThreads = 256;
constexpr int kSqpWaves = kSqpThreads / kWave;

#ifndef CTMI_SQP_MIN_WAVES
#define CTMI_SQP_MIN_WAVES 4
#endif
// QUANT = false: the rotation alone (jobs.out takes the rotated sub-rows, whole groups on
// their way out through the image as well, so that loads and stores are both whole lines).
#ifndef CTMI_SR_GROUPS
#define CTMI_SR_GROUPS 1  // the rotation alone: groups of 16 sub-rows a wavefront takes (14336x4096: 1: 0.76 of the HBM peak, 2: 0.73, 4: 0.69)
#endif
#ifndef CTMI_SR_STORE
#define CTMI_SR_STORE stg_nt
#endif
#ifndef CTMI_SR_IMAGE_MANY
#define CTMI_SR_IMAGE_MANY 1  // the rotation alone: launches over several tensors use the image too
#endif
template <bool MANY, bool SIGN_IN, bool SIGN_OUT, bool QUANT = true>
__global__ void __launch_bounds__(kSqpThreads, CTMI_SQP_MIN_WAVES)
sylvester128_quant_pack_kernel(HadJobs jobs, int64_t n_groups, const float* __restrict__ s_in,
                    const float* __restrict__ s_out, float inv_sqrt_n, QpCfg cfg) {
  constexpr int B = 128, KS = 4, NP = 4, G = QUANT ? CTMI_SQP_GROUPS : CTMI_SR_GROUPS;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int l16 = lane & 15, lq = lane >> 4;
  const int64_t g0 = ((int64_t)blockIdx.x * kSqpWaves + wave) * G;
  if (g0 >= n_groups) return;

  // Where the groups' sub-rows are, and their loads (all issued before anything else).  A
  // group of 16 sub-rows is one stretch of 4 KB: whole groups are loaded as such, lanes side
  // by side (whole memory lines per instruction), and reach the operand layout through an
  // image in LDS that belongs to the wavefront alone (no barrier); sub-rows of the image lie
  // 16 bytes further apart than they are long, so that the 16 lanes that read one column of
  // pieces hit different banks.  A ragged last group is loaded in the operand layout directly.
  // (launches over several tensors load in the operand layout throughout: with the image they
  // measured 10 % slower, launches of one tensor 6 % faster)
  constexpr bool kImage = QUANT ? (CTMI_SQP_IMAGE && !MANY) : (!MANY || CTMI_SR_IMAGE_MANY);
  constexpr int kPitch = (2 * B + 16) / 4;  // dwords between sub-rows of the image
  __shared__ __attribute__((aligned(16))) uint32_t image_lds[kSqpWaves][kImage ? G * 16 * kPitch : 1];
  int job[G];
  int64_t row[G];
  bool keep[G], whole[G];
  bf16x8_t xf[G][KS];
#pragma unroll
  for (int t = 0; t < G; ++t) {
    int64_t g = g0 + t, local;
    const bool live = g < n_groups;
    if (!live) g = n_groups - 1;  // past the end: the last group again, nothing stored
    job[t] = had_job<MANY>(jobs, g, &local);
    row[t] = local * 16 + l16;
    keep[t] = live && row[t] < jobs.n_sub[job[t]];
    whole[t] = kImage && local * 16 + 16 <= jobs.n_sub[job[t]];  // wave-uniform
    if (row[t] >= jobs.n_sub[job[t]]) row[t] = jobs.n_sub[job[t]] - 1;  // ragged last group
    const uint16_t* base = static_cast<const uint16_t*>(jobs.x[job[t]]);
    const uint16_t* src = whole[t] ? base + local * 16 * B + lane * 8 : base + row[t] * B + 8 * lq;
    const int step = whole[t] ? 512 : 32;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      xf[t][ks] = __builtin_bit_cast(bf16x8_t, CTMI_SQP_LOAD<uint16_t, 8>(src + step * ks));
  }
  // sign-bit masks of this lane's inputs (k = 32 ks + 8 lq + e) and outputs (c = 32 p + 8 lq + e)
  uint32_t flip_in[SIGN_IN ? KS : 1][4], flip_out[SIGN_OUT ? NP : 1][4];
  auto masks = [&](const float* __restrict__ signs, uint32_t (*flip)[4]) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const Vec<uint32_t, 4> lo = ldg<uint32_t, 4>(reinterpret_cast<const uint32_t*>(signs) + 32 * q + 8 * lq);
      const Vec<uint32_t, 4> hi = ldg<uint32_t, 4>(reinterpret_cast<const uint32_t*>(signs) + 32 * q + 8 * lq + 4);
      flip[q][0] = ((lo.v[0] >> 16) & 0x8000u) | (lo.v[1] & 0x80000000u);
      flip[q][1] = ((lo.v[2] >> 16) & 0x8000u) | (lo.v[3] & 0x80000000u);
      flip[q][2] = ((hi.v[0] >> 16) & 0x8000u) | (hi.v[1] & 0x80000000u);
      flip[q][3] = ((hi.v[2] >> 16) & 0x8000u) | (hi.v[3] & 0x80000000u);
    }
  };
  if constexpr (SIGN_IN) masks(s_in, flip_in);
  if constexpr (SIGN_OUT) masks(s_out, flip_out);
  // the two fragments: entry e of row m = l16 in the k block of lane quarter lq
  u32x4_t frag[2];
#pragma unroll
  for (int b = 0; b < 2; ++b)
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const uint32_t rowbits = (uint32_t)(4 * b + (l16 & 3));
      const uint32_t common = (uint32_t)__builtin_popcount(lq & (l16 >> 2));
      const uint32_t lo = ((common + __builtin_popcount((2 * d) & rowbits)) & 1u) ? 0xBF80u : 0x3F80u;
      const uint32_t hi = ((common + __builtin_popcount((2 * d + 1) & rowbits)) & 1u) ? 0xBF80u : 0x3F80u;
      frag[b][d] = lo | (hi << 16);
    }
  const bf16x8_t f0 = __builtin_bit_cast(bf16x8_t, frag[0]), f1 = __builtin_bit_cast(bf16x8_t, frag[1]);
#if CTMI_SQP_NEG_FRAG
  const bf16x8_t f0n = __builtin_bit_cast(bf16x8_t, frag[0] ^ 0x80008000u);
  const bf16x8_t f1n = __builtin_bit_cast(bf16x8_t, frag[1] ^ 0x80008000u);
#endif

#pragma unroll
  for (int t = 0; t < G; ++t) {
    if (whole[t]) {
      // piece j of the stretch is piece j % 16 of sub-row j / 16; the operand wants the piece
      // of sub-row l16 at columns 32 ks + 8 lq
      uint32_t* img = &image_lds[wave][t * 16 * kPitch];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int j = ks * kWave + lane;
        *reinterpret_cast<u32x4_t*>(&img[(j >> 4) * kPitch + (j & 15) * 4]) = __builtin_bit_cast(u32x4_t, xf[t][ks]);
      }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        xf[t][ks] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4_t*>(&img[l16 * kPitch + 16 * ks + 4 * lq]));
    }
    if constexpr (SIGN_IN) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        u32x4_t xs = __builtin_bit_cast(u32x4_t, xf[t][ks]);
#pragma unroll
        for (int d = 0; d < 4; ++d) xs[d] ^= flip_in[ks][d];
        xf[t][ks] = __builtin_bit_cast(bf16x8_t, xs);
      }
    }
#if !CTMI_SQP_NEG_FRAG
    bf16x8_t xneg[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      xneg[ks] = __builtin_bit_cast(bf16x8_t, __builtin_bit_cast(u32x4_t, xf[t][ks]) ^ 0x80008000u);
#endif
    Vec<uint32_t, 4> o[NP];  // the rotated sub-row in bf16: columns 32 p + 8 lq .. + 8
    // max |x| of what this lane holds, on the fp32 values before they are rounded (rounding
    // is monotonic: the largest magnitude stays the largest).  The maximum drops NaNs, and the
    // min-max observer must not: a NaN among the inputs makes every output of the sub-row a
    // NaN (one look at one value finds it), infinities among them make every output an
    // infinity or a NaN (the maximum is then infinite); both go the exact way below.
#if CTMI_SQP_FP32_MAX
    float top = 0.0f;
    bool odd = false;
#else
    typedef uint16_t u16x2_t __attribute__((ext_vector_type(2)));
    u16x2_t top2 = {0, 0};
#endif
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      f32x4_t a0 = {0.0f, 0.0f, 0.0f, 0.0f}, a1 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const bool minus = (__builtin_popcount(ks & p) & 1) != 0;
#if CTMI_SQP_NEG_FRAG
        a0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(minus ? f0n : f0, xf[t][ks], a0, 0, 0, 0);
        a1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(minus ? f1n : f1, xf[t][ks], a1, 0, 0, 0);
#else
        const bf16x8_t xk = minus ? xneg[ks] : xf[t][ks];
        a0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f0, xk, a0, 0, 0, 0);
        a1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f1, xk, a1, 0, 0, 0);
#endif
      }
      float v[8];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v[e] = a0[e] * inv_sqrt_n;
        v[4 + e] = a1[e] * inv_sqrt_n;
      }
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        o[p].v[w] = pack_bf16x2(v[2 * w], v[2 * w + 1]);
        if constexpr (SIGN_OUT) o[p].v[w] ^= flip_out[p][w];
        if constexpr (QUANT) {
#if CTMI_SQP_FP32_MAX
          top = __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf(v[2 * w]), __builtin_fabsf(v[2 * w + 1])), top);
#else
          top2 = __builtin_elementwise_max(top2, __builtin_bit_cast(u16x2_t, o[p].v[w] & 0x7FFF7FFFu));
#endif
        }
      }
#if CTMI_SQP_FP32_MAX
      if (QUANT && p == 0) odd = v[0] != v[0];
#endif
    }
    // A sum that cancels exactly is +0 whatever the column's sign (the sign belongs to the
    // matrix, the accumulator starts at +0): zeros among the outputs that leave as rotated
    // values give back the sign bit the mask put on them.
    auto unsigned_zeros = [](uint32_t w) -> uint32_t {
      typedef uint16_t u16x2_t __attribute__((ext_vector_type(2)));
      const u16x2_t one = {1, 1};
      const u16x2_t nz = __builtin_elementwise_min(__builtin_bit_cast(u16x2_t, w & 0x7FFF7FFFu), one);
      return w & ((__builtin_bit_cast(uint32_t, nz) << 15) | 0x7FFF7FFFu);
    };
    if constexpr (!QUANT) {
      if constexpr (SIGN_OUT) {
#pragma unroll
        for (int p = 0; p < NP; ++p)
#pragma unroll
          for (int w = 0; w < 4; ++w) o[p].v[w] = unsigned_zeros(o[p].v[w]);
      }
      uint16_t* dst = static_cast<uint16_t*>(jobs.out[job[t]]);
      if (whole[t] && keep[t]) {
        // back through the image: the lane's pieces of sub-row l16, then the stretch as it
        // lies in memory (keep is true for every lane of a whole group)
        uint32_t* img = &image_lds[wave][t * 16 * kPitch];
#pragma unroll
        for (int p = 0; p < NP; ++p)
          *reinterpret_cast<u32x4_t*>(&img[l16 * kPitch + 16 * p + 4 * lq]) = __builtin_bit_cast(u32x4_t, o[p]);
        const int64_t at = (row[t] - l16) * B + lane * 8;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const int j = ks * kWave + lane;
          const u32x4_t piece = *reinterpret_cast<const u32x4_t*>(&img[(j >> 4) * kPitch + (j & 15) * 4]);
          CTMI_SR_STORE<uint16_t, 8>(dst + at + 512 * ks, __builtin_bit_cast(Vec<uint16_t, 8>, piece));
        }
      } else if (!whole[t] && keep[t]) {
#pragma unroll
        for (int p = 0; p < NP; ++p)
          CTMI_SR_STORE<uint16_t, 8>(dst + row[t] * B + 32 * p + 8 * lq, __builtin_bit_cast(Vec<uint16_t, 8>, o[p]));
      }
      continue;
    }
    // max |x| of the sub-row: the 4 lanes l16 + 16 q agree through two lane exchanges
    // (magnitudes of non-negative floats order like their bit patterns, a NaN above everything)
#if !CTMI_SQP_FP32_MAX
    // (bf16 magnitudes order like their bit patterns, a NaN above everything: the maximum is
    // taken on the packed 16-bit halves, two elements per instruction)
    uint32_t mag = (uint32_t)(top2.x > top2.y ? top2.x : top2.y) << 16;
#else
    uint32_t mag = __float_as_uint(top);
    if (odd || !(top < __builtin_inff())) {
      // the rare group with a NaN or an infinity: the maximum over the rounded values, bit by bit
      mag = 0;
#pragma unroll
      for (int p = 0; p < NP; ++p)
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const uint32_t lo = (o[p].v[w] & 0x7FFFu) << 16, hi = o[p].v[w] & 0x7FFF0000u;
          mag = max(mag, max(lo, hi));
        }
    } else {
      mag = (uint32_t)f32_to_bf16(__uint_as_float(mag)) << 16;  // rounded as the outputs are
    }
#endif
#pragma unroll
    for (int d = 16; d < 64; d <<= 1) {
      const uint32_t other = (uint32_t)__shfl_xor((int)mag, d, kWave);
      mag = other > mag ? other : mag;
    }
    mag >>= 16;
    const float sv = symmetric_scale<BF16>(bf16_to_f32((uint16_t)mag), mag > 0x7F80u, cfg.sym_div);
    const int j = job[t];
    int32_t* packed = static_cast<int32_t*>(jobs.out[j]);
    uint16_t* scale = static_cast<uint16_t*>(jobs.scale[j]);
    uint16_t* rotated = static_cast<uint16_t*>(jobs.rotated[j]);
    uint32_t w[NP];
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      w[p] = (uint32_t)quant_pack8<BF16, BF16, 4, false>(__builtin_bit_cast(Vec<uint16_t, 8>, o[p]), sv, 0.0f,
                                                         cfg.bit_min, cfg.bit_max).v[0];
      if (rotated && keep[t]) {
        Vec<uint32_t, 4> r = o[p];
        if constexpr (SIGN_OUT) {
#pragma unroll
          for (int d = 0; d < 4; ++d) r.v[d] = unsigned_zeros(r.v[d]);
        }
        CTMI_SQP_STORE<uint16_t, 8>(rotated + row[t] * B + 32 * p + 8 * lq, __builtin_bit_cast(Vec<uint16_t, 8>, r));
      }
    }
    // Lane (l16, lq) holds packed words 4 p + lq of its sub-row; the 4 lanes of a sub-row
    // transpose their 4 x 4 words in two exchanges (lanes 32 apart, then neighbouring rows
    // of 16 lanes), after which lane lq stores words 4 lq .. 4 lq + 3: 16 bytes.
    {
      auto s02 = __builtin_amdgcn_permlane32_swap(w[0], w[2], false, false);
      auto s13 = __builtin_amdgcn_permlane32_swap(w[1], w[3], false, false);
      auto s01 = __builtin_amdgcn_permlane16_swap(s02[0], s13[0], false, false);
      auto s23 = __builtin_amdgcn_permlane16_swap(s02[1], s13[1], false, false);
      w[0] = s01[0];
      w[1] = s01[1];
      w[2] = s23[0];
      w[3] = s23[1];
    }
    if (keep[t]) {
      if (lq == 0) scale[row[t]] = f32_to_bf16(sv);
      Vec<int32_t, 4> out4;
#pragma unroll
      for (int q = 0; q < 4; ++q) out4.v[q] = (int32_t)w[q];
      CTMI_SQP_STORE<int32_t, 4>(packed + row[t] * (B / 8) + 4 * lq, out4);
    }
  }
}

// jobs: t.end counts groups of 16 sub-rows (a tensor's last one may be ragged)
static void sylvester128_launch(const HadJobs& t, int filled, const float* sign_in, const float* sign_out,
                                const QpCfg& c, hipStream_t st) {
  const int64_t n_groups = t.end[filled - 1];
  const float inv = 1.0f / sqrtf(128.0f);
  const unsigned grid = (unsigned)cdiv(n_groups, kSqpWaves * CTMI_SQP_GROUPS);
#define CTMI_SQP(MANY)                                                                                  \
  if (sign_in && sign_out)                                                                              \
    hipLaunchKernelGGL((sylvester128_quant_pack_kernel<MANY, true, true>), grid, kSqpThreads, 0, st, t,     \
                       n_groups, sign_in, sign_out, inv, c);                                            \
  else if (sign_in)                                                                                     \
    hipLaunchKernelGGL((sylvester128_quant_pack_kernel<MANY, true, false>), grid, kSqpThreads, 0, st, t,    \
                       n_groups, sign_in, sign_out, inv, c);                                            \
  else if (sign_out)                                                                                    \
    hipLaunchKernelGGL((sylvester128_quant_pack_kernel<MANY, false, true>), grid, kSqpThreads, 0, st, t,    \
                       n_groups, sign_in, sign_out, inv, c);                                            \
  else                                                                                                  \
    hipLaunchKernelGGL((sylvester128_quant_pack_kernel<MANY, false, false>), grid, kSqpThreads, 0, st, t,   \
                       n_groups, sign_in, sign_out, inv, c)
  if (filled == 1) { CTMI_SQP(false); } else { CTMI_SQP(true); }
#undef CTMI_SQP
}

// the rotation alone; jobs: t.end counts groups of 16 sub-rows (a tensor's last one may be ragged)
static void sylvester128_rows_launch(const HadJobs& t, int filled, const float* sign_in,
                                     const float* sign_out, hipStream_t st) {
  const int64_t n_groups = t.end[filled - 1];
  const float inv = 1.0f / sqrtf(128.0f);
  const unsigned grid = (unsigned)cdiv(n_groups, kSqpWaves * CTMI_SR_GROUPS);
  const QpCfg c{};
#define CTMI_SR(MANY)                                                                                   \
  if (sign_in && sign_out)                                                                              \
    hipLaunchKernelGGL((sylvester128_quant_pack_kernel<MANY, true, true, false>), grid, kSqpThreads, 0, \
                       st, t, n_groups, sign_in, sign_out, inv, c);                                     \
  else if (sign_in)                                                                                     \
    hipLaunchKernelGGL((sylvester128_quant_pack_kernel<MANY, true, false, false>), grid, kSqpThreads,   \
                       0, st, t, n_groups, sign_in, sign_out, inv, c);                                  \
  else if (sign_out)                                                                                    \
    hipLaunchKernelGGL((sylvester128_quant_pack_kernel<MANY, false, true, false>), grid, kSqpThreads,   \
                       0, st, t, n_groups, sign_in, sign_out, inv, c);                                  \
  else                                                                                                  \
    hipLaunchKernelGGL((sylvester128_quant_pack_kernel<MANY, false, false, false>), grid, kSqpThreads,  \
                       0, st, t, n_groups, sign_in, sign_out, inv, c)
  if (filled == 1) { CTMI_SR(false); } else { CTMI_SR(true); }
#undef CTMI_SR
}

// ---------------------------------------------------------------- Kronecker sizes, bf16, no LDS staging
// n = A * B (1024 = 32 x 32, 2048 = 32 x 64, 4096 = 64 x 64): one wavefront per
// data row, the row viewed as X [A sub-rows][B].  Both stages run on
// v_mfma_f32_16x16x32_bf16 with operands that never leave the registers:
//
//   stage 1   T = X * Mb.  A operand = X: lane (i + 16 q) holds 8 neighbouring
//             elements of a sub-row (one 16-byte global load); B operand = Mb,
//             kept in registers.  The result tile has lane (j + 16 iq) holding 4
//             sub-rows of column j.  Sub-rows are handed to the row labels of
//             two tiles so that these come out as 8 neighbouring sub-rows
//             32 P + 8 iq + {0..7}: exactly the 8 k-values a lane supplies to
//             the next product.
//   stage 2   Y^T = T^T * Ma, i.e. D[c][a'] = sum_a T[a][c] Ma[a][a'].  A operand
//             = the T values just computed (fp32 split into three bf16 terms, so
//             the contraction is fp32-accurate), B operand = Ma, in registers.
//             Lane (a' + 16 cq) ends up with 4 columns of output sub-row a';
//             columns are handed to the column labels of stage 1 so that two
//             tiles give 8 neighbouring columns: one 16-byte global store.
//
// Signs (entries +1 / -1) are XOR masks on the bf16 sign bits of X and of the
// output; they are per position within the row, the same for every row, and sit
// in LDS in the lanes' own layout.
//
// B = 64: a sub-row is one 128-byte line.  Its two halves (column pairs p = 0, 1) come out
// of stage 2 one after the other; the first is held back so that both stores leave
// together and meet in the cache as a whole line.
//
// QUANT (B = 64, bfloat16): the W4A16 pipeline for group size 128 in the epilogue, as in
// hadamard_quant_pack_kernel.  A group is two neighbouring output sub-rows, i.e. the 8
// lanes (l16 ^ 1, every lq) with both halves: they agree on max |x| through three lane
// exchanges, then each lane quantizes and packs its 2 x 8 values into two words.  jobs.out
// is then the packed tensor, jobs.scale the group scales, jobs.rotated (optional) the
// rotated tensor.
//
// A > 64 (224 x 64 = 14336, 224 x 32 = 7168: the reference's Hadamard matrices of size
// K * 2^m with its known 224 x 224 block as Ma): a row is 112 registers a lane, so one wave
// per SIMD, and Ma (100 KB in bf16) does not fit in registers: its fragments sit in LDS, in
// the lanes' own layout, and are read at each use (one read serves the three products of
// the split intermediate).
template <int A, int B>
struct KronLds {
  static constexpr bool kBig = A > 64;
#ifndef CTMI_HAD_KRON_MA_LDS_FROM
#define CTMI_HAD_KRON_MA_LDS_FROM 65  // smallest A whose Ma is read from LDS instead of registers
#endif
  static constexpr bool kMaLds = A >= CTMI_HAD_KRON_MA_LDS_FROM;
  static constexpr int KS = B / 32, MT = A / 16, NT = B / 16, PS = A / 32, AT = A / 16;
  static constexpr size_t sign_in = (size_t)MT * KS * kWave * 16;
  static constexpr size_t sign_out = (size_t)AT * (NT / 2) * kWave * 16;
  static constexpr size_t ma = kMaLds ? (size_t)AT * PS * kWave * 16 : 0;
  static constexpr size_t bytes = sign_in + sign_out + ma;
};

template <int A, int B, bool HALF, bool MANY, bool QUANT = false>
__global__ void __launch_bounds__(kKronThreads)
__attribute__((amdgpu_waves_per_eu(A > 64 ? 1 : CTMI_HAD_KRON_WAVES)))
hadamard_kron_kernel(HadJobs jobs, int64_t n_rows, const uint16_t* __restrict__ mbt,
                     const uint16_t* __restrict__ mat, const float* __restrict__ s_in,
                     const float* __restrict__ s_out, float inv_sqrt_n, QpCfg cfg) {
  static_assert(!QUANT || (B == 64 && !HALF), "the fused epilogue is written for 64-wide bf16 sub-rows");
  static_assert(A % 32 == 0 && B % 32 == 0, "whole k steps");
  constexpr bool BIG = KronLds<A, B>::kBig;
  constexpr bool MA_LDS = KronLds<A, B>::kMaLds;
  static_assert(!(BIG && QUANT), "the fused epilogue holds half rows back: not with A > 64");
  constexpr int N = A * B;
  constexpr int KS = B / 32;   // k steps of stage 1
  constexpr int MT = A / 16;   // sub-row tiles
  constexpr int NT = B / 16;   // column tiles
  constexpr int PS = A / 32;   // k steps of stage 2 (pairs of sub-row tiles)
  constexpr int AT = A / 16;   // output sub-row tiles
  constexpr int NSPLIT = 3;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int l16 = lane & 15, lq = lane >> 4;
  const int perm = 8 * (l16 / 4) + (l16 % 4);  // label -> position within a pair of tiles
  // HALF: float16 tensors.  Stage 1 runs on v_mfma_f32_16x16x32_f16 (Mb converts from
  // bfloat16 to float16 exactly); stage 2 works on the fp32 intermediate as before.
  using xfrag_t = typename std::conditional<HALF, f16x8_t, bf16x8_t>::type;

  extern __shared__ __align__(16) unsigned char kron_lds[];
  typedef u32x4_t lane_row_t[kWave];
  lane_row_t* sign_in_lds = reinterpret_cast<lane_row_t*>(kron_lds);
  lane_row_t* sign_out_lds = reinterpret_cast<lane_row_t*>(kron_lds + KronLds<A, B>::sign_in);
  lane_row_t* ma_lds = reinterpret_cast<lane_row_t*>(kron_lds + KronLds<A, B>::sign_in +
                                                     KronLds<A, B>::sign_out);
  const bool signed_io = s_in || s_out;
  if (signed_io) {
    const uint32_t* pin = reinterpret_cast<const uint32_t*>(s_in ? (const void*)s_in : (const void*)mbt);
    const uint32_t* pout = reinterpret_cast<const uint32_t*>(s_out ? (const void*)s_out : (const void*)mbt);
    const uint32_t use_in = s_in ? 1u : 0u, use_out = s_out ? 1u : 0u;
    for (int f = wave; f < MT * KS; f += kKronWaves) {
      const int m = f / KS, ks = f % KS;
      const int pos = (32 * (m / 2) + 4 * (m % 2) + perm) * B + 32 * ks + 8 * lq;
      u32x4_t w;
#pragma unroll
      for (int d = 0; d < 4; ++d)
        w[d] = (((pin[pos + 2 * d] >> 31) & use_in) << 15) | (((pin[pos + 2 * d + 1] >> 31) & use_in) << 31);
      sign_in_lds[f][lane] = w;
    }
    for (int f = wave; f < AT * (NT / 2); f += kKronWaves) {
      const int at = f / (NT / 2), p = f % (NT / 2);
      const int pos = (16 * at + l16) * B + 32 * p + 8 * lq;
      u32x4_t w;
#pragma unroll
      for (int d = 0; d < 4; ++d)
        w[d] = (((pout[pos + 2 * d] >> 31) & use_out) << 15) | (((pout[pos + 2 * d + 1] >> 31) & use_out) << 31);
      sign_out_lds[f][lane] = w;
    }
  }
  if constexpr (MA_LDS) {
    for (int f = wave; f < AT * PS; f += kKronWaves) {
      const int at = f / PS, ps = f % PS;
      ma_lds[f][lane] = *reinterpret_cast<const u32x4_t*>(mat + (16 * at + l16) * A + 32 * ps + 8 * lq);
    }
  }
  if (signed_io || MA_LDS) __syncthreads();

  // the two small matrices, as B operands
  xfrag_t mbf[NT][KS];
  bf16x8_t maf[MA_LDS ? 1 : AT][MA_LDS ? 1 : PS];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      Vec<uint32_t, 4> m = __builtin_bit_cast(
          Vec<uint32_t, 4>,
          ldg<uint16_t, 8>(mbt + (32 * (nt / 2) + 4 * (nt % 2) + perm) * B + 32 * ks + 8 * lq));
      if constexpr (HALF) {
#pragma unroll
        for (int w = 0; w < 4; ++w)
          m.v[w] = (uint32_t)f32_to_f16(bf16_lo(m.v[w])) | ((uint32_t)f32_to_f16(bf16_hi(m.v[w])) << 16);
      }
      mbf[nt][ks] = __builtin_bit_cast(xfrag_t, m);
    }
  if constexpr (!MA_LDS) {
#pragma unroll
    for (int at = 0; at < AT; ++at)
#pragma unroll
      for (int ps = 0; ps < PS; ++ps)
        maf[at][ps] = __builtin_bit_cast(
            bf16x8_t, ldg<uint16_t, 8>(mat + (16 * at + l16) * A + 32 * ps + 8 * lq));
  }

  const int64_t stride = (int64_t)gridDim.x * kKronWaves;
  for (int64_t row = (int64_t)blockIdx.x * kKronWaves + wave; row < n_rows; row += stride) {
    int64_t local;
    const int j = had_job<MANY>(jobs, row, &local);  // n_rows: data rows over all jobs
    const uint16_t* src = static_cast<const uint16_t*>(jobs.x[j]) + local * N;
    uint16_t* dst = QUANT ? static_cast<uint16_t*>(jobs.rotated[j])
                          : static_cast<uint16_t*>(jobs.out[j]);
    if (!QUANT || dst) dst += local * N;
    int32_t* packed = nullptr;
    uint16_t* scale = nullptr;
    if constexpr (QUANT) {
      packed = static_cast<int32_t*>(jobs.out[j]) + local * (N / 8);
      scale = static_cast<uint16_t*>(jobs.scale[j]) + local * (N / 128);
    }
    u32x4_t held[B == 64 && !BIG ? AT : 1];  // first halves of the output sub-rows
    xfrag_t xf[MT][KS];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        xf[m][ks] = __builtin_bit_cast(
            xfrag_t,
            ldg<uint16_t, 8>(src + (32 * (m / 2) + 4 * (m % 2) + perm) * B + 32 * ks + 8 * lq));
    if (signed_io) {
#pragma unroll
      for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const u32x4_t f = sign_in_lds[m * KS + ks][lane];
          xf[m][ks] = __builtin_bit_cast(xfrag_t, __builtin_bit_cast(u32x4_t, xf[m][ks]) ^ f);
        }
    }
#pragma unroll
    for (int p = 0; p < NT / 2; ++p) {
      // ---- stage 1 for column tiles 2p and 2p+1, split for stage 2
      bf16x8_t tf[2][PS][NSPLIT];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int nt = 2 * p + h;
#pragma unroll
        for (int ps = 0; ps < PS; ++ps) {
          f32x4_t lo = {0.0f, 0.0f, 0.0f, 0.0f}, hi = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            if constexpr (HALF) {
              lo = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf[2 * ps][ks], mbf[nt][ks], lo, 0, 0, 0);
              hi = __builtin_amdgcn_mfma_f32_16x16x32_f16(xf[2 * ps + 1][ks], mbf[nt][ks], hi, 0, 0, 0);
            } else {
              lo = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xf[2 * ps][ks], mbf[nt][ks], lo, 0, 0, 0);
              hi = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xf[2 * ps + 1][ks], mbf[nt][ks], hi, 0, 0, 0);
            }
          }
          float t[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
          u32x4_t parts[NSPLIT];
#pragma unroll
          for (int sp = 0; sp < NSPLIT; ++sp) {
#pragma unroll
            for (int d = 0; d < 4; ++d) {
              const uint32_t w = pack_bf16x2(t[2 * d], t[2 * d + 1]);
              parts[sp][d] = w;
              t[2 * d] -= bf16_lo(w);
              t[2 * d + 1] -= bf16_hi(w);
            }
            tf[h][ps][sp] = __builtin_bit_cast(bf16x8_t, parts[sp]);
          }
        }
      }
      // ---- stage 2: every output sub-row tile for these 32 columns
#pragma unroll
      for (int at = 0; at < AT; ++at) {
        f32x4_t y0 = {0.0f, 0.0f, 0.0f, 0.0f}, y1 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int ps = 0; ps < PS; ++ps) {
          bf16x8_t mf;
          if constexpr (MA_LDS) {
            // keeps the compiler from hoisting these (loop-invariant) LDS reads out of the
            // row loop, back into hundreds of registers
            asm volatile("" ::: "memory");
            mf = __builtin_bit_cast(bf16x8_t, ma_lds[at * PS + ps][lane]);
          } else {
            mf = maf[at][ps];
          }
#pragma unroll
          for (int sp = NSPLIT - 1; sp >= 0; --sp) {  // small terms first
            y0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(tf[0][ps][sp], mf, y0, 0, 0, 0);
            y1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(tf[1][ps][sp], mf, y1, 0, 0, 0);
          }
        }
        u32x4_t o;
        if constexpr (HALF) {
#pragma unroll
          for (int d = 0; d < 2; ++d) {
            o[d] = (uint32_t)f32_to_f16(y0[2 * d] * inv_sqrt_n) |
                   ((uint32_t)f32_to_f16(y0[2 * d + 1] * inv_sqrt_n) << 16);
            o[2 + d] = (uint32_t)f32_to_f16(y1[2 * d] * inv_sqrt_n) |
                       ((uint32_t)f32_to_f16(y1[2 * d + 1] * inv_sqrt_n) << 16);
          }
        } else {
          o[0] = pack_bf16x2(y0[0] * inv_sqrt_n, y0[1] * inv_sqrt_n);
          o[1] = pack_bf16x2(y0[2] * inv_sqrt_n, y0[3] * inv_sqrt_n);
          o[2] = pack_bf16x2(y1[0] * inv_sqrt_n, y1[1] * inv_sqrt_n);
          o[3] = pack_bf16x2(y1[2] * inv_sqrt_n, y1[3] * inv_sqrt_n);
        }
        if (signed_io) o ^= sign_out_lds[at * (NT / 2) + p][lane];
        uint16_t* at_dst = dst + (16 * at + l16) * B + 8 * lq;
        if constexpr (B != 64 || BIG) {
          stg<uint16_t, 8>(at_dst + 32 * p, __builtin_bit_cast(Vec<uint16_t, 8>, o));
        } else if (p == 0) {
          held[at] = o;
        } else if constexpr (!QUANT) {
          stg<uint16_t, 8>(at_dst, __builtin_bit_cast(Vec<uint16_t, 8>, held[at]));
          stg<uint16_t, 8>(at_dst + 32, __builtin_bit_cast(Vec<uint16_t, 8>, o));
        } else {
          // max |x| of the group on the packed 16-bit halves (bf16 magnitudes order like
          // their bit patterns, a NaN above everything), then over the group's 8 lanes
          typedef uint16_t u16x2_t __attribute__((ext_vector_type(2)));
          u16x2_t top = {0, 0};
#pragma unroll
          for (int w = 0; w < 4; ++w) {
            top = __builtin_elementwise_max(top, __builtin_bit_cast(u16x2_t, held[at][w] & 0x7FFF7FFFu));
            top = __builtin_elementwise_max(top, __builtin_bit_cast(u16x2_t, o[w] & 0x7FFF7FFFu));
          }
          uint32_t mag = top.x > top.y ? top.x : top.y;
#pragma unroll
          for (int d = 1; d < 64; d = d == 1 ? 16 : d << 1) {
            const uint32_t other = (uint32_t)__shfl_xor((int)mag, d, kWave);
            mag = other > mag ? other : mag;
          }
          // calculate_qparams, symmetric, in bf16 (helpers.py:101-122)
          float sv = bf16_to_f32(f32_to_bf16(bf16_to_f32((uint16_t)mag) / cfg.sym_div));
          sv = (sv != sv) ? sv : fmaxf(sv, 1.1920928955078125e-07f);
          const Vec<int32_t, 1> w0 = quant_pack8<BF16, BF16, 4, false>(
              __builtin_bit_cast(Vec<uint16_t, 8>, held[at]), sv, 0.0f, cfg.bit_min, cfg.bit_max);
          const Vec<int32_t, 1> w1 = quant_pack8<BF16, BF16, 4, false>(
              __builtin_bit_cast(Vec<uint16_t, 8>, o), sv, 0.0f, cfg.bit_min, cfg.bit_max);
          const int sub = 16 * at + l16;
          packed[sub * (B / 8) + lq] = w0.v[0];
          packed[sub * (B / 8) + 4 + lq] = w1.v[0];
          if (lq == 0 && (l16 & 1) == 0) scale[sub / 2] = f32_to_bf16(sv);
          if (dst) {
            stg<uint16_t, 8>(at_dst, __builtin_bit_cast(Vec<uint16_t, 8>, held[at]));
            stg<uint16_t, 8>(at_dst + 32, __builtin_bit_cast(Vec<uint16_t, 8>, o));
          }
        }
      }
    }
  }
}

// jobs: units are data rows of A * B elements
template <int A, int B, bool HALF>
static int launch_had_kron_jobs(const HadJobs& jobs, int n_jobs, const HadArgs& a, hipStream_t st) {
  const int64_t n_rows = jobs.end[n_jobs - 1];
  const int64_t wgs = cdiv(n_rows, kKronWaves);
  // as many workgroups as are resident at once (register-limited; one wave per SIMD for A > 64)
  const int waves = A > 64 ? 1 : (A * B <= 1024 ? 8 : (A * B <= 2048 ? 4 : CTMI_HAD_KRON_WAVES));
  const int64_t cap = 256 * 4 * waves / kKronWaves;
  const unsigned grid = (unsigned)(wgs < cap ? wgs : cap);
  const QpCfg none{};
  constexpr size_t lds = KronLds<A, B>::bytes;
  auto one = hadamard_kron_kernel<A, B, HALF, false>;
  auto many = hadamard_kron_kernel<A, B, HALF, true>;
  auto kern = n_jobs == 1 ? one : many;
  if (lds > 48 * 1024) {
    // the attribute belongs to the kernel as loaded on one device; setting it again is cheap
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess)
      return set_error(CTMI_ERR_HIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  }
  hipLaunchKernelGGL(kern, grid, kKronThreads, lds, st, jobs, n_rows, a.mbt, a.mat, a.s_in, a.s_out,
                     1.0f / a.sqrt_n, none);
  return CTMI_OK;
}

// the same with the quantization epilogue (bf16, B = 64, group size 128)
template <int A>
static int launch_had_kron_quant_jobs(const HadJobs& jobs, int n_jobs, const HadArgs& a,
                                      const QpCfg& cfg, hipStream_t st) {
  const int64_t n_rows = jobs.end[n_jobs - 1];
  const int64_t wgs = cdiv(n_rows, kKronWaves);
  const int64_t cap = 256 * 4 * (A * 64 <= 2048 ? 4 : CTMI_HAD_KRON_WAVES) / kKronWaves;
  const unsigned grid = (unsigned)(wgs < cap ? wgs : cap);
  constexpr size_t lds = KronLds<A, 64>::bytes;
  if (n_jobs == 1)
    hipLaunchKernelGGL((hadamard_kron_kernel<A, 64, false, false, true>), grid, kKronThreads, lds, st,
                       jobs, n_rows, a.mbt, a.mat, a.s_in, a.s_out, 1.0f / a.sqrt_n, cfg);
  else
    hipLaunchKernelGGL((hadamard_kron_kernel<A, 64, false, true, true>), grid, kKronThreads, lds, st,
                       jobs, n_rows, a.mbt, a.mat, a.s_in, a.s_out, 1.0f / a.sqrt_n, cfg);
  return CTMI_OK;
}

template <int A, int B, typename IO>
static int launch_had(const HadArgs& a, hipStream_t st) {
  using C = HadCfg<A, B, IO>;
  // the attribute belongs to the kernel as loaded on one device: once per device
  constexpr int kMaxDevices = 64;
  static std::atomic<bool> configured[kMaxDevices];
  auto kern = hadamard_mfma_kernel<A, B, IO>;
  if (C::lds_bytes > 48 * 1024) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) dev = -1;
    const bool tracked = dev >= 0 && dev < kMaxDevices;
    if (!tracked || !configured[dev].load(std::memory_order_acquire)) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                         hipFuncAttributeMaxDynamicSharedMemorySize,
                                         (int)C::lds_bytes);
      if (e != hipSuccess)
        return set_error(CTMI_ERR_HIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
      if (tracked) configured[dev].store(true, std::memory_order_release);
    }
  }
  const int64_t tiles = cdiv(a.n_sub, C::S);
  const int64_t cap = 256 * 8;
  const unsigned grid = (unsigned)(tiles < cap ? tiles : cap);
  hipLaunchKernelGGL(kern, grid, kHadThreads, C::lds_bytes, st, a);
  return CTMI_OK;
}

template <typename IO>
static int dispatch_had(int a_dim, int b_dim, const HadArgs& a, hipStream_t st) {
#define CTMI_HAD(AA, BB) \
  if (a_dim == AA && b_dim == BB) return launch_had<AA, BB, IO>(a, st);
  CTMI_HAD(1, 32) CTMI_HAD(1, 64) CTMI_HAD(1, 128)
  CTMI_HAD(32, 32) CTMI_HAD(32, 64) CTMI_HAD(64, 64) CTMI_HAD(64, 128)
#undef CTMI_HAD
  return set_error(CTMI_ERR_UNSUPPORTED, "no MFMA kernel for the factorisation %d x %d", a_dim,
                   b_dim);
}

// the kernels that keep their operands in registers (and take several tensors per launch)
static bool had_in_registers(int io_dtype, int a_dim, int b_dim) {
  if (io_dtype != CTMI_BF16 && io_dtype != CTMI_F16) return false;
  if (a_dim == 1) return b_dim == 32 || b_dim == 64 || b_dim == 128;
  return (a_dim == 32 && (b_dim == 32 || b_dim == 64)) || (a_dim == 64 && b_dim == 64) ||
         (a_dim == 224 && (b_dim == 32 || b_dim == 64));
}

static int launch_had_jobs(const HadJobs& jobs, int n_jobs, int io_dtype, int a_dim, int b_dim,
                           const HadArgs& a, hipStream_t st) {
  const bool half = io_dtype == CTMI_F16;
#define CTMI_ROWS(BB) (half ? launch_had_rows_jobs<BB, true>(jobs, n_jobs, a, st) \
                            : launch_had_rows_jobs<BB, false>(jobs, n_jobs, a, st))
#define CTMI_KRON(AA, BB) (half ? launch_had_kron_jobs<AA, BB, true>(jobs, n_jobs, a, st) \
                                : launch_had_kron_jobs<AA, BB, false>(jobs, n_jobs, a, st))
  if (a_dim == 1) return b_dim == 32 ? CTMI_ROWS(32) : (b_dim == 64 ? CTMI_ROWS(64) : CTMI_ROWS(128));
  if (a_dim == 32) return b_dim == 32 ? CTMI_KRON(32, 32) : CTMI_KRON(32, 64);
  if (a_dim == 224) return b_dim == 32 ? CTMI_KRON(224, 32) : CTMI_KRON(224, 64);
  return CTMI_KRON(64, 64);
#undef CTMI_ROWS
#undef CTMI_KRON
}

}  // namespace ctmi

using namespace ctmi;

extern "C" int ctmi_hadamard_supported(int32_t a_dim, int32_t b_dim, int32_t io_dtype) {
  // 224 x 32 and 224 x 64 (7168 and 14336, Ma any +-1 matrix of order 224): 16-bit tensors
  if (a_dim == 224 && (b_dim == 32 || b_dim == 64)) return io_dtype == CTMI_BF16 || io_dtype == CTMI_F16;
  const bool pair = (a_dim == 1 && (b_dim == 32 || b_dim == 64 || b_dim == 128)) ||
                    (a_dim == 32 && (b_dim == 32 || b_dim == 64)) ||
                    (a_dim == 64 && (b_dim == 64 || b_dim == 128));
  if (!pair) return 0;
  if (io_dtype == CTMI_BF16) return 1;
  // wider inputs need 2-3 staged copies: the largest factorisation does not fit in LDS
  if (io_dtype == CTMI_F16 || io_dtype == CTMI_F32) return !(a_dim == 64 && b_dim == 128);
  return 0;
}

// does the rotation by Sylvester's matrix of 128 run without a matrix argument?
static bool sylvester128_rows_ok(int32_t a_dim, int32_t b_dim, int32_t io_dtype) {
  return a_dim == 1 && b_dim == 128 && io_dtype == CTMI_BF16;
}

extern "C" int ctmi_hadamard_sylvester_inner_supported(int32_t a_dim, int32_t b_dim, int32_t io_dtype) {
  return a_dim > 1 && block_sylvester64_supported(a_dim, b_dim, io_dtype, false);
}

extern "C" int ctmi_hadamard_apply(const void* x, void* out, int32_t io_dtype, int64_t numel,
                                   int32_t a_dim, int32_t b_dim, const void* ma_t,
                                   const void* mb_t, const float* sign_in, const float* sign_out,
                                   void* stream) {
  CTMI_REQUIRE(numel >= 0, CTMI_ERR_VALUE, "negative size");
  CTMI_REQUIRE(a_dim >= 1 && b_dim >= 1, CTMI_ERR_VALUE, "bad factor sizes");
  CTMI_REQUIRE(io_dtype == CTMI_BF16 || io_dtype == CTMI_F16 || io_dtype == CTMI_F32,
               CTMI_ERR_UNSUPPORTED, "transforms take float16/bfloat16/float32 tensors");
  const int64_t n = (int64_t)a_dim * b_dim;
  CTMI_REQUIRE(numel % n == 0, CTMI_ERR_VALUE,
               "tensor size %lld is not a multiple of the transform size %lld", (long long)numel,
               (long long)n);
  if (!mb_t && (a_dim > 1 || sylvester128_rows_ok(a_dim, b_dim, io_dtype))) {
    // Mb = Sylvester's matrix: the product with Ma on the matrix cores, butterflies for Mb
    // (or, for a block of 128, the kernel that keeps no matrix in memory)
    ctmi_hadamard_job job;
    job.x = x;
    job.out = out;
    job.numel = numel;
    return ctmi_hadamard_apply_many(&job, 1, io_dtype, a_dim, b_dim, ma_t, mb_t, sign_in, sign_out, stream);
  }
  CTMI_REQUIRE(ctmi_hadamard_supported(a_dim, b_dim, io_dtype), CTMI_ERR_UNSUPPORTED,
               "no MFMA kernel for the factorisation %d x %d with this dtype", a_dim, b_dim);
  if (numel == 0) return CTMI_OK;
  CTMI_REQUIRE(x && out && mb_t && (a_dim == 1 || ma_t), CTMI_ERR_VALUE, "NULL tensor pointer");
  CTMI_REQUIRE((uintptr_t)x % 16 == 0 && (uintptr_t)out % 16 == 0 && (uintptr_t)mb_t % 16 == 0 &&
                   (uintptr_t)ma_t % 16 == 0,
               CTMI_ERR_VALUE, "tensors must be 16-byte aligned");
  HadArgs a;
  a.x = x;
  a.out = out;
  a.mbt = (const uint16_t*)mb_t;
  a.mat = (const uint16_t*)ma_t;
  a.s_in = sign_in;
  a.s_out = sign_out;
  a.n_sub = numel / b_dim;
  a.sqrt_n = sqrtf((float)n);
  hipStream_t st = (hipStream_t)stream;
  int rc;
  if (had_in_registers(io_dtype, a_dim, b_dim)) {
    HadJobs jobs;
    clear_jobs(&jobs);
    jobs.x[0] = x;
    jobs.out[0] = out;
    jobs.n_sub[0] = a.n_sub;
    jobs.end[0] = a_dim == 1 ? a.n_sub / 16 : a.n_sub / a_dim;
    rc = launch_had_jobs(jobs, 1, io_dtype, a_dim, b_dim, a, st);
  } else if (io_dtype == CTMI_BF16) rc = dispatch_had<BF16>(a_dim, b_dim, a, st);
  else if (io_dtype == CTMI_F16) rc = dispatch_had<F16>(a_dim, b_dim, a, st);
  else rc = dispatch_had<F32>(a_dim, b_dim, a, st);
  if (rc) return rc;
  return check_launch("ctmi_hadamard_apply");
}

extern "C" int ctmi_hadamard_apply_many(const ctmi_hadamard_job* jobs, int64_t n_jobs,
                                        int32_t io_dtype, int32_t a_dim, int32_t b_dim,
                                        const void* ma_t, const void* mb_t, const float* sign_in,
                                        const float* sign_out, void* stream) {
  CTMI_REQUIRE(n_jobs >= 0 && (jobs || n_jobs == 0), CTMI_ERR_VALUE, "bad job list");
  if (n_jobs == 0) return CTMI_OK;
  CTMI_REQUIRE(a_dim >= 1 && b_dim >= 1, CTMI_ERR_VALUE, "bad factor sizes");
  CTMI_REQUIRE(io_dtype == CTMI_BF16 || io_dtype == CTMI_F16 || io_dtype == CTMI_F32,
               CTMI_ERR_UNSUPPORTED, "transforms take float16/bfloat16/float32 tensors");
  if (!mb_t && sylvester128_rows_ok(a_dim, b_dim, io_dtype)) {
    // Sylvester's matrix of 128 on bfloat16 tensors: no matrix in memory, any number of sub-rows
    for (int64_t i = 0; i < n_jobs; ++i) {
      const ctmi_hadamard_job& j = jobs[i];
      CTMI_REQUIRE(j.numel >= 0 && j.numel % b_dim == 0, CTMI_ERR_VALUE,
                   "job %lld: tensor size %lld is not a multiple of the transform size %d", (long long)i,
                   (long long)j.numel, b_dim);
      CTMI_REQUIRE(j.numel == 0 || (j.x && j.out), CTMI_ERR_VALUE, "job %lld: NULL tensor pointer", (long long)i);
      CTMI_REQUIRE((uintptr_t)j.x % 16 == 0 && (uintptr_t)j.out % 16 == 0, CTMI_ERR_VALUE,
                   "tensors must be 16-byte aligned");
    }
    CTMI_REQUIRE((uintptr_t)sign_in % 16 == 0 && (uintptr_t)sign_out % 16 == 0, CTMI_ERR_VALUE,
                 "sign vectors must be 16-byte aligned");
    HadJobs t;
    clear_jobs(&t);
    int filled = 0;
    bool any = false;
    for (int64_t i = 0; i <= n_jobs; ++i) {
      if (i < n_jobs && jobs[i].numel > 0) {
        t.x[filled] = jobs[i].x;
        t.out[filled] = jobs[i].out;
        t.n_sub[filled] = jobs[i].numel / b_dim;
        t.end[filled] = (filled ? t.end[filled - 1] : 0) + cdiv(jobs[i].numel / b_dim, (int64_t)16);
        ++filled;
      }
      if (filled == kHadMaxJobs || (i == n_jobs && filled)) {
        sylvester128_rows_launch(t, filled, sign_in, sign_out, (hipStream_t)stream);
        clear_jobs(&t);
        filled = 0;
        any = true;
      }
    }
    return any ? check_launch("ctmi_hadamard_apply_many") : CTMI_OK;
  }
  const bool sylvester_inner = !mb_t && a_dim > 1;
  if (sylvester_inner)
    CTMI_REQUIRE(ctmi_hadamard_sylvester_inner_supported(a_dim, b_dim, io_dtype) && !(sign_in && sign_out),
                 CTMI_ERR_UNSUPPORTED,
                 "without mb_t (Mb = Sylvester's matrix): b_dim 4 ... 64 with a_dim up to 256 or b_dim 128 "
                 "with a_dim up to 224, bfloat16 or float16 tensors, signs on one side; got %d x %d",
                 a_dim, b_dim);
  else
    CTMI_REQUIRE(ctmi_hadamard_supported(a_dim, b_dim, io_dtype), CTMI_ERR_UNSUPPORTED,
                 "no MFMA kernel for the factorisation %d x %d with this dtype", a_dim, b_dim);
  const int64_t n = (int64_t)a_dim * b_dim;
  // validate everything before anything is enqueued
  for (int64_t i = 0; i < n_jobs; ++i) {
    const ctmi_hadamard_job& j = jobs[i];
    CTMI_REQUIRE(j.numel >= 0 && j.numel % n == 0, CTMI_ERR_VALUE,
                 "job %lld: tensor size %lld is not a multiple of the transform size %lld",
                 (long long)i, (long long)j.numel, (long long)n);
    CTMI_REQUIRE(j.numel == 0 || (j.x && j.out), CTMI_ERR_VALUE, "job %lld: NULL tensor pointer",
                 (long long)i);
    CTMI_REQUIRE((uintptr_t)j.x % 16 == 0 && (uintptr_t)j.out % 16 == 0, CTMI_ERR_VALUE,
                 "tensors must be 16-byte aligned");
    // a block above 224 rows takes two launches, and the second reads the runs again
    CTMI_REQUIRE(!(sylvester_inner && a_dim > 224) || j.numel == 0 || j.x != j.out, CTMI_ERR_VALUE,
                 "job %lld: blocks of more than 224 rows are not transformed in place", (long long)i);
  }
  CTMI_REQUIRE(n_jobs == 0 || ((mb_t || sylvester_inner) && (a_dim == 1 || ma_t)), CTMI_ERR_VALUE,
               "NULL matrix pointer");
  CTMI_REQUIRE((uintptr_t)mb_t % 16 == 0 && (uintptr_t)ma_t % 16 == 0, CTMI_ERR_VALUE,
               "tensors must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  if (sylvester_inner) {
    FwhtJob batch[kFwhtMaxJobs];
    int filled = 0;
    bool any = false;
    for (int64_t i = 0; i <= n_jobs; ++i) {
      if (i < n_jobs && jobs[i].numel > 0) {
        FwhtJob& b = batch[filled++];
        b.x = jobs[i].x;
        b.out = jobs[i].out;
        b.packed = nullptr;
        b.scale = nullptr;
        b.rows = jobs[i].numel / n;
      }
      if (filled == kFwhtMaxJobs || (i == n_jobs && filled)) {
        const int rc = block_sylvester64_launch(batch, filled, io_dtype, a_dim, b_dim, (const uint16_t*)ma_t, sign_in, sign_out,
                                                1.0f / sqrtf((float)n), st);
        if (rc) return rc;
        filled = 0;
        any = true;
      }
    }
    return any ? check_launch("ctmi_hadamard_apply_many") : CTMI_OK;
  }
  HadArgs a;
  a.x = nullptr;
  a.out = nullptr;
  a.mbt = (const uint16_t*)mb_t;
  a.mat = (const uint16_t*)ma_t;
  a.s_in = sign_in;
  a.s_out = sign_out;
  a.n_sub = 0;
  a.sqrt_n = sqrtf((float)n);
  // tensors made of whole units share launches, kHadMaxJobs at a time; the others
  // (a ragged last group, dtypes on the LDS-staged kernel) get a call of their own
  const int64_t unit = a_dim == 1 ? 16 * (int64_t)b_dim : n;
  const bool shared = had_in_registers(io_dtype, a_dim, b_dim);
  HadJobs t;
  clear_jobs(&t);
  int filled = 0;
  for (int64_t i = 0; i < n_jobs; ++i) {
    const ctmi_hadamard_job& j = jobs[i];
    if (j.numel == 0) continue;
    if (!shared || j.numel % unit != 0) {
      int rc = ctmi_hadamard_apply(j.x, j.out, io_dtype, j.numel, a_dim, b_dim, ma_t, mb_t, sign_in,
                                   sign_out, stream);
      if (rc) return rc;
      continue;
    }
    t.x[filled] = j.x;
    t.out[filled] = j.out;
    t.n_sub[filled] = j.numel / b_dim;
    t.end[filled] = (filled ? t.end[filled - 1] : 0) + j.numel / unit;
    if (++filled == kHadMaxJobs) {
      int rc = launch_had_jobs(t, filled, io_dtype, a_dim, b_dim, a, st);
      if (rc) return rc;
      clear_jobs(&t);
      filled = 0;
    }
  }
  bool any = false;
  for (int64_t i = 0; i < n_jobs; ++i) any |= jobs[i].numel != 0;
  if (!any) return CTMI_OK;
  if (filled) {
    int rc = launch_had_jobs(t, filled, io_dtype, a_dim, b_dim, a, st);
    if (rc) return rc;
  }
  return check_launch("ctmi_hadamard_apply_many");
}

static int hqp_check(int32_t io_dtype, int32_t b_dim, int32_t num_bits, int32_t symmetric) {
  CTMI_REQUIRE(io_dtype == CTMI_BF16, CTMI_ERR_UNSUPPORTED,
               "the fused rotation + quantization takes bfloat16 tensors");
  CTMI_REQUIRE(b_dim == 32 || b_dim == 64 || b_dim == 128, CTMI_ERR_UNSUPPORTED,
               "block (= group) size must be 32, 64 or 128, got %d", b_dim);
  CTMI_REQUIRE(num_bits == 4 && symmetric, CTMI_ERR_UNSUPPORTED,
               "only symmetric 4-bit integer quantization is fused");
  return CTMI_OK;
}

static int hqp_check_job(const ctmi_hadamard_pack_job& j, int32_t b_dim) {
  CTMI_REQUIRE(j.numel >= 0, CTMI_ERR_VALUE, "negative size");
  CTMI_REQUIRE(j.numel % b_dim == 0, CTMI_ERR_VALUE,
               "tensor size %lld is not a multiple of the block size %d", (long long)j.numel, b_dim);
  if (j.numel == 0) return CTMI_OK;
  CTMI_REQUIRE(j.x && j.packed && j.scale, CTMI_ERR_VALUE, "NULL tensor pointer");
  CTMI_REQUIRE((uintptr_t)j.x % 16 == 0 && (uintptr_t)j.rotated % 16 == 0 &&
                   (uintptr_t)j.packed % 16 == 0 && (uintptr_t)j.scale % 2 == 0,
               CTMI_ERR_VALUE, "tensors must be 16-byte aligned");
  return CTMI_OK;
}

static void hqp_launch(const HadJobs& t, int filled, int32_t b_dim, const void* mb_t,
                       const float* sign_in, const float* sign_out, int32_t num_bits,
                       hipStream_t st) {
  QpCfg c{};
  quant_range(CTMI_QTYPE_INT, num_bits, &c.bit_min, &c.bit_max);
  c.range = c.bit_max - c.bit_min;
  c.sym_div = (float)((double)c.range / 2.0);
  c.qtype = CTMI_QTYPE_INT;
  c.num_bits = num_bits;
  c.symmetric = 1;
  c.mt = c.zp_sub_dtype = c.scale_dtype = CTMI_BF16;
  c.zp_dtype = CTMI_I8;
  const int64_t n_groups = t.end[filled - 1];
  const float inv = 1.0f / sqrtf((float)b_dim);
  if (!mb_t) {  // Sylvester's matrix of 128 (checked by the caller)
    sylvester128_launch(t, filled, sign_in, sign_out, c, st);
    return;
  }
  const int64_t wgs = cdiv(n_groups, kHqpWaves * CTMI_HQP_GROUPS);
  const int64_t cap = 256 * CTMI_HQP_WG_PER_CU;
  const unsigned grid = (unsigned)(wgs < cap ? wgs : cap);
#define CTMI_HQP(BB)                                                                             \
  if (filled == 1)                                                                               \
    hipLaunchKernelGGL((hadamard_quant_pack_kernel<BB, false>), grid, kHqpThreads, 0, st, t,     \
                       n_groups, (const uint16_t*)mb_t, sign_in, sign_out, inv, c);              \
  else                                                                                           \
    hipLaunchKernelGGL((hadamard_quant_pack_kernel<BB, true>), grid, kHqpThreads, 0, st, t,      \
                       n_groups, (const uint16_t*)mb_t, sign_in, sign_out, inv, c)
  if (b_dim == 32) { CTMI_HQP(32); }
  else if (b_dim == 64) { CTMI_HQP(64); }
  else { CTMI_HQP(128); }
#undef CTMI_HQP
}

extern "C" int ctmi_hadamard_quant_pack_many(const ctmi_hadamard_pack_job* jobs, int64_t n_jobs,
                                             int32_t io_dtype, int32_t b_dim, const void* mb_t,
                                             const float* sign_in, const float* sign_out,
                                             int32_t num_bits, int32_t symmetric, void* stream) {
  CTMI_REQUIRE(n_jobs >= 0 && (jobs || n_jobs == 0), CTMI_ERR_VALUE, "bad job list");
  int rc = hqp_check(io_dtype, b_dim, num_bits, symmetric);
  if (rc) return rc;
  if (n_jobs == 0) return CTMI_OK;
  for (int64_t i = 0; i < n_jobs; ++i) {
    rc = hqp_check_job(jobs[i], b_dim);
    if (rc) return rc;
  }
  CTMI_REQUIRE((mb_t || b_dim == 128) && (uintptr_t)mb_t % 16 == 0, CTMI_ERR_VALUE,
               "the matrix must be given, 16-byte aligned (NULL stands for Sylvester's matrix of 128)");
  CTMI_REQUIRE(mb_t || ((uintptr_t)sign_in % 16 == 0 && (uintptr_t)sign_out % 16 == 0), CTMI_ERR_VALUE,
               "sign vectors must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  HadJobs t;
  clear_jobs(&t);
  int filled = 0;
  for (int64_t i = 0; i < n_jobs; ++i) {
    const ctmi_hadamard_pack_job& j = jobs[i];
    if (j.numel == 0) continue;
    t.x[filled] = j.x;
    t.out[filled] = j.packed;
    t.scale[filled] = j.scale;
    t.rotated[filled] = j.rotated;
    t.n_sub[filled] = j.numel / b_dim;
    t.end[filled] = (filled ? t.end[filled - 1] : 0) + cdiv(j.numel / b_dim, 16);
    if (++filled == kHadMaxJobs) {
      hqp_launch(t, filled, b_dim, mb_t, sign_in, sign_out, num_bits, st);
      clear_jobs(&t);
      filled = 0;
    }
  }
  bool any = false;
  for (int64_t i = 0; i < n_jobs; ++i) any |= jobs[i].numel != 0;
  if (!any) return CTMI_OK;
  if (filled) hqp_launch(t, filled, b_dim, mb_t, sign_in, sign_out, num_bits, st);
  return check_launch("ctmi_hadamard_quant_pack_many");
}

extern "C" int ctmi_hadamard_kron_quant_pack_many(const ctmi_hadamard_pack_job* jobs, int64_t n_jobs,
                                                  int32_t io_dtype, int32_t a_dim, int32_t b_dim,
                                                  const void* ma_t, const void* mb_t,
                                                  const float* sign_in, const float* sign_out,
                                                  int32_t group_size, int32_t num_bits,
                                                  int32_t symmetric, void* stream) {
  CTMI_REQUIRE(n_jobs >= 0 && (jobs || n_jobs == 0), CTMI_ERR_VALUE, "bad job list");
  CTMI_REQUIRE(io_dtype == CTMI_BF16, CTMI_ERR_UNSUPPORTED,
               "the fused rotation + quantization takes bfloat16 tensors");
  CTMI_REQUIRE((a_dim == 32 || a_dim == 64) && b_dim == 64, CTMI_ERR_UNSUPPORTED,
               "the fused rotation + quantization covers the factorisations 32 x 64 and 64 x 64, "
               "got %d x %d", a_dim, b_dim);
  CTMI_REQUIRE(group_size == 128, CTMI_ERR_UNSUPPORTED, "group size must be 128, got %d", group_size);
  CTMI_REQUIRE(num_bits == 4 && symmetric, CTMI_ERR_UNSUPPORTED,
               "only symmetric 4-bit integer quantization is fused");
  if (n_jobs == 0) return CTMI_OK;
  const int64_t n = (int64_t)a_dim * b_dim;
  for (int64_t i = 0; i < n_jobs; ++i) {
    const ctmi_hadamard_pack_job& j = jobs[i];
    CTMI_REQUIRE(j.numel >= 0 && j.numel % n == 0, CTMI_ERR_VALUE,
                 "job %lld: tensor size %lld is not a multiple of the transform size %lld",
                 (long long)i, (long long)j.numel, (long long)n);
    if (j.numel == 0) continue;
    CTMI_REQUIRE(j.x && j.packed && j.scale, CTMI_ERR_VALUE, "job %lld: NULL tensor pointer",
                 (long long)i);
    CTMI_REQUIRE((uintptr_t)j.x % 16 == 0 && (uintptr_t)j.rotated % 16 == 0 &&
                     (uintptr_t)j.packed % 4 == 0 && (uintptr_t)j.scale % 2 == 0,
                 CTMI_ERR_VALUE, "tensors must be 16-byte aligned");
  }
  CTMI_REQUIRE(mb_t && ma_t && (uintptr_t)mb_t % 16 == 0 && (uintptr_t)ma_t % 16 == 0, CTMI_ERR_VALUE,
               "the matrices must be given, 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  QpCfg c{};
  quant_range(CTMI_QTYPE_INT, num_bits, &c.bit_min, &c.bit_max);
  c.range = c.bit_max - c.bit_min;
  c.sym_div = (float)((double)c.range / 2.0);
  c.qtype = CTMI_QTYPE_INT;
  c.num_bits = num_bits;
  c.symmetric = 1;
  c.mt = c.zp_sub_dtype = c.scale_dtype = CTMI_BF16;
  c.zp_dtype = CTMI_I8;
  HadArgs a;
  a.x = nullptr;
  a.out = nullptr;
  a.mbt = (const uint16_t*)mb_t;
  a.mat = (const uint16_t*)ma_t;
  a.s_in = sign_in;
  a.s_out = sign_out;
  a.n_sub = 0;
  a.sqrt_n = sqrtf((float)n);
  HadJobs t;
  clear_jobs(&t);
  int filled = 0;
  bool any = false;
  auto flush = [&]() {
    if (a_dim == 32) launch_had_kron_quant_jobs<32>(t, filled, a, c, st);
    else launch_had_kron_quant_jobs<64>(t, filled, a, c, st);
    clear_jobs(&t);
    filled = 0;
  };
  for (int64_t i = 0; i < n_jobs; ++i) {
    const ctmi_hadamard_pack_job& j = jobs[i];
    if (j.numel == 0) continue;
    any = true;
    t.x[filled] = j.x;
    t.out[filled] = j.packed;
    t.scale[filled] = j.scale;
    t.rotated[filled] = j.rotated;
    t.n_sub[filled] = j.numel / b_dim;
    t.end[filled] = (filled ? t.end[filled - 1] : 0) + j.numel / n;
    if (++filled == kHadMaxJobs) flush();
  }
  if (!any) return CTMI_OK;
  if (filled) flush();
  return check_launch("ctmi_hadamard_kron_quant_pack_many");
}

extern "C" int ctmi_hadamard_quant_pack(const void* x, int32_t io_dtype, int64_t numel, int32_t b_dim,
                                        const void* mb_t, const float* sign_in,
                                        const float* sign_out, int32_t num_bits, int32_t symmetric,
                                        int32_t* packed, void* scale, void* rotated, void* stream) {
  ctmi_hadamard_pack_job job;
  job.x = x;
  job.packed = packed;
  job.scale = scale;
  job.rotated = rotated;
  job.numel = numel;
  int rc = ctmi_hadamard_quant_pack_many(&job, 1, io_dtype, b_dim, mb_t, sign_in, sign_out, num_bits,
                                         symmetric, stream);
  return rc;
}
