// Sylvester-Hadamard transforms of runs of 1024 ... 8192 elements
//
//   deterministic_hadamard_matrix, random_hadamard_matrix   transform/utils/hadamard.py:33-89
//   HadamardTransform.forward                               transform/factory/hadamard.py:104-121
//
// For a power of two n the reference's matrices are Sylvester's H_n, with a diagonal of random
// signs in front for the random kind.  x H_n needs no matrix: it is log2(n) butterfly stages,
// n additions each.
#include <utility>

#include "ctmi_device.h"
#include "ctmi_host.h"
#include "fwht.h"
#include "quant_fast.h"

namespace ctmi {
namespace {

// Sylvester transforms of 1024 ... 8192 elements: every butterfly stage in registers.
//
// The stages of a Walsh-Hadamard transform commute (one per bit of the element index), so a
// thread that holds 2^SB elements whose indices differ in SB chosen bits can run those SB
// stages on its own, and the run only has to be regrouped between such passes.  A workgroup
// of n / 2^SB threads takes a run through three groupings with the run in LDS in between:
//   pass 0  bits 0-2 and the top SB-3 bits: what a thread gets from 16-byte loads that the
//           wavefront issues over consecutive addresses
//   pass 1  bits 3 .. 3+SB-1
//   pass 2  the remaining bits (topped up with bits already done when there are fewer than SB)
// and back to the grouping of pass 0 for the stores.  12 stages of n = 4096 cost 12 additions
// per element and 6 LDS accesses, no matrix products and no splitting of the fp32
// intermediate into bfloat16 terms.  Per pass the slot offsets are compile-time constants
// (ds instruction offsets); a thread's base index is computed once.  The run is padded by 8
// floats every 2^(3+SB) elements, which spreads the 4-byte accesses of pass 1 over the banks.
template <int L, int SB>
struct FwhtPlan {
  static constexpr int kTop = SB - 3;
  static constexpr uint32_t kAll = (1u << L) - 1u;
  static constexpr uint32_t kMask0 = 7u | (((1u << kTop) - 1u) << (L - kTop));
  static constexpr uint32_t kMask1 = ((1u << SB) - 1u) << 3;
  static constexpr uint32_t kRest = kAll & ~(kMask0 | kMask1);
  static constexpr uint32_t top_up(uint32_t m) {
    for (int b = L - 1; b >= 0 && __builtin_popcount(m) < SB; --b) m |= 1u << b;
    return m;
  }
  static constexpr uint32_t kMask2 = top_up(kRest);
  static_assert(L >= 2 * SB && __builtin_popcount(kRest) <= SB, "three passes cover the index");
  static constexpr uint32_t mask(int pass) { return pass == 0 ? kMask0 : pass == 1 ? kMask1 : kMask2; }
  static constexpr uint32_t stages(int pass) { return pass == 0 ? kMask0 : pass == 1 ? kMask1 : kRest; }
  // bits of v placed at the set positions of m, lowest first
  static constexpr uint32_t deposit(uint32_t v, uint32_t m) {
    uint32_t e = 0;
    for (int b = 0; b < L; ++b)
      if ((m >> b) & 1u) {
        e |= (v & 1u) << b;
        v >>= 1;
      }
    return e;
  }
  static constexpr uint32_t padded(uint32_t e) { return e + ((e >> (3 + SB)) << 3); }
  static constexpr uint32_t kFloats = padded(1u << L);
  // slot r of a pass: offset in the padded run (base and offset have no bits in common, so
  // padded(base | off) = padded(base) + padded(off))
  static constexpr uint32_t slot(int pass, int r) { return padded(deposit((uint32_t)r, mask(pass))); }
  // does slot bit j of a pass stand for an index bit whose stage this pass runs?
  static constexpr bool runs_stage(int pass, int j) {
    const uint32_t pos = deposit(1u << j, mask(pass));
    return (stages(pass) & pos) != 0;
  }
  template <int PASS, int R>
  static constexpr uint32_t kSlot = slot(PASS, R);
  template <int PASS, int J>
  static constexpr bool kRuns = runs_stage(PASS, J);
};

template <typename P, int PASS, int S, int J>
__device__ __forceinline__ void fwht_stage(float (&v)[S]) {
  if constexpr (P::template kRuns<PASS, J>) {
#pragma unroll
    for (int i = 0; i < S; ++i) {
      if ((i & (1 << J)) == 0) {
        const float u = v[i], w = v[i + (1 << J)];
        v[i] = u + w;
        v[i + (1 << J)] = u - w;
      }
    }
  }
}

template <typename P, int PASS, int S, int... J>
__device__ __forceinline__ void fwht_slots(float (&v)[S], std::integer_sequence<int, J...>) {
  (fwht_stage<P, PASS, S, J>(v), ...);
}

template <typename P, int PASS, int S, int... R>
__device__ __forceinline__ void fwht_read_pass(const float* run, uint32_t base, float (&v)[S],
                                               std::integer_sequence<int, R...>) {
  ((v[R] = run[base + P::template kSlot<PASS, R>]), ...);
}

template <typename P, int PASS, int S, int... R>
__device__ __forceinline__ void fwht_write_pass(float* run, uint32_t base, const float (&v)[S],
                                                std::integer_sequence<int, R...>) {
  ((run[base + P::template kSlot<PASS, R>] = v[R]), ...);
}

// Between passes: a workgroup of one wavefront needs no barrier (its LDS instructions
// execute in order, and the compiler keeps stores and loads of the run in order)
template <int T>
__device__ __forceinline__ void fwht_sync() {
  if constexpr (T > kWave) __syncthreads();
}

template <typename P, int S, int... Q>
__device__ __forceinline__ void fwht_store_pass0(float* run, uint32_t base, const float (&v)[S],
                                                 std::integer_sequence<int, Q...>) {
  ((*reinterpret_cast<float4*>(&run[base + P::template kSlot<0, 4 * Q>]) =
        make_float4(v[4 * Q], v[4 * Q + 1], v[4 * Q + 2], v[4 * Q + 3])), ...);
}

template <typename P, int S, int... Q>
__device__ __forceinline__ void fwht_load_pass0(const float* run, uint32_t base, float (&v)[S],
                                                std::integer_sequence<int, Q...>) {
  float4 f[S / 4];
  ((f[Q] = *reinterpret_cast<const float4*>(&run[base + P::template kSlot<0, 4 * Q>])), ...);
#pragma unroll
  for (int q = 0; q < S / 4; ++q) {
    v[4 * q] = f[q].x;
    v[4 * q + 1] = f[q].y;
    v[4 * q + 2] = f[q].z;
    v[4 * q + 3] = f[q].w;
  }
}

// Up to kFwhtMaxJobs tensors per launch; a run is found by its number among all of them.
struct FwhtTable {
  const void* x[kFwhtMaxJobs];
  void* out[kFwhtMaxJobs];
  int32_t* packed[kFwhtMaxJobs];
  void* scale[kFwhtMaxJobs];
  int64_t end[kFwhtMaxJobs];  // running total of runs, job 0 .. j (unused: INT64_MAX)
  int64_t total;
};

// (a run number is the same in all lanes of a workgroup, which the compiler cannot always see:
// said outright, the search and the table reads behind it are scalar instructions; as vector
// loads they would make every prefetch wait for all loads in flight)
template <bool MANY>
__device__ __forceinline__ int fwht_job(const FwhtTable& t, int64_t run, int64_t* local) {
  if constexpr (!MANY) {
    *local = run;
    return 0;
  }
  {
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)run);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)run >> 32));
    run = (int64_t)(((uint64_t)hi << 32) | lo);
  }
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

// What a thread does with K finished vectors of 8 neighbouring elements, vector k at element
// (t * 8 + (q0 + k) * N / NVALL) of the run: scale, round, flip signs, then store, or
// (QUANT) quantize, pack and store.  flip: the thread's masks for all NVALL vectors.
template <typename IO, int N, int NVALL, int K, bool SIGN_OUT, bool QUANT>
__device__ __forceinline__ void fwht_emit(const float* v, int q0, uint32_t t, float factor,
                                          const uint32_t* flip, typename IO::raw* yr,
                                          int32_t* packed, void* scale_out, int64_t local,
                                          float rcp_div, const QpCfg& cfg) {
  using R = typename IO::raw;
  constexpr int DW = 8 * (int)sizeof(R) / 4;
  Vec<uint32_t, DW> o[K];
#pragma unroll
  for (int k = 0; k < K; ++k) {
    float f[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = v[k * 8 + i] * factor;
    o[k] = __builtin_bit_cast(Vec<uint32_t, DW>, pack8_from_f32<IO>(f));
    if constexpr (SIGN_OUT) {
#pragma unroll
      for (int d = 0; d < DW; ++d) o[k].v[d] ^= flip[(q0 + k) * DW + d];
    }
    if constexpr (!QUANT) stg_nt<R, 8>(yr + (q0 + k) * (N / NVALL), __builtin_bit_cast(Vec<R, 8>, o[k]));
  }
  if constexpr (QUANT) {
    static_assert(K % 2 == 0, "two vectors share a dword in the reduction");
    // max |x| of each group of 128: on the packed 16-bit halves inside a vector (bf16
    // magnitudes order like their bit patterns, a NaN above everything), then over the 16
    // lanes of the group by rotations within the row of 16, two vectors to a dword
    typedef uint16_t u16x2_t __attribute__((ext_vector_type(2)));
    auto pk_max = [](uint32_t x, uint32_t y) {
      return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2_t, x),
                                                                    __builtin_bit_cast(u16x2_t, y)));
    };
    uint32_t top[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const uint32_t m = pk_max(pk_max(o[k].v[0] & 0x7FFF7FFFu, o[k].v[1] & 0x7FFF7FFFu),
                                pk_max(o[k].v[2] & 0x7FFF7FFFu, o[k].v[3] & 0x7FFF7FFFu));
      top[k] = pk_max(m, m >> 16) & 0xFFFFu;  // the vector's maximum in the low half
    }
#pragma unroll
    for (int p = 0; p < K / 2; ++p) {
      uint32_t m = top[2 * p] | (top[2 * p + 1] << 16);
      m = pk_max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x128, 0xF, 0xF, false));  // row_ror:8
      m = pk_max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x124, 0xF, 0xF, false));  // row_ror:4
      m = pk_max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x122, 0xF, 0xF, false));  // row_ror:2
      m = pk_max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x121, 0xF, 0xF, false));  // row_ror:1
      top[2 * p] = m & 0xFFFFu;
      top[2 * p + 1] = m >> 16;
    }
#pragma unroll
    for (int k = 0; k < K; ++k) {
      // calculate_qparams, symmetric, in bf16 (helpers.py:101-122): bf16(max / 7.5); the
      // product with the reciprocal rounds to the same bf16 (both operands have 8-bit
      // significands, so the quotient keeps its distance from every rounding midpoint)
      const uint32_t mag = top[k];
      float sv = bf16_lo(pack_bf16x2(bf16_to_f32((uint16_t)mag) * rcp_div, 0.0f));
      sv = mag > 0x7F80u ? __uint_as_float(0x7FC00000u) : fmaxf(sv, 1.1920928955078125e-07f);
      const Vec<int32_t, 1> word = quant_pack8<BF16, BF16, 4, false>(
          __builtin_bit_cast(Vec<uint16_t, 8>, o[k]), sv, 0.0f, cfg.bit_min, cfg.bit_max);
      const int64_t vec = local * (N / 8) + t + (q0 + k) * (N / NVALL / 8);  // this vector's number in the tensor
      __builtin_nontemporal_store(word.v[0], packed + vec);
      // sv is a bf16 value: its upper half is its encoding
      if ((t & 15u) == 0) static_cast<uint16_t*>(scale_out)[vec >> 4] = (uint16_t)(__float_as_uint(sv) >> 16);
      if (yr) stg_nt<R, 8>(yr + (q0 + k) * (N / NVALL), __builtin_bit_cast(Vec<R, 8>, o[k]));
    }
  }
}

// QUANT (bfloat16): the rotated values are rounded to bfloat16 and go through the W4A16
// pipeline for group size 128 before they leave the registers: a group is the vectors of 16
// neighbouring lanes, which agree on max |x| through four lane exchanges; each lane then
// quantizes its 8 values with the group's scale and packs them into one word
// (min-max observer, calculate_qparams and pack_to_int32 as in ctmi_observe_pack_quantized).
template <typename IO, int L, int SB, bool SIGN_IN, bool SIGN_OUT, bool MANY, bool QUANT>
__global__ void __launch_bounds__(1 << (L - SB))
fwht_lds_kernel(FwhtTable tab, const float* __restrict__ sign_in, const float* __restrict__ sign_out,
                const float* __restrict__ w0, float scale, QpCfg cfg) {
  static_assert(!QUANT || IO::id == CTMI_BF16, "the fused epilogue is written for bfloat16");
  using P = FwhtPlan<L, SB>;
  using R = typename IO::raw;
  constexpr int N = 1 << L, S = 1 << SB, NV = S / 8, T = N >> SB;
  __shared__ __attribute__((aligned(16))) float run[P::kFloats];
  const uint32_t t = threadIdx.x;
  const uint32_t base0 = P::padded(t << 3);
  const uint32_t base1 = P::padded(P::deposit(t, P::kAll & ~P::kMask1));
  const uint32_t base2 = P::padded(P::deposit(t, P::kAll & ~P::kMask2));
  const float factor = (w0 ? w0[0] : 1.0f) * scale;
  // This thread's signs, the same for every run, as masks on the sign bits of the raw
  // elements (a vector of 8 is DW dwords): x * (+-1) is a flipped sign bit, and two 16-bit
  // elements flip in one instruction.
  constexpr int DW = 8 * (int)sizeof(R) / 4;
  uint32_t flip_in[SIGN_IN ? NV * DW : 1], flip_out[SIGN_OUT ? NV * DW : 1];
  auto sign_masks = [&](const float* __restrict__ signs, uint32_t* flip) {
#pragma unroll
    for (int q = 0; q < NV; ++q) {
      const Vec<uint32_t, 8> s8 = ldg<uint32_t, 8>(reinterpret_cast<const uint32_t*>(signs) + (t << 3) + q * (N / NV));
#pragma unroll
      for (int d = 0; d < DW; ++d) {
        if constexpr (sizeof(R) == 2)
          flip[q * DW + d] = ((s8.v[2 * d] >> 16) & 0x8000u) | (s8.v[2 * d + 1] & 0x80000000u);
        else
          flip[q * DW + d] = s8.v[d] & 0x80000000u;
      }
    }
  };
  if constexpr (SIGN_IN) sign_masks(sign_in, flip_in);
  if constexpr (SIGN_OUT) sign_masks(sign_out, flip_out);
  const float rcp_div = QUANT ? 1.0f / cfg.sym_div : 0.0f;

  // the next run's loads are in flight while this one goes through its passes
  Vec<R, 8> in[NV];
  auto fetch = [&](int64_t r) {
    if (r < tab.total) {
      int64_t local;
      const int j = fwht_job<MANY>(tab, r, &local);
      const R* __restrict__ xr = static_cast<const R*>(tab.x[j]) + local * N + (t << 3);
#pragma unroll
      for (int q = 0; q < NV; ++q) in[q] = ldg_nt<R, 8>(xr + q * (N / NV));
    }
  };
  const int64_t step = gridDim.x;
  fetch(blockIdx.x);
  for (int64_t row = blockIdx.x; row < tab.total; row += step) {
    float v[S];
#pragma unroll
    for (int q = 0; q < NV; ++q) {
      Vec<uint32_t, DW> raw = __builtin_bit_cast(Vec<uint32_t, DW>, in[q]);
      if constexpr (SIGN_IN) {
#pragma unroll
        for (int d = 0; d < DW; ++d) raw.v[d] ^= flip_in[q * DW + d];
      }
      const Vec<R, 8> xq = __builtin_bit_cast(Vec<R, 8>, raw);
#pragma unroll
      for (int i = 0; i < 8; ++i) v[q * 8 + i] = IO::to_f32(xq.v[i]);
    }
    fetch(row + step);
    fwht_slots<P, 0, S>(v, std::make_integer_sequence<int, SB>{});
    // no barrier before this: what a thread overwrites of the previous run only this thread
    // read (same grouping), after the barrier that ended that run's last pass
    fwht_store_pass0<P, S>(run, base0, v, std::make_integer_sequence<int, S / 4>{});
    fwht_sync<T>();
    fwht_read_pass<P, 1, S>(run, base1, v, std::make_integer_sequence<int, S>{});
    fwht_slots<P, 1, S>(v, std::make_integer_sequence<int, SB>{});
    fwht_write_pass<P, 1, S>(run, base1, v, std::make_integer_sequence<int, S>{});
    fwht_sync<T>();
    if constexpr (P::kRest != 0) {
      fwht_read_pass<P, 2, S>(run, base2, v, std::make_integer_sequence<int, S>{});
      fwht_slots<P, 2, S>(v, std::make_integer_sequence<int, SB>{});
      fwht_write_pass<P, 2, S>(run, base2, v, std::make_integer_sequence<int, S>{});
      fwht_sync<T>();
    }
    fwht_load_pass0<P, S>(run, base0, v, std::make_integer_sequence<int, S / 4>{});
    int64_t local;
    const int j = fwht_job<MANY>(tab, row, &local);
    R* yr = static_cast<R*>(tab.out[j]);
    if (!QUANT || yr) yr += local * N + (t << 3);
    fwht_emit<IO, N, NV, NV, SIGN_OUT, QUANT>(v, 0, t, factor, flip_out, yr, QUANT ? tab.packed[j] : nullptr,
                                              QUANT ? tab.scale[j] : nullptr, local, rcp_div, cfg);
  }
}

// Runs of 4096 bfloat16 elements, half of the stages on the matrix cores.
//
// A run is a 64 x 64 matrix Z (element 64 i + j) and its transform is H Z H.  The factor over
// j takes bfloat16 inputs, so Z H is exact as one product on the matrix cores (no splitting of
// anything into bfloat16 terms): 16 instructions v_mfma_f32_32x32x16_bf16 whose A operands
// are 16-byte pieces of the rows of Z (loaded as whole lines, then picked out of an image of
// the run in LDS: loading the pieces directly makes four instructions share every line, and
// measured a third slower) and whose B operands are pieces of H that never change.  In the accumulators a lane holds, for one column j', rows
// i = 32 rt + 8 b + 4 g + r with g = lane / 32: one exchange between the lane halves
// (v_permlane32_swap, paired with the butterfly over g) leaves lane l with all 64 rows of
// column j' = l, and the other five stages over i are additions in registers.  The run then
// goes through LDS once more, half a run at a time, to reach the layout of the stores: 8
// neighbouring elements a lane, lanes side by side.  9 KB of LDS a wavefront.
// Per element: 6 butterfly additions instead of 12, LDS traffic of 6 bytes each way instead
// of 12.
typedef __bf16 fwht_bf16x8_t __attribute__((ext_vector_type(8)));
typedef float fwht_f32x16_t __attribute__((ext_vector_type(16)));

#ifndef CTMI_FWHT_MFMA_PLAIN_WAVES
#define CTMI_FWHT_MFMA_PLAIN_WAVES 4  // wavefronts per SIMD the variant without signs is compiled for (128 registers)
#endif
template <bool SIGN_IN, bool SIGN_OUT, bool MANY, bool QUANT>
__global__ void __launch_bounds__(kWave, (!SIGN_IN && !SIGN_OUT && !QUANT) ? CTMI_FWHT_MFMA_PLAIN_WAVES : 1)
fwht_mfma_kernel(FwhtTable tab, const float* __restrict__ sign_in, const float* __restrict__ sign_out,
                 const float* __restrict__ w0, float scale, QpCfg cfg) {
  constexpr int N = 4096, NV = 8;
  // One buffer, two uses per run: the run as it comes from memory (64 rows of 64 bfloat16,
  // 144 bytes apart so that the 16-byte pieces the lanes pick out of 32 different rows fall
  // into different banks), then half the transformed run as fp32 (32 rows of 64).  All
  // accesses are dword vectors, so the compiler keeps them in program order.
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  constexpr int kPitch = 36;  // dwords between rows of the bfloat16 image
  __shared__ __attribute__((aligned(16))) uint32_t lds[64 * kPitch];
  const uint32_t l = threadIdx.x, c = l & 31u, g = l >> 5;
  const float factor = (w0 ? w0[0] : 1.0f) * scale;
  const float rcp_div = QUANT ? 1.0f / cfg.sym_div : 0.0f;
  // H[k][j'] = (-1)^popcount(k & j') for k = 16 ks + 8 g + e, j' = 32 ct + c, as bf16:
  // (-1)^popcount((8 g + e) & c) for ks = 0, times (-1)^(c >> 4) for odd ks, times -1 for
  // ks >= 2 in the upper column tile (that sign goes to the other operand)
  u32x4 h_even, h_odd;
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const uint32_t k0 = 8 * g + 2 * d;
    const uint32_t lo = (__builtin_popcount(k0 & c) & 1) ? 0xBF80u : 0x3F80u;
    const uint32_t hi = (__builtin_popcount((k0 + 1) & c) & 1) ? 0xBF80u : 0x3F80u;
    h_even[d] = lo | (hi << 16);
    h_odd[d] = h_even[d] ^ ((c & 16u) ? 0x80008000u : 0u);
  }
  // sign masks of this lane's vectors (elements 8 l + 512 q + e), in and out
  uint32_t flip_in[SIGN_IN ? 32 : 1], flip_out[SIGN_OUT ? 32 : 1];
  auto sign_masks = [&](const float* __restrict__ signs, uint32_t* flip) {
#pragma unroll
    for (int q = 0; q < NV; ++q) {
      const Vec<uint32_t, 8> s8 = ldg<uint32_t, 8>(reinterpret_cast<const uint32_t*>(signs) + (l << 3) + 512 * q);
#pragma unroll
      for (int d = 0; d < 4; ++d)
        flip[q * 4 + d] = ((s8.v[2 * d] >> 16) & 0x8000u) | (s8.v[2 * d + 1] & 0x80000000u);
    }
  };
  if constexpr (SIGN_IN) sign_masks(sign_in, flip_in);
  if constexpr (SIGN_OUT) sign_masks(sign_out, flip_out);
  // the next run's loads are in flight while this one is worked on
  u32x4 in[NV];
  auto fetch = [&](int64_t r) {
    if (r < tab.total) {
      int64_t local;
      const int j = fwht_job<MANY>(tab, r, &local);
      const uint16_t* __restrict__ xr = static_cast<const uint16_t*>(tab.x[j]) + local * N + (l << 3);
#pragma unroll
      for (int q = 0; q < NV; ++q)
        in[q] = __builtin_bit_cast(u32x4, ldg_nt<uint16_t, 8>(xr + 512 * q));
    }
  };
  const int64_t step = gridDim.x;
  fetch(blockIdx.x);
  for (int64_t row = blockIdx.x; row < tab.total; row += step) {
    // vector l + 64 q is row (l / 8 + 8 q) of Z, columns 8 (l % 8) ...
#pragma unroll
    for (int q = 0; q < NV; ++q) {
      u32x4 w = in[q];
      if constexpr (SIGN_IN) {
#pragma unroll
        for (int d = 0; d < 4; ++d) w[d] ^= flip_in[q * 4 + d];
      }
      *reinterpret_cast<u32x4*>(&lds[((l >> 3) + 8 * q) * kPitch + 4 * (l & 7u)]) = w;
    }
    fetch(row + step);
    fwht_f32x16_t acc[2][2];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int ct = 0; ct < 2; ++ct)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[rt][ct][i] = 0.0f;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int rt = 0; rt < 2; ++rt) {
        // A operand: row 32 rt + c of Z, columns 16 ks + 8 g ...
        const u32x4 a = *reinterpret_cast<const u32x4*>(&lds[(32 * rt + c) * kPitch + 8 * ks + 4 * g]);
        const fwht_bf16x8_t hf = __builtin_bit_cast(fwht_bf16x8_t, (ks & 1) ? h_odd : h_even);
        acc[rt][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(fwht_bf16x8_t, a), hf,
                                                             acc[rt][0], 0, 0, 0);
        const u32x4 a1 = ks >= 2 ? a ^ 0x80008000u : a;
        acc[rt][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(fwht_bf16x8_t, a1), hf,
                                                             acc[rt][1], 0, 0, 0);
      }
    // acc[rt][ct][4 b + r] = (Z H)[32 rt + 8 b + 4 g + r][32 ct + c].  The exchange pairs the two
    // column tiles: afterwards lane l has column j' = l, and u[i] for all 64 rows i.
    float u[64];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int bv = 0; bv < 16; ++bv) {
        const auto pr = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc[rt][0][bv]),
                                                         __float_as_uint(acc[rt][1][bv]), false, false);
        const float lower = __uint_as_float(pr[0]), upper = __uint_as_float(pr[1]);  // g = 0, g = 1
        const int i0 = 32 * rt + 8 * (bv >> 2) + (bv & 3);
        u[i0] = lower + upper;
        u[i0 + 4] = lower - upper;
      }
#pragma unroll
    for (int st = 1; st < 64; st <<= 1) {
      if (st == 4) continue;  // the stage over g is done
#pragma unroll
      for (int i = 0; i < 64; ++i) {
        if ((i & st) == 0) {
          const float p = u[i], m = u[i + st];
          u[i] = p + m;
          u[i + st] = p - m;
        }
      }
    }
    int64_t local;
    const int j = fwht_job<MANY>(tab, row, &local);
    uint16_t* yr = static_cast<uint16_t*>(tab.out[j]);
    if (!QUANT || yr) yr += local * N + (l << 3);
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      // rows 32 hf ... 32 hf + 31 of the run through LDS: lane l writes its column, then reads
      // the vectors l, l + 64, l + 128, l + 192 of this half (8 neighbouring elements each)
#pragma unroll
      for (int ii = 0; ii < 32; ++ii) lds[ii * 64 + l] = __float_as_uint(u[32 * hf + ii]);
      float v[32];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const u32x4 f0 = *reinterpret_cast<const u32x4*>(&lds[(l + 64 * q) * 8]);
        const u32x4 f1 = *reinterpret_cast<const u32x4*>(&lds[(l + 64 * q) * 8 + 4]);
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          v[q * 8 + d] = __uint_as_float(f0[d]);
          v[q * 8 + 4 + d] = __uint_as_float(f1[d]);
        }
      }
      fwht_emit<BF16, N, NV, 4, SIGN_OUT, QUANT>(v, 4 * hf, l, factor, flip_out, yr,
                                                 QUANT ? tab.packed[j] : nullptr,
                                                 QUANT ? tab.scale[j] : nullptr, local, rcp_div, cfg);
    }
  }
}

#ifndef CTMI_FWHT_STREAM_FROM
#define CTMI_FWHT_STREAM_FROM 8192
#endif
// A workgroup takes every grid-th run, so all workgroups have to be resident together and
// carry equally many runs: one that starts when another has finished runs alone for as long
// again.  How many fit a compute unit (registers, LDS) is the runtime's to say; *resident_wgs
// caches the answer per kernel (the same on every device of one process: one architecture).
template <typename Kernel>
int launch_persistent(Kernel kern, int threads, int* resident_wgs, const FwhtTable& tab,
                      const float* sign_in, const float* sign_out, const float* w0, float scale,
                      const QpCfg& cfg, hipStream_t st, int64_t stream_from = INT64_MAX) {
  if (*resident_wgs == 0) {
    int per_cu = 0, dev = 0, cus = 0;
    hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, threads, 0);
    if (e == hipSuccess) e = hipGetDevice(&dev);
    if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return set_error(CTMI_ERR_HIP, "occupancy query: %s", hipGetErrorString(e));
    *resident_wgs = (per_cu > 0 ? per_cu : 1) * (cus > 0 ? cus : 256);
  }
  const int64_t resident = *resident_wgs;
  // (stream_from: from that many runs on a workgroup takes one run and leaves, and the
  // hardware hands out the runs)
  const int64_t runs_each = tab.total >= stream_from ? 1 : (tab.total + resident - 1) / resident;
  const unsigned grid = (unsigned)((tab.total + runs_each - 1) / runs_each);
  hipLaunchKernelGGL(kern, grid, threads, 0, st, tab, sign_in, sign_out, w0, scale, cfg);
  return CTMI_OK;
}

template <typename IO, int L, int SB, bool SIGN_IN, bool SIGN_OUT, bool MANY, bool QUANT>
int launch_fwht_variant(const FwhtTable& tab, const float* sign_in, const float* sign_out,
                        const float* w0, float scale, const QpCfg& cfg, hipStream_t st) {
  static int resident_wgs = 0;
  return launch_persistent(fwht_lds_kernel<IO, L, SB, SIGN_IN, SIGN_OUT, MANY, QUANT>, 1 << (L - SB),
                           &resident_wgs, tab, sign_in, sign_out, w0, scale, cfg, st);
}

template <bool SIGN_IN, bool SIGN_OUT, bool MANY, bool QUANT>
int launch_fwht_mfma_variant(const FwhtTable& tab, const float* sign_in, const float* sign_out,
                             const float* w0, float scale, const QpCfg& cfg, hipStream_t st) {
  static int resident_wgs = 0;
  // The rotation alone on 8192 runs or more: one run per workgroup (14336x4096: 0.70 of the HBM
  // peak against 0.65 with every workgroup resident and looping; at 4096 runs the loop wins,
  // 0.62 against 0.50, and with the quantization behind it the loop wins at every size).
  return launch_persistent(fwht_mfma_kernel<SIGN_IN, SIGN_OUT, MANY, QUANT>, kWave, &resident_wgs, tab,
                           sign_in, sign_out, w0, scale, cfg, st, QUANT ? INT64_MAX : CTMI_FWHT_STREAM_FROM);
}

template <bool QUANT>
int launch_fwht_mfma(const FwhtTable& tab, bool many, const float* si, const float* so, const float* w0,
                     float scale, const QpCfg& cfg, hipStream_t st) {
#define CTMI_FWHT_CASE(IN, OUT)                                                                  \
  return many ? launch_fwht_mfma_variant<IN, OUT, true, QUANT>(tab, si, so, w0, scale, cfg, st)  \
              : launch_fwht_mfma_variant<IN, OUT, false, QUANT>(tab, si, so, w0, scale, cfg, st)
  if (si && so) CTMI_FWHT_CASE(true, true);
  if (si) CTMI_FWHT_CASE(true, false);
  if (so) CTMI_FWHT_CASE(false, true);
  CTMI_FWHT_CASE(false, false);
#undef CTMI_FWHT_CASE
}

template <typename IO, int L, int SB, bool QUANT>
int launch_fwht_size(const FwhtTable& tab, bool many, const float* si, const float* so, const float* w0,
                     float scale, const QpCfg& cfg, hipStream_t st) {
#define CTMI_FWHT_CASE(IN, OUT)                                                                    \
  return many ? launch_fwht_variant<IO, L, SB, IN, OUT, true, QUANT>(tab, si, so, w0, scale, cfg, st) \
              : launch_fwht_variant<IO, L, SB, IN, OUT, false, QUANT>(tab, si, so, w0, scale, cfg, st)
  if (si && so) CTMI_FWHT_CASE(true, true);
  if (si) CTMI_FWHT_CASE(true, false);
  if (so) CTMI_FWHT_CASE(false, true);
  CTMI_FWHT_CASE(false, false);
#undef CTMI_FWHT_CASE
}

#ifndef CTMI_FWHT_SB
#define CTMI_FWHT_SB 4, 4, 6, 5  // log2 of the elements a thread holds for runs of 1024 ... 8192
#endif

template <typename IO, bool QUANT>
int launch_fwht(int n, const FwhtTable& tab, bool many, const float* si, const float* so,
                const float* w0, float scale, const QpCfg& cfg, hipStream_t st) {
  constexpr int kSb[4] = {CTMI_FWHT_SB};
#ifndef CTMI_FWHT_4096_MFMA
#define CTMI_FWHT_4096_MFMA 1  // bfloat16 runs of 4096: the kernel that shares the work with the matrix cores
#endif
  if constexpr (CTMI_FWHT_4096_MFMA && IO::id == CTMI_BF16) {
    if (n == 4096) return launch_fwht_mfma<QUANT>(tab, many, si, so, w0, scale, cfg, st);
  }
  switch (n) {
    case 1024: return launch_fwht_size<IO, 10, kSb[0], QUANT>(tab, many, si, so, w0, scale, cfg, st);
    case 2048: return launch_fwht_size<IO, 11, kSb[1], QUANT>(tab, many, si, so, w0, scale, cfg, st);
    case 4096: return launch_fwht_size<IO, 12, kSb[2], QUANT>(tab, many, si, so, w0, scale, cfg, st);
    default: return launch_fwht_size<IO, 13, kSb[3], QUANT>(tab, many, si, so, w0, scale, cfg, st);
  }
}

}  // namespace

int fwht_launch(const FwhtJob* jobs, int n_jobs, int io_dtype, int n, const float* sign_in,
                const float* sign_out, const float* w0, float scale, const QpCfg* quant,
                hipStream_t st) {
  CTMI_REQUIRE(fwht_size_supported(n), CTMI_ERR_UNSUPPORTED, "no butterfly kernel for runs of %d elements", n);
  CTMI_REQUIRE(n_jobs >= 1 && n_jobs <= kFwhtMaxJobs, CTMI_ERR_VALUE, "1 to %d tensors a launch", kFwhtMaxJobs);
  CTMI_REQUIRE(!quant || io_dtype == CTMI_BF16, CTMI_ERR_UNSUPPORTED,
               "the fused rotation + quantization takes bfloat16 tensors");
  CTMI_REQUIRE((uintptr_t)sign_in % 16 == 0 && (uintptr_t)sign_out % 16 == 0, CTMI_ERR_VALUE,
               "sign vectors must be 16-byte aligned");
  FwhtTable tab;
  int64_t total = 0;
  for (int i = 0; i < kFwhtMaxJobs; ++i) {
    const bool live = i < n_jobs;
    tab.x[i] = live ? jobs[i].x : nullptr;
    tab.out[i] = live ? jobs[i].out : nullptr;
    tab.packed[i] = live ? jobs[i].packed : nullptr;
    tab.scale[i] = live ? jobs[i].scale : nullptr;
    if (live) {
      CTMI_REQUIRE(jobs[i].rows > 0 && jobs[i].x && (quant ? jobs[i].packed && jobs[i].scale : jobs[i].out != nullptr),
                   CTMI_ERR_VALUE, "tensor %d: NULL pointer or no runs", i);
      CTMI_REQUIRE((uintptr_t)jobs[i].x % 16 == 0 && (uintptr_t)jobs[i].out % 16 == 0 &&
                       (uintptr_t)jobs[i].packed % 4 == 0 && (uintptr_t)jobs[i].scale % 2 == 0,
                   CTMI_ERR_VALUE, "a transform of %d elements takes tensors aligned to 16 bytes", n);
      total += jobs[i].rows;
    }
    tab.end[i] = live ? total : INT64_MAX;
  }
  tab.total = total;
  const QpCfg none{};
  const bool many = n_jobs > 1;
  if (quant) return launch_fwht<BF16, true>(n, tab, many, sign_in, sign_out, w0, scale, *quant, st);
  switch (io_dtype) {
    case CTMI_BF16: return launch_fwht<BF16, false>(n, tab, many, sign_in, sign_out, w0, scale, none, st);
    case CTMI_F16: return launch_fwht<F16, false>(n, tab, many, sign_in, sign_out, w0, scale, none, st);
    case CTMI_F32: return launch_fwht<F32, false>(n, tab, many, sign_in, sign_out, w0, scale, none, st);
    default: return set_error(CTMI_ERR_UNSUPPORTED, "transforms take float16/bfloat16/float32 tensors");
  }
}

}  // namespace ctmi

using namespace ctmi;

extern "C" int ctmi_sylvester_supported(int32_t n, int32_t io_dtype) {
  return fwht_size_supported(n) && (io_dtype == CTMI_BF16 || io_dtype == CTMI_F16 || io_dtype == CTMI_F32);
}

extern "C" int ctmi_sylvester_apply_many(const ctmi_hadamard_job* jobs, int64_t n_jobs, int32_t io_dtype,
                                         int32_t n, const float* sign_in, const float* sign_out,
                                         void* stream) {
  CTMI_REQUIRE(n_jobs >= 0 && (jobs || n_jobs == 0), CTMI_ERR_VALUE, "bad job list");
  CTMI_REQUIRE(io_dtype == CTMI_BF16 || io_dtype == CTMI_F16 || io_dtype == CTMI_F32,
               CTMI_ERR_UNSUPPORTED, "transforms take float16/bfloat16/float32 tensors");
  CTMI_REQUIRE(fwht_size_supported(n), CTMI_ERR_UNSUPPORTED,
               "Sylvester transforms of 1024, 2048, 4096 and 8192 elements are built, not %d", n);
  // everything is checked before anything is enqueued
  for (int64_t i = 0; i < n_jobs; ++i) {
    const ctmi_hadamard_job& j = jobs[i];
    CTMI_REQUIRE(j.numel >= 0 && j.numel % n == 0, CTMI_ERR_VALUE,
                 "job %lld: tensor size %lld is not a multiple of the transform size %d", (long long)i,
                 (long long)j.numel, n);
    CTMI_REQUIRE(j.numel == 0 || (j.x && j.out), CTMI_ERR_VALUE, "job %lld: NULL tensor pointer", (long long)i);
    CTMI_REQUIRE((uintptr_t)j.x % 16 == 0 && (uintptr_t)j.out % 16 == 0, CTMI_ERR_VALUE,
                 "job %lld: tensors must be 16-byte aligned", (long long)i);
  }
  CTMI_REQUIRE((uintptr_t)sign_in % 16 == 0 && (uintptr_t)sign_out % 16 == 0, CTMI_ERR_VALUE,
               "sign vectors must be 16-byte aligned");
  const float scale = 1.0f / sqrtf((float)n);
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
      const int rc = fwht_launch(batch, filled, io_dtype, n, sign_in, sign_out, nullptr, scale, nullptr,
                                 (hipStream_t)stream);
      if (rc) return rc;
      filled = 0;
      any = true;
    }
  }
  return any ? check_launch("ctmi_sylvester_apply_many") : CTMI_OK;
}

extern "C" int ctmi_sylvester_quant_pack_many(const ctmi_hadamard_pack_job* jobs, int64_t n_jobs,
                                              int32_t io_dtype, int32_t n, const float* sign_in,
                                              const float* sign_out, int32_t group_size,
                                              int32_t num_bits, int32_t symmetric, void* stream) {
  CTMI_REQUIRE(n_jobs >= 0 && (jobs || n_jobs == 0), CTMI_ERR_VALUE, "bad job list");
  CTMI_REQUIRE(io_dtype == CTMI_BF16, CTMI_ERR_UNSUPPORTED,
               "the fused rotation + quantization takes bfloat16 tensors");
  CTMI_REQUIRE(fwht_size_supported(n), CTMI_ERR_UNSUPPORTED,
               "Sylvester transforms of 1024, 2048, 4096 and 8192 elements are built, not %d", n);
  CTMI_REQUIRE(group_size == 128, CTMI_ERR_UNSUPPORTED, "group size must be 128, got %d", group_size);
  CTMI_REQUIRE(num_bits == 4 && symmetric, CTMI_ERR_UNSUPPORTED,
               "only symmetric 4-bit integer quantization is fused");
  for (int64_t i = 0; i < n_jobs; ++i) {
    const ctmi_hadamard_pack_job& j = jobs[i];
    CTMI_REQUIRE(j.numel >= 0 && j.numel % n == 0, CTMI_ERR_VALUE,
                 "job %lld: tensor size %lld is not a multiple of the transform size %d", (long long)i,
                 (long long)j.numel, n);
    CTMI_REQUIRE(j.numel == 0 || (j.x && j.packed && j.scale), CTMI_ERR_VALUE,
                 "job %lld: NULL tensor pointer", (long long)i);
    CTMI_REQUIRE((uintptr_t)j.x % 16 == 0 && (uintptr_t)j.rotated % 16 == 0 &&
                     (uintptr_t)j.packed % 4 == 0 && (uintptr_t)j.scale % 2 == 0,
                 CTMI_ERR_VALUE, "job %lld: tensors must be 16-byte aligned", (long long)i);
  }
  CTMI_REQUIRE((uintptr_t)sign_in % 16 == 0 && (uintptr_t)sign_out % 16 == 0, CTMI_ERR_VALUE,
               "sign vectors must be 16-byte aligned");
  QpCfg c{};
  quant_range(CTMI_QTYPE_INT, num_bits, &c.bit_min, &c.bit_max);
  c.range = c.bit_max - c.bit_min;
  c.sym_div = (float)((double)c.range / 2.0);
  c.qtype = CTMI_QTYPE_INT;
  c.num_bits = num_bits;
  c.symmetric = 1;
  c.mt = c.zp_sub_dtype = c.scale_dtype = CTMI_BF16;
  c.zp_dtype = CTMI_I8;
  const float scale = 1.0f / sqrtf((float)n);
  FwhtJob batch[kFwhtMaxJobs];
  int filled = 0;
  bool any = false;
  for (int64_t i = 0; i <= n_jobs; ++i) {
    if (i < n_jobs && jobs[i].numel > 0) {
      FwhtJob& b = batch[filled++];
      b.x = jobs[i].x;
      b.out = jobs[i].rotated;
      b.packed = jobs[i].packed;
      b.scale = jobs[i].scale;
      b.rows = jobs[i].numel / n;
    }
    if (filled == kFwhtMaxJobs || (i == n_jobs && filled)) {
      const int rc = fwht_launch(batch, filled, io_dtype, n, sign_in, sign_out, nullptr, scale, &c,
                                 (hipStream_t)stream);
      if (rc) return rc;
      filled = 0;
      any = true;
    }
  }
  return any ? check_launch("ctmi_sylvester_quant_pack_many") : CTMI_OK;
}

