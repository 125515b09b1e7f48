// FP4 e2m1 nibble packing (nvfp4-pack-quantized format).
//
//   pack_fp4_to_uint8      compressors/quantized_compressors/fp4_quantized.py:135-178
//   unpack_fp4_from_uint8  fp4_quantized.py:187-221
//   NVFP4PackedCompressor.compress_weight / decompress_weight  fp4_quantized.py:84-123
//
// Code = 3-bit index into {0,.5,1,1.5,2,3,4,6} | sign bit << 3; element 2j is
// the low nibble of byte j, element 2j+1 the high nibble.
#include <type_traits>

#include "ctmi_device.h"
#include "ctmi_host.h"
#include "minmax.h"
#include "qdq_core.h"
#include "qparams.h"
#include "quant_core.h"
#include "quant_fast.h"
#include "job_table.h"
#include "vec_geom.h"

namespace ctmi {

// Index chosen by the reference for one element: argmin_k |(|x| - lut[k])|
// with the subtraction rounded to x's dtype (the reference subtracts tensors
// of that dtype) and the first minimum winning; NaN distances win outright,
// as in torch.argmin.  Values that sit on the e2m1 grid — the only ones a
// quantized tensor holds — take the short path.
template <int XDT>
__device__ __forceinline__ int fp4_nearest_code(float x) {
  const float a = fabsf(x);
  int c = fp4_bucket(a);
  if (fp4_code_to_f32(c) != a) {
    c = 0;
    float best = fabsf(round_ct<XDT>(a - 0.0f));
    if (best == best) {
#pragma unroll
      for (int k = 1; k < 8; ++k) {
        const float d = fabsf(round_ct<XDT>(a - fp4_code_to_f32(k)));
        if (d != d) { c = k; break; }
        if (d < best) { best = d; c = k; }
      }
    }
  }
  return c | ((int)(f2u(x) >> 31) << 3);
}

__device__ __forceinline__ int fp4_nearest_code_rt(float x, int xdt) {
  if (xdt == CTMI_BF16) return fp4_nearest_code<CTMI_BF16>(x);
  if (xdt == CTMI_F16) return fp4_nearest_code<CTMI_F16>(x);
  return fp4_nearest_code<CTMI_F32>(x);
}

// 8 fp32 values -> 8 e2m1 codes (element i in bits [4i, 4i+4)) with the hardware
// converter: round to nearest even on the e2m1 grid = the reference's bucket
// boundaries (quant_args.py:55-68), saturating at +-6, sign kept.
__device__ __forceinline__ uint32_t fp4_pack8_hw(const float* t) {
  uint32_t w = 0;
  w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, t[0], t[1], 1.0f, 0);
  w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, t[2], t[3], 1.0f, 1);
  w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, t[4], t[5], 1.0f, 2);
  w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, t[6], t[7], 1.0f, 3);
  return w;
}

// 8 codes of a dword -> 8 fp32 values (exact; code 8 is -0.0)
__device__ __forceinline__ void fp4_unpack8_hw(uint32_t w, float* t) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  f32x2 r;
  r = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 0); t[0] = r.x; t[1] = r.y;
  r = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 1); t[2] = r.x; t[3] = r.y;
  r = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 2); t[4] = r.x; t[5] = r.y;
  r = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 3); t[6] = r.x; t[7] = r.y;
}

// ------------------------------------------------------------------ standalone pack / unpack
// 8 elements -> one 32-bit word; a lane takes kFp4Vecs of them, all loads first; the tensor is
// read and written once: streaming loads and stores
constexpr int kFp4Vecs = 4;

template <typename XT>
__global__ void __launch_bounds__(256)
fp4_pack_vec_kernel(const typename XT::raw* __restrict__ x, uint32_t* __restrict__ out,
                    int64_t nvec) {
  constexpr int U = kFp4Vecs;
  constexpr int H = 16 / (int)sizeof(typename XT::raw);  // elements of a 16-byte load
  const int64_t v0 = (int64_t)blockIdx.x * (256 * U) + threadIdx.x;
  Vec<typename XT::raw, H> a[U][8 / H];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t v = v0 + k * 256;
    const typename XT::raw* at = x + (v < nvec ? v : nvec - 1) * 8;  // past the end: re-read, not stored
#pragma unroll
    for (int h = 0; h < 8 / H; ++h) a[k][h] = ldg_nt<typename XT::raw, H>(at + h * H);
  }
  // A quantized tensor holds values of the grid only: the hardware converter gives their
  // codes, and converting back tells whether a value was one (bit for bit, so that -0.0 and
  // NaNs are told apart).  If any lane of the wavefront met another value, the wavefront goes
  // through the reference's nearest-value search instead (one branch for all its elements).
  uint32_t acc[U];
  bool off_grid = false;
#pragma unroll
  for (int k = 0; k < U; ++k) {
    float t[8], back[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) t[i] = XT::to_f32(a[k][i / H].v[i % H]);
    acc[k] = fp4_pack8_hw(t);
    fp4_unpack8_hw(acc[k], back);
#pragma unroll
    for (int i = 0; i < 8; ++i) off_grid |= f2u(back[i]) != f2u(t[i]);
  }
  if (__builtin_amdgcn_ballot_w64(off_grid) != 0) {
#pragma unroll
    for (int k = 0; k < U; ++k) {
      acc[k] = 0;
#pragma unroll
      for (int i = 0; i < 8; ++i)
        acc[k] |= (uint32_t)fp4_nearest_code<XT::id>(XT::to_f32(a[k][i / H].v[i % H])) << (4 * i);
    }
  }
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t v = v0 + k * 256;
    if (v < nvec) __builtin_nontemporal_store(acc[k], out + v);
  }
}

// one thread per output byte
__global__ void __launch_bounds__(256)
fp4_pack_kernel(const void* __restrict__ x, int x_dtype, uint8_t* __restrict__ out, int64_t nbytes) {
  for (int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; b < nbytes;
       b += (int64_t)gridDim.x * blockDim.x) {
    const int lo = fp4_nearest_code_rt(load_f32(x, x_dtype, 2 * b), x_dtype);
    const int hi = fp4_nearest_code_rt(load_f32(x, x_dtype, 2 * b + 1), x_dtype);
    out[b] = (uint8_t)(lo | (hi << 4));
  }
}

template <typename OT>
__global__ void __launch_bounds__(256)
fp4_unpack_vec_kernel(const uint32_t* __restrict__ in, typename OT::raw* __restrict__ out,
                      int64_t nvec) {
  constexpr int U = kFp4Vecs;
  constexpr int H = 16 / (int)sizeof(typename OT::raw);  // elements of a 16-byte store
  const int64_t v0 = (int64_t)blockIdx.x * (256 * U) + threadIdx.x;
  uint32_t w[U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t v = v0 + k * 256;
    w[k] = __builtin_nontemporal_load(in + (v < nvec ? v : nvec - 1));
  }
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int64_t v = v0 + k * 256;
    float f[8];
    fp4_unpack8_hw(w[k], f);
    const Vec<typename OT::raw, 8> o = pack8_from_f32<OT>(f);  // values of the grid, none a NaN
    if (v < nvec) {
#pragma unroll
      for (int h = 0; h < 8 / H; ++h) {
        Vec<typename OT::raw, H> part;
#pragma unroll
        for (int e = 0; e < H; ++e) part.v[e] = o.v[h * H + e];
        stg_nt<typename OT::raw, H>(out + v * 8 + h * H, part);
      }
    }
  }
}

__global__ void __launch_bounds__(256)
fp4_unpack_kernel(const uint8_t* __restrict__ in, void* __restrict__ out, int out_dtype,
                  int64_t nbytes) {
  for (int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; b < nbytes;
       b += (int64_t)gridDim.x * blockDim.x) {
    const int w = in[b];
    store_from_f32(out, out_dtype, 2 * b, fp4_decode(w & 15));
    store_from_f32(out, out_dtype, 2 * b + 1, fp4_decode(w >> 4));
  }
}

// ------------------------------------------------------------------ fused nvfp4, generic
struct Fp4Args {
  const void* x;
  void* out;
  const void* scale;
  const void* zp;
  const float* gscale;
  const int32_t* col_group;
  int64_t rows, cols;
  int64_t s_rows, s_cols, blk_rows, blk_cols;
  int x_dtype, out_dtype, scale_dtype, zp_dtype;
  QuantCfg q;
};

__device__ __forceinline__ float fp4_eff_scale(const Fp4Args& a, int64_t r, int64_t c,
                                               int64_t* si_out) {
  const int64_t srow = (r / a.blk_rows) % a.s_rows;
  const int64_t scol = a.col_group ? (int64_t)a.col_group[c] : c / a.blk_cols;
  const int64_t si = srow * a.s_cols + scol;
  *si_out = si;
  float s = load_f32(a.scale, a.scale_dtype, si);
  if (a.gscale) s = s / a.gscale[0];
  return s;
}

// The reference quantizes to e2m1 values held in x.dtype (forward.py:327 casts
// the group result back), then indexes them; a value on the grid survives that
// cast unchanged, so the code can be taken straight from the quantized value.
__device__ __forceinline__ int fp4_code_of_quantized(float v) {
  return fp4_bucket(fabsf(v)) | ((int)(f2u(v) >> 31) << 3);
}

__global__ void __launch_bounds__(256) nvfp4_compress_generic_kernel(Fp4Args a) {
  const int64_t hc = a.cols / 2;
  const int64_t total = a.rows * hc;
  for (int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; b < total;
       b += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = b / hc, j = b - r * hc;
    int code[2];
    for (int h = 0; h < 2; ++h) {
      const int64_t c = 2 * j + h;
      int64_t si;
      const float s = fp4_eff_scale(a, r, c, &si);
      const float z = a.zp ? round_to(load_f32(a.zp, a.zp_dtype, si), a.x_dtype) : 0.0f;
      const float v =
          quantize_value(load_f32(a.x, a.x_dtype, r * a.cols + c), s, z, a.zp != nullptr, a.q);
      code[h] = fp4_code_of_quantized(v);
    }
    ((uint8_t*)a.out)[b] = (uint8_t)(code[0] | (code[1] << 4));
  }
}

__global__ void __launch_bounds__(256) nvfp4_decompress_generic_kernel(Fp4Args a) {
  const int64_t hc = a.cols / 2;
  const int64_t total = a.rows * a.cols;
  for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < total;
       e += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = e / a.cols, c = e - r * a.cols;
    const int w = ((const uint8_t*)a.x)[r * hc + c / 2];
    const float qv = fp4_decode((c & 1) ? (w >> 4) : (w & 15));
    int64_t si;
    const float s = fp4_eff_scale(a, r, c, &si);
    store_from_f32(a.out, a.out_dtype, e, dequantize_value(qv, s, 0.0f, false, a.q.dt));
  }
}

// ------------------------------------------------------------------ fused nvfp4, vectorised
// fp8 e4m3 local scales + fp32 global scale; arithmetic in fp32 (bf16/fp16/fp32
// input divided by an fp32 scale promotes to fp32).  One workgroup per chunk,
// every load of a chunk issued before the first value is looked at; chunks that
// lie wholly inside the tensor run without per-lane bounds checks.
#ifndef CTMI_FP4_TUNING
#define CTMI_FP4_TUNING 512, 2
#endif
constexpr int kFp4Tuning[2] = {CTMI_FP4_TUNING};
constexpr int kFp4Block = kFp4Tuning[0], kFp4Unroll = kFp4Tuning[1];

// The reference's chain for 8 elements: x / s, + zp, clamp to +-6, cast_to_fp4
// (forward.py:471-482, quant_args.py:55-68), one exact division per element.
template <typename XT, bool HAS_ZP>
__device__ __forceinline__ uint32_t nvfp4_codes_exact(const Vec<typename XT::raw, 8>& xv, float s,
                                                      float z) {
  uint32_t acc = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    float t = XT::to_f32(xv.v[i]) / s;
    if (HAS_ZP) t = t + z;
    t = clamp_nan(t, -6.0f, 6.0f);
    // sign of cast_to_fp4's product: exact zeros lose their sign
    const uint32_t neg = (t < 0.0f) ? 8u : 0u;
    acc |= ((uint32_t)fp4_bucket(fabsf(t)) | neg) << (4 * i);
  }
  return acc;
}

// The effective scale of a group is fp32(fp8 code) / global_scale: only 256 values
// per weight.  A workgroup works them out once (the exact division, the reciprocal
// and whether the scale is in the range where the fast path holds) while its loads
// are in flight, and a group's arithmetic starts from one 16-byte LDS read instead
// of a division and a reciprocal.
struct alignas(16) Fp4Scale {
  float s;   // fp32(fp8 code) / global_scale, the exact quotient
  float r;   // rcp(s) for the fast path, or NaN where only the division is safe
  float y;   // rcp(s) after one Newton step: what an IEEE division multiplies by
  float pad;
};

__device__ __forceinline__ void build_scale_lut(Fp4Scale* lut, float gs) {
  const int t = threadIdx.x;
  if (t < 256) {
    const float s = __builtin_amdgcn_cvt_f32_fp8(t, 0) / gs;
    // below 2^12 a quotient of the smallest bfloat16 / float16 magnitude stays above
    // the addend of nvfp4_codes_fast; above 2^-60 the residuals of nvfp4_codes_divided
    // stay in the normal range for every input that can reach a code other than zero
    const bool tame = s >= 8.673617379884035e-19f && s < 4096.0f;
    const float y0 = __builtin_amdgcn_rcpf(s);
    Fp4Scale e;
    e.s = s;
    e.r = tame ? y0 : __uint_as_float(0x7fc00000u);
    e.y = __builtin_fmaf(__builtin_fmaf(-s, y0, 1.0f), y0, y0);
    e.pad = 0.0f;
    lut[t] = e;
  }
  __syncthreads();
}

// The codes of 8 elements without divisions and with ONE conversion per pair (the
// hardware's e2m1 converter is several times slower than an fma; converting a lower and
// an upper bracket of every quotient made it the bottleneck).
// q = x * rcp(s) is within 3 ulp of the reference's quotient x / s (rcp: 1 ulp, the
// product: 1/2, the reference's own rounding: 1/2, a tie broken by the addend: 1).
// Every rounding boundary of the e2m1 grid (0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5) has a
// significand of 1, 1.25, 1.5 or 1.75: its low 21 bits are zero.  So if the low 21 bits
// of q are not within 8 of zero (mod 2^21), no boundary lies between q and the exact
// quotient, both convert to the same code, and the converter's round-to-nearest-even
// is the reference's bucket rule.  Otherwise (8 values in a million, an infinity, a
// scale outside the tame range, whose reciprocal is a NaN with those bits zero, and
// whatever sits near a power of two) the wavefront redoes the vector with exact
// divisions.  The addend, 16 ulp of the smallest denormal, is absorbed by every
// quotient that matters; it keeps exact zeros (which have no bits set) out of the
// slow path and turns a -0 quotient into +0 as the reference's sign(0) = 0 does,
// while a negative quotient that rounds to zero keeps its sign (code 8).  A NaN
// element has no defined code in the reference (the sign of a NaN product); it gets
// whatever the converter gives and touches no other element.
// *ok is cleared when the codes returned may differ from the reference's; the caller
// then redoes the vector with nvfp4_codes_exact.  No branch in here, on purpose: a
// wave-level branch after every vector (skip the exact path if all lanes are fine)
// cost this kernel a fifth of its speed.  Callers store what the fast path gives for
// all their vectors, test once, and overwrite in the rare case.
template <typename XT>
__device__ __forceinline__ uint32_t nvfp4_codes_fast(const Vec<typename XT::raw, 8>& xv,
                                                     const Fp4Scale& e, bool* ok) {
  const float c0 = __uint_as_float(0x10u);
  float q[8];
  uint32_t nearest = 0xffffffffu;
#pragma unroll
  for (int i = 0; i < 8; i += 2) {
    const float x0 = XT::to_f32(xv.v[i]), x1 = XT::to_f32(xv.v[i + 1]);
    q[i] = __builtin_fmaf(x0, e.r, c0);
    q[i + 1] = __builtin_fmaf(x1, e.r, c0);
    // the low 21 bits, moved to the top, of the bit pattern + 8
    const uint32_t t0 = (__float_as_uint(q[i]) + 8u) << 11, t1 = (__float_as_uint(q[i + 1]) + 8u) << 11;
    nearest = min(nearest, min(t0, t1));
    if constexpr (XT::id == CTMI_F32) {
      // float32 inputs reach below the addend: a quotient in the denormal range that is
      // not the addend itself (x == 0) takes the exact path
      const uint32_t a0 = __float_as_uint(q[i]) & 0x7fffffffu, a1 = __float_as_uint(q[i + 1]) & 0x7fffffffu;
      if ((a0 < 0x00800000u && a0 != 0x10u) || (a1 < 0x00800000u && a1 != 0x10u)) nearest = 0;
    }
  }
  *ok &= nearest >= (16u << 11);
  return fp4_pack8_hw(q);
}

// Second tier, for the vectors the fast path is not sure of.  Weights of one tensor
// share few distinct quotient significands (a bfloat16 has 128, the scales of a tensor 8,
// and a global scale computed in bfloat16 has 8 bits itself), so quotients that ROUND to
// a boundary such as 1.25, or sit on a grid value such as 1.5, are systematic: in one
// tensor of three every wavefront meets one.  What settles them is the correctly rounded
// quotient, and that is five multiply-adds away: with y the Newton-refined reciprocal
// from the table,
//     q0 = x y;  q1 = q0 + (x - s q0) y;  q2 = q1 + (x - s q1) y
// is, instruction for instruction, what an IEEE float division x / s executes between
// its pre-scaling and its fix-up, and those two only act when the exponents of x and s
// lie 96 or more apart or an operand, a reciprocal or the quotient leaves the normal
// range.  So for a tame scale (2^-60 <= s < 2^12) and 2^-30 <= |x| < 2^30 (or x == 0)
// q2 is bit for bit the reference's x / s, at a third of the cost of the general
// division; anything else clears *ok and takes nvfp4_codes_exact.
__device__ __forceinline__ float nvfp4_quotient_divided(float x, const Fp4Scale& e, bool* fine) {
  const uint32_t mag = __float_as_uint(x) & 0x7fffffffu;
  *fine &= (mag - 0x30800000u) < (0x4e800000u - 0x30800000u) || mag == 0;
  const float q0 = x * e.y;
  const float q1 = __builtin_fmaf(__builtin_fmaf(-e.s, q0, x), e.y, q0);
  const float q2 = __builtin_fmaf(__builtin_fmaf(-e.s, q1, x), e.y, q1);
  return q2 + 0.0f;  // an exact zero loses its sign, as in the reference's sign(0) = 0
}

template <typename XT>
__device__ __forceinline__ uint32_t nvfp4_codes_divided(const Vec<typename XT::raw, 8>& xv,
                                                        const Fp4Scale& e, bool* ok) {
  float q[8];
  bool fine = e.r == e.r;  // a tame scale
#pragma unroll
  for (int i = 0; i < 8; ++i) q[i] = nvfp4_quotient_divided(XT::to_f32(xv.v[i]), e, &fine);
  *ok &= fine;
  return fp4_pack8_hw(q);
}

// Who does the second tier.  In a tensor whose quotients hit boundaries systematically
// three elements in two thousand are in doubt, but that is one or two in nearly every
// wavefront, and a wavefront that redoes all its vectors for them doubles its arithmetic.
// So the lanes that hold a doubtful vector put it into a queue of their wavefront in
// LDS, and the queue is worked through four lanes to a vector (a lane takes two elements
// and produces one byte of codes): sixteen vectors cost what one cost before.  The
// owners then take their four bytes back.  Nothing here leaves the wavefront: LDS
// instructions of one wavefront execute in order, so all it needs is that the compiler
// keeps the order as well.
constexpr int kFp4RedoCap = 32;  // vectors per wavefront; beyond that every lane redoes its own

template <typename XT>
struct Fp4Redo {
  Vec<typename XT::raw, 8> x[kFp4RedoCap];
  uint32_t sraw[kFp4RedoCap];
  uint32_t codes[kFp4RedoCap];
};

__device__ __forceinline__ void lds_in_order() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

// false: not done here (too many doubtful vectors, or one outside the range the
// division-free sequence covers); codes[] is then untouched or partly replaced by
// equally valid codes of vectors that were fine
template <typename XT, int U>
__device__ __forceinline__ bool nvfp4_redo_doubtful(const Vec<typename XT::raw, 8>* xv,
                                                    const uint8_t* sraw, const bool* okk,
                                                    uint32_t* codes, const Fp4Scale* lut,
                                                    Fp4Redo<XT>& q) {
  const uint32_t lane = threadIdx.x & 63u;
  uint32_t count = 0, slot[U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const uint64_t m = __builtin_amdgcn_ballot_w64(!okk[k]);
    slot[k] = count + __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
    count += (uint32_t)__builtin_popcountll(m);
  }
  if (count > (uint32_t)kFp4RedoCap) return false;
#pragma unroll
  for (int k = 0; k < U; ++k) {
    if (!okk[k]) {
      q.x[slot[k]] = xv[k];
      q.sraw[slot[k]] = sraw[k];
    }
  }
  lds_in_order();
  bool fine = true;
  for (uint32_t base = 0; base < count; base += 16) {
    const uint32_t e = base + (lane >> 2), pair = lane & 3u;
    if (e < count) {
      const Fp4Scale sc = lut[q.sraw[e]];
      fine &= sc.r == sc.r;
      const typename XT::raw* px = reinterpret_cast<const typename XT::raw*>(&q.x[e]) + 2 * pair;
      const float qa = nvfp4_quotient_divided(XT::to_f32(px[0]), sc, &fine);
      const float qb = nvfp4_quotient_divided(XT::to_f32(px[1]), sc, &fine);
      reinterpret_cast<uint8_t*>(&q.codes[e])[pair] =
          (uint8_t)__builtin_amdgcn_cvt_scalef32_pk_fp4_f32(0u, qa, qb, 1.0f, 0);
    }
  }
  lds_in_order();
  if (!wave_all(fine)) return false;
#pragma unroll
  for (int k = 0; k < U; ++k)
    if (!okk[k]) codes[k] = q.codes[slot[k]];
  return true;
}

// The codes of a wavefront's U vectors once the fast path has flagged some of them
// (okk[k] false): the queue above, else the division-free sequence for every vector,
// else exact divisions.
template <typename XT, int U>
__device__ __forceinline__ void nvfp4_settle_codes(const Vec<typename XT::raw, 8>* xv,
                                                   const uint8_t* sraw, const bool* okk,
                                                   uint32_t* codes, const Fp4Scale* lut,
                                                   Fp4Redo<XT>* redo) {
  if (nvfp4_redo_doubtful<XT, U>(xv, sraw, okk, codes, lut, redo[threadIdx.x >> 6])) return;
  bool ok = true;
#pragma unroll
  for (int k = 0; k < U; ++k) codes[k] = nvfp4_codes_divided<XT>(xv[k], lut[sraw[k]], &ok);
  if (wave_all(ok)) return;
#pragma unroll
  for (int k = 0; k < U; ++k) codes[k] = nvfp4_codes_exact<XT, false>(xv[k], lut[sraw[k]].s, 0.0f);
}

template <typename XT, bool HAS_ZP>
__global__ void __launch_bounds__(kFp4Block)
nvfp4_compress_vec_kernel(const typename XT::raw* __restrict__ x, const uint8_t* __restrict__ scale,
                          const uint8_t* __restrict__ zp, const float* __restrict__ gscale,
                          uint32_t* __restrict__ out, VecGeom g) {
  constexpr int B = kFp4Block, U = kFp4Unroll;
  __shared__ Fp4Scale lut[256];
  __shared__ Fp4Redo<XT> redo[B / 64];
  const float gs = gscale[0];
  const uint32_t v0 = blockIdx.x * (B * U) + threadIdx.x;
  const bool full = (blockIdx.x + 1) * (uint32_t)(B * U) <= g.nvec;
  auto body = [&](auto guard) {
    constexpr bool GUARD = decltype(guard)::value;
    uint32_t si[U];
#pragma unroll
    for (int k = 0; k < U; ++k) si[k] = scale_index(min(v0 + k * B, g.nvec - 1), g);
    Vec<typename XT::raw, 8> xv[U];
    uint8_t sraw[U], zraw[U];
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const uint32_t v = v0 + k * B;
      if (!GUARD || v < g.nvec) {
        xv[k] = ldg_nt<typename XT::raw, 8>(x + (size_t)v * 8);
        sraw[k] = scale[si[k]];
        if constexpr (HAS_ZP) zraw[k] = zp[si[k]];
      } else {
        xv[k] = {};
        sraw[k] = 0;
        if constexpr (HAS_ZP) zraw[k] = 0;
      }
    }
    build_scale_lut(lut, gs);
    bool okk[U], plain = true;
    uint32_t codes[U];
#pragma unroll
    for (int k = 0; k < U; ++k) {
      okk[k] = true;
      if (!GUARD || v0 + k * B < g.nvec) {
        // a zero point of zero (what symmetric schemes carry) only turns -0 into +0, which
        // the fast path does as well; any other takes the exact path
        if constexpr (HAS_ZP) plain &= (zraw[k] & 0x7f) == 0;
        codes[k] = nvfp4_codes_fast<XT>(xv[k], lut[sraw[k]], &okk[k]);
      }
    }
    bool ok = plain;
#pragma unroll
    for (int k = 0; k < U; ++k) ok &= okk[k];
    if (__builtin_expect(!wave_all(ok), 0)) {
      if (!HAS_ZP || wave_all(plain)) {
        nvfp4_settle_codes<XT, U>(xv, sraw, okk, codes, lut, redo);
      } else {
#pragma unroll
        for (int k = 0; k < U; ++k) {
          // zero_point.to(x.dtype): an fp8 value is exact in every wider float type
          const float z = HAS_ZP ? __builtin_amdgcn_cvt_f32_fp8((int)zraw[k], 0) : 0.0f;
          codes[k] = nvfp4_codes_exact<XT, HAS_ZP>(xv[k], lut[sraw[k]].s, z);
        }
      }
    }
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const uint32_t v = v0 + k * B;
      if (!GUARD || v < g.nvec) __builtin_nontemporal_store(codes[k], out + v);
    }
  };
  if (full) body(std::false_type{});
  else body(std::true_type{});
}

template <typename OT>
__global__ void __launch_bounds__(kFp4Block)
nvfp4_decompress_vec_kernel(const uint32_t* __restrict__ packed, const uint8_t* __restrict__ scale,
                            const float* __restrict__ gscale, typename OT::raw* __restrict__ out,
                            VecGeom g) {
  constexpr int B = kFp4Block, U = kFp4Unroll;
  __shared__ Fp4Scale lut[256];
  const float gs = gscale[0];
  const uint32_t v0 = blockIdx.x * (B * U) + threadIdx.x;
  const bool full = (blockIdx.x + 1) * (uint32_t)(B * U) <= g.nvec;
  auto body = [&](auto guard) {
    constexpr bool GUARD = decltype(guard)::value;
    uint32_t si[U];
#pragma unroll
    for (int k = 0; k < U; ++k) si[k] = scale_index(min(v0 + k * B, g.nvec - 1), g);
    uint32_t pv[U];
    uint8_t sraw[U];
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const uint32_t v = v0 + k * B;
      if (!GUARD || v < g.nvec) {
        pv[k] = packed[v];
        sraw[k] = scale[si[k]];
      } else {
        sraw[k] = 0;
      }
    }
    build_scale_lut(lut, gs);
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const uint32_t v = v0 + k * B;
      if (!GUARD || v < g.nvec) {
        const float s = lut[sraw[k]].s;
        float t[8];
        fp4_unpack8_hw(pv[k], t);
#pragma unroll
        for (int i = 0; i < 8; ++i) t[i] *= s;
        stg_nt<typename OT::raw, 8>(out + (size_t)v * 8, pack8_exact_from_f32<OT>(t));
      }
    }
  };
  if (full) body(std::false_type{});
  else body(std::true_type{});
}

// The two kernels above for up to kMaxJobs weights per launch (job_table.h), for
// scales numbered like the items (rows of whole groups, which is every nvfp4 weight
// the compressor sees).  A job's zero-point slot carries its global scale: the
// format is symmetric and stores no zero points.
template <typename XT>
__global__ void __launch_bounds__(kFp4Block) nvfp4_compress_chain_kernel(ChainTable t) {
  constexpr int B = kFp4Block, U = kFp4Unroll;
  uint32_t local, nvec;
  const ChainJob job = find_job(t, blockIdx.x, &local, &nvec);
  const auto* x = static_cast<const typename XT::raw*>(job.src);
  const auto* scale = static_cast<const uint8_t*>(job.scale);
  auto* out = static_cast<uint32_t*>(job.dst);
  const float gs = reinterpret_cast<const float*>(job.zp)[0];
  const uint32_t v0 = local * (B * U) + threadIdx.x;
  const bool full = (local + 1) * (uint32_t)(B * U) <= nvec;
  __shared__ Fp4Scale lut[256];
  __shared__ Fp4Redo<XT> redo[B / 64];
  auto body = [&](auto guard) {
    constexpr bool GUARD = decltype(guard)::value;
    Vec<typename XT::raw, 8> xv[U];
    uint8_t sraw[U];
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const uint32_t v = v0 + k * B;
      if (!GUARD || v < nvec) {
        xv[k] = ldg_nt<typename XT::raw, 8>(x + (size_t)v * 8);
        sraw[k] = scale[v >> job.shift];
      } else {
        xv[k] = {};
        sraw[k] = 0;
      }
    }
    build_scale_lut(lut, gs);
    bool okk[U], ok = true;
    uint32_t codes[U];
#pragma unroll
    for (int k = 0; k < U; ++k) {
      okk[k] = true;
      if (!GUARD || v0 + k * B < nvec) codes[k] = nvfp4_codes_fast<XT>(xv[k], lut[sraw[k]], &okk[k]);
      ok &= okk[k];
    }
    if (__builtin_expect(!wave_all(ok), 0)) nvfp4_settle_codes<XT, U>(xv, sraw, okk, codes, lut, redo);
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const uint32_t v = v0 + k * B;
      if (!GUARD || v < nvec) __builtin_nontemporal_store(codes[k], out + v);
    }
  };
  if (full) body(std::false_type{});
  else body(std::true_type{});
}

template <typename OT>
__global__ void __launch_bounds__(kFp4Block) nvfp4_decompress_chain_kernel(ChainTable t) {
  constexpr int B = kFp4Block, U = kFp4Unroll;
  uint32_t local, nvec;
  const ChainJob job = find_job(t, blockIdx.x, &local, &nvec);
  const auto* packed = static_cast<const uint32_t*>(job.src);
  const auto* scale = static_cast<const uint8_t*>(job.scale);
  auto* out = static_cast<typename OT::raw*>(job.dst);
  const float gs = reinterpret_cast<const float*>(job.zp)[0];
  const uint32_t v0 = local * (B * U) + threadIdx.x;
  const bool full = (local + 1) * (uint32_t)(B * U) <= nvec;
  __shared__ Fp4Scale lut[256];
  auto body = [&](auto guard) {
    constexpr bool GUARD = decltype(guard)::value;
    uint32_t pv[U];
    uint8_t sraw[U];
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const uint32_t v = v0 + k * B;
      if (!GUARD || v < nvec) {
        pv[k] = packed[v];
        sraw[k] = scale[v >> job.shift];
      } else {
        sraw[k] = 0;
      }
    }
    build_scale_lut(lut, gs);
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const uint32_t v = v0 + k * B;
      if (!GUARD || v < nvec) {
        const float s = lut[sraw[k]].s;
        float f[8];
        fp4_unpack8_hw(pv[k], f);
#pragma unroll
        for (int i = 0; i < 8; ++i) f[i] *= s;
        stg_nt<typename OT::raw, 8>(out + (size_t)v * 8, pack8_exact_from_f32<OT>(f));
      }
    }
  };
  if (full) body(std::false_type{});
  else body(std::true_type{});
}

// quantize + dequantize in one pass (fake_quantize of forward.py:150-189 for the
// nvfp4 scheme): out = XT(e2m1(x / s) * s), s = fp32(scale) / global_scale
// (fake-quantize moves 4 bytes per element: one item per lane in flight is enough)
constexpr int kFp4QdqBlock = 256, kFp4QdqUnroll = 1;
template <typename XT>
__global__ void __launch_bounds__(kFp4QdqBlock)
nvfp4_qdq_vec_kernel(const typename XT::raw* __restrict__ x, const uint8_t* __restrict__ scale,
                     const float* __restrict__ gscale, typename XT::raw* __restrict__ out,
                     VecGeom g) {
  constexpr int B = kFp4QdqBlock, U = kFp4QdqUnroll;
  static_assert(B >= 256, "the scale table is built by 256 threads");
  __shared__ Fp4Scale lut[256];
  __shared__ Fp4Redo<XT> redo[B / 64];
  const float gs = gscale[0];
  const uint32_t v0 = blockIdx.x * (B * U) + threadIdx.x;
  const bool full = (blockIdx.x + 1) * (uint32_t)(B * U) <= g.nvec;
  auto body = [&](auto guard) {
    constexpr bool GUARD = decltype(guard)::value;
    uint32_t si[U];
#pragma unroll
    for (int k = 0; k < U; ++k) si[k] = scale_index(min(v0 + k * B, g.nvec - 1), g);
    Vec<typename XT::raw, 8> xv[U];
    uint8_t sraw[U];
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const uint32_t v = v0 + k * B;
      if (!GUARD || v < g.nvec) {
        xv[k] = ldg_nt<typename XT::raw, 8>(x + (size_t)v * 8);
        sraw[k] = scale[si[k]];
      } else {
        xv[k] = {};
        sraw[k] = 0;
      }
    }
    build_scale_lut(lut, gs);
    auto emit = [&](int k, uint32_t codes, float s) {
      float t[8];
      fp4_unpack8_hw(codes, t);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float xi = XT::to_f32(xv[k].v[i]);
        t[i] = xi != xi ? xi : t[i] * s;  // a NaN stays one (no code stands for it)
      }
      stg_nt<typename XT::raw, 8>(out + (size_t)(v0 + k * B) * 8, pack8_exact_from_f32<XT>(t));
    };
    bool okk[U], ok = true;
    uint32_t codes[U];
#pragma unroll
    for (int k = 0; k < U; ++k) {
      okk[k] = true;
      if (!GUARD || v0 + k * B < g.nvec) codes[k] = nvfp4_codes_fast<XT>(xv[k], lut[sraw[k]], &okk[k]);
      ok &= okk[k];
    }
    if (__builtin_expect(!wave_all(ok), 0)) nvfp4_settle_codes<XT, U>(xv, sraw, okk, codes, lut, redo);
#pragma unroll
    for (int k = 0; k < U; ++k)
      if (!GUARD || v0 + k * B < g.nvec) emit(k, codes[k], lut[sraw[k]].s);
  };
  if (full) body(std::false_type{});
  else body(std::true_type{});
}

// fake-quantize entry for ctmi_qdq; false = not this kernel's case, nothing launched
bool nvfp4_qdq_try_vectorised(const void* x, int x_dtype, void* out, int out_dtype, int64_t rows,
                              int64_t cols, const ctmi_qparams* qp, hipStream_t st) {
  if (qp->qtype != CTMI_QTYPE_FLOAT || qp->num_bits != 4 || !qp->global_scale ||
      qp->scale_dtype != CTMI_F8E4M3 || qp->zero_point || x_dtype != out_dtype)
    return false;
  if (x_dtype != CTMI_BF16 && x_dtype != CTMI_F16 && x_dtype != CTMI_F32) return false;
  const int bytes = 8 * dtype_size(x_dtype);
  if ((uintptr_t)x % bytes || (uintptr_t)out % bytes) return false;
  VecGeom g;
  if (!vec_geometry(qp, rows, cols, &g, true)) return false;
  const int64_t grid = cdiv(g.nvec, kFp4QdqBlock * kFp4QdqUnroll);
  const auto* sc = (const uint8_t*)qp->scale;
  if (x_dtype == CTMI_BF16) hipLaunchKernelGGL(nvfp4_qdq_vec_kernel<BF16>, (unsigned)grid, kFp4QdqBlock, 0, st, (const uint16_t*)x, sc, qp->global_scale, (uint16_t*)out, g);
  else if (x_dtype == CTMI_F16) hipLaunchKernelGGL(nvfp4_qdq_vec_kernel<F16>, (unsigned)grid, kFp4QdqBlock, 0, st, (const uint16_t*)x, sc, qp->global_scale, (uint16_t*)out, g);
  else hipLaunchKernelGGL(nvfp4_qdq_vec_kernel<F32>, (unsigned)grid, kFp4QdqBlock, 0, st, (const float*)x, sc, qp->global_scale, (float*)out, g);
  return true;
}

// calculate_qparams (helpers.py:67-146) for one group of an fp4 scheme with a
// global scale, min / max in XT: scale = fp8(clamp(gs * XT(max|x| / 6), +-448)),
// zero replaced by 0.125.  Returns the fp8 code, *sv = its value.
template <typename XT>
__device__ __forceinline__ uint8_t nvfp4_group_scale(float absmax, bool has_nan, float gs,
                                                     float* sv) {
  float t;
  if constexpr (XT::id == CTMI_BF16) {
    // bf16 / bf16 (6 is a bf16 value): the product with the reciprocal rounds to
    // the same bf16 as the quotient
    t = absmax * 0.16666667163372039794921875f;
  } else {
    t = absmax / 6.0f;
  }
  float s = gs * round_xt<XT>(t);
  has_nan |= s != s;  // inf * 0
  s = __builtin_fminf(__builtin_fmaxf(s, -448.0f), 448.0f);
  uint32_t code = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(s, s, 0, false) & 0xffu;
  float value = __builtin_amdgcn_cvt_f32_fp8((int)code, 0);
  if (value == 0.0f) {
    code = 0x20u;  // 0.125
    value = 0.125f;
  }
  if (has_nan) {
    code = 0x7fu;
    value = __builtin_nanf("");
  }
  *sv = value;
  return (uint8_t)code;
}

// Dynamic nvfp4 activations (forward.py:414-451 with a tensor_group scheme): the
// group scales come from the 16 elements themselves (helpers.py:149-205, :67-146),
// which are then fake-quantized with them without leaving the registers.  Two
// neighbouring lanes hold one group.
template <typename XT>
__global__ void __launch_bounds__(kFp4Block)
nvfp4_dynamic_kernel(const typename XT::raw* __restrict__ x, const float* __restrict__ gscale,
                     typename XT::raw* __restrict__ out, uint8_t* __restrict__ scale_out,
                     uint8_t* __restrict__ zp_out, uint32_t nvec) {
  constexpr int B = kFp4Block, U = 2;
  __shared__ Fp4Scale lut[256];
  __shared__ Fp4Redo<XT> redo[B / 64];
  const float gs = gscale[0];
  const uint32_t v0 = blockIdx.x * (B * U) + threadIdx.x;
  Vec<typename XT::raw, 8> xv[U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const uint32_t v = v0 + k * B;
    xv[k] = ldg_nt<typename XT::raw, 8>(x + (size_t)(v < nvec ? v : nvec - 1) * 8);
  }
  build_scale_lut(lut, gs);
  auto emit = [&](int k, uint32_t c, float s) {
    const uint32_t v = v0 + k * B;
    float t[8];
    fp4_unpack8_hw(c, t);
#pragma unroll
    for (int i = 0; i < 8; ++i) t[i] *= s;  // a NaN in the group made s NaN
    if (v < nvec) stg_nt<typename XT::raw, 8>(out + (size_t)v * 8, pack8_exact_from_f32<XT>(t));
  };
  bool okk[U], ok = true;
  uint8_t sraw[U];
  uint32_t codes[U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const uint32_t v = v0 + k * B;
    float sv;
    uint8_t code;
    if constexpr (sizeof(typename XT::raw) == 2) {
      const uint32_t m = group_umax(2, absmax8_bits<XT>(xv[k]));
      constexpr uint32_t kInf = XT::id == CTMI_BF16 ? 0x7f80u : 0x7c00u;
      code = nvfp4_group_scale<XT>(XT::to_f32((typename XT::raw)m), m > kInf, gs, &sv);
    } else {
      float lo = __builtin_inff(), hi = -__builtin_inff();
      bool unordered = false;
      vec_minmax<XT>(xv[k], &lo, &hi, &unordered);
      group_minmax(2, &lo, &hi);
      // max(|min(lo, 0)|, |max(hi, 0)|)
      code = nvfp4_group_scale<XT>(__builtin_fmaxf(__builtin_fmaxf(-lo, hi), 0.0f),
                                   group_any(2, unordered), gs, &sv);
    }
    if (v < nvec && (threadIdx.x & 1) == 0) {
      if (scale_out) scale_out[v >> 1] = code;
      if (zp_out) zp_out[v >> 1] = 0;  // fp8 zero
    }
    sraw[k] = code;
    okk[k] = true;
    codes[k] = nvfp4_codes_fast<XT>(xv[k], lut[code], &okk[k]);
    ok &= okk[k];
  }
  if (__builtin_expect(!wave_all(ok), 0)) nvfp4_settle_codes<XT, U>(xv, sraw, okk, codes, lut, redo);
#pragma unroll
  for (int k = 0; k < U; ++k) emit(k, codes[k], lut[sraw[k]].s);
}

// One-shot nvfp4 compression of a weight whose global scale is known: group scales
// (min-max observer + calculate_qparams, tests/mock_observer.py:38-113,
// helpers.py:101-120) and NVFP4PackedCompressor.compress_weight
// (fp4_quantized.py:84-107) with those scales and their all-zero zero points, the
// weight read once.
constexpr int kFp4ObserveU = 2;

template <typename XT>
__device__ __forceinline__ void nvfp4_observe_compress_chunk(const typename XT::raw* __restrict__ x,
                                                             float gs, uint32_t* __restrict__ packed,
                                                             uint8_t* __restrict__ scale_out,
                                                             uint32_t nvec, uint32_t chunk,
                                                             Fp4Scale* lut, Fp4Redo<XT>* redo) {
  constexpr int B = kFp4Block, U = kFp4ObserveU;
  const uint32_t v0 = chunk * (B * U) + threadIdx.x;
  Vec<typename XT::raw, 8> xv[U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const uint32_t v = v0 + k * B;
    xv[k] = ldg_nt<typename XT::raw, 8>(x + (size_t)(v < nvec ? v : nvec - 1) * 8);
  }
  build_scale_lut(lut, gs);
  bool okk[U], ok = true;
  uint8_t sraw[U];
  uint32_t codes[U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const uint32_t v = v0 + k * B;
    float sv;
    uint8_t code;
    if constexpr (sizeof(typename XT::raw) == 2) {
      const uint32_t m = group_umax(2, absmax8_bits<XT>(xv[k]));
      constexpr uint32_t kInf = XT::id == CTMI_BF16 ? 0x7f80u : 0x7c00u;
      code = nvfp4_group_scale<XT>(XT::to_f32((typename XT::raw)m), m > kInf, gs, &sv);
    } else {
      float lo = __builtin_inff(), hi = -__builtin_inff();
      bool unordered = false;
      vec_minmax<XT>(xv[k], &lo, &hi, &unordered);
      group_minmax(2, &lo, &hi);
      code = nvfp4_group_scale<XT>(__builtin_fmaxf(__builtin_fmaxf(-lo, hi), 0.0f),
                                   group_any(2, unordered), gs, &sv);
    }
    sraw[k] = code;
    okk[k] = true;
    codes[k] = nvfp4_codes_fast<XT>(xv[k], lut[code], &okk[k]);
    ok &= okk[k];
    if (v < nvec && (threadIdx.x & 1) == 0) scale_out[v >> 1] = code;
  }
  if (__builtin_expect(!wave_all(ok), 0)) nvfp4_settle_codes<XT, U>(xv, sraw, okk, codes, lut, redo);
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const uint32_t v = v0 + k * B;
    if (v < nvec) __builtin_nontemporal_store(codes[k], packed + v);
  }
}

template <typename XT>
__global__ void __launch_bounds__(kFp4Block)
nvfp4_observe_compress_kernel(const typename XT::raw* __restrict__ x,
                              const float* __restrict__ gscale, uint32_t* __restrict__ packed,
                              uint8_t* __restrict__ scale_out, uint32_t nvec) {
  __shared__ Fp4Scale lut[256];
  __shared__ Fp4Redo<XT> redo[kFp4Block / 64];
  nvfp4_observe_compress_chunk<XT>(x, gscale[0], packed, scale_out, nvec, blockIdx.x, lut, redo);
}

// ... for up to kMaxJobs weights per launch: job.scale is written, the zero-point slot
// carries the global scale (as in nvfp4_compress_chain_kernel)
template <typename XT>
__global__ void __launch_bounds__(kFp4Block) nvfp4_observe_compress_chain_kernel(ChainTable t) {
  __shared__ Fp4Scale lut[256];
  __shared__ Fp4Redo<XT> redo[kFp4Block / 64];
  uint32_t local, nvec;
  const ChainJob job = find_job(t, blockIdx.x, &local, &nvec);
  nvfp4_observe_compress_chunk<XT>(static_cast<const typename XT::raw*>(job.src),
                                   reinterpret_cast<const float*>(job.zp)[0],
                                   static_cast<uint32_t*>(job.dst),
                                   static_cast<uint8_t*>(const_cast<void*>(job.scale)), nvec, local, lut, redo);
}

// The observer on its own for the same scheme (tests/mock_observer.py:38-113 +
// helpers.py:101-120): group-16 fp8 scales (and their all-zero zero points) of a 16-bit
// tensor, with the arithmetic of the fused kernels above (absmax on the raw bits, one
// scale per pair of lanes) instead of the general min / max observer.
template <typename XT>
__global__ void __launch_bounds__(kFp4Block)
nvfp4_observe_kernel(const typename XT::raw* __restrict__ x, const float* __restrict__ gscale,
                     uint8_t* __restrict__ scale_out, uint8_t* __restrict__ zp_out, uint32_t nvec) {
  static_assert(sizeof(typename XT::raw) == 2, "16-bit inputs");
  constexpr int B = kFp4Block, U = 4;
  const float gs = gscale[0];
  const uint32_t v0 = blockIdx.x * (B * U) + threadIdx.x;
  Vec<typename XT::raw, 8> xv[U];
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const uint32_t v = v0 + k * B;
    xv[k] = ldg_nt<typename XT::raw, 8>(x + (size_t)(v < nvec ? v : nvec - 1) * 8);
  }
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const uint32_t v = v0 + k * B;
    const uint32_t m = group_umax(2, absmax8_bits<XT>(xv[k]));
    constexpr uint32_t kInf = XT::id == CTMI_BF16 ? 0x7f80u : 0x7c00u;
    float sv;
    const uint8_t code = nvfp4_group_scale<XT>(XT::to_f32((typename XT::raw)m), m > kInf, gs, &sv);
    if (v < nvec && (threadIdx.x & 1) == 0) {
      scale_out[v >> 1] = code;
      if (zp_out) zp_out[v >> 1] = 0;  // fp8 zero
    }
  }
}

// scales-only entry for ctmi_observe_qparams; false = not this kernel's case
bool nvfp4_observe_try(const void* x, int x_dtype, int64_t rows, int64_t cols, int64_t blk_cols,
                       const float* gscale, void* scale_out, void* zp_out, const QpCfg& c,
                       hipStream_t st) {
  if (!gscale || blk_cols != 16 || cols % 16 || !c.fp4_global || (uintptr_t)x % 16) return false;
  if (x_dtype != CTMI_BF16 && x_dtype != CTMI_F16) return false;
  const int64_t nvec = rows * cols / 8;
  const int64_t grid = cdiv(nvec, kFp4Block * 4);
  if (nvec >= (1ll << 32) || grid >= (1ll << 31)) return false;
  auto* so = (uint8_t*)scale_out;
  auto* zo = (uint8_t*)zp_out;
  if (x_dtype == CTMI_BF16) hipLaunchKernelGGL(nvfp4_observe_kernel<BF16>, (unsigned)grid, kFp4Block, 0, st, (const uint16_t*)x, gscale, so, zo, (uint32_t)nvec);
  else hipLaunchKernelGGL(nvfp4_observe_kernel<F16>, (unsigned)grid, kFp4Block, 0, st, (const uint16_t*)x, gscale, so, zo, (uint32_t)nvec);
  return true;
}

bool nvfp4_dynamic_try(const void* x, int x_dtype, void* out, int64_t rows, int64_t cols,
                       int64_t blk_cols, const float* gscale, void* scale_out, void* zp_out,
                       const QpCfg& c, hipStream_t st) {
  if (!gscale || blk_cols != 16 || cols % 16 || !c.fp4_global) return false;
  const int64_t nvec = rows * cols / 8;
  const int64_t grid = cdiv(nvec, kFp4Block * 2);
  if (nvec >= (1ll << 32) || grid >= (1ll << 31)) return false;
  auto* so = (uint8_t*)scale_out;
  auto* zo = (uint8_t*)zp_out;
  if (x_dtype == CTMI_BF16) hipLaunchKernelGGL(nvfp4_dynamic_kernel<BF16>, (unsigned)grid, kFp4Block, 0, st, (const uint16_t*)x, gscale, (uint16_t*)out, so, zo, (uint32_t)nvec);
  else if (x_dtype == CTMI_F16) hipLaunchKernelGGL(nvfp4_dynamic_kernel<F16>, (unsigned)grid, kFp4Block, 0, st, (const uint16_t*)x, gscale, (uint16_t*)out, so, zo, (uint32_t)nvec);
  else if (x_dtype == CTMI_F32) hipLaunchKernelGGL(nvfp4_dynamic_kernel<F32>, (unsigned)grid, kFp4Block, 0, st, (const float*)x, gscale, (float*)out, so, zo, (uint32_t)nvec);
  else return false;
  return true;
}

static int fill_fp4(Fp4Args* a, const ctmi_qparams* qp, int64_t rows, int64_t cols) {
  a->scale = qp->scale;
  a->zp = qp->zero_point;
  a->gscale = qp->global_scale;
  a->col_group = qp->col_group;
  a->rows = rows;
  a->cols = cols;
  a->s_rows = qp->s_rows;
  a->s_cols = qp->s_cols;
  a->blk_rows = qp->blk_rows;
  a->blk_cols = qp->blk_cols;
  a->scale_dtype = qp->scale_dtype;
  a->zp_dtype = qp->zp_dtype;
  a->q.qtype = CTMI_QTYPE_FLOAT;
  a->q.num_bits = 4;
  a->q.qmin = -6.0f;
  a->q.qmax = 6.0f;
  a->q.dt = qp->global_scale ? CTMI_F32 : qp->scale_dtype;
  return CTMI_OK;
}

}  // namespace ctmi

using namespace ctmi;

static int check_float3(int dtype, const char* what) {
  CTMI_REQUIRE(dtype == CTMI_F32 || dtype == CTMI_F16 || dtype == CTMI_BF16, CTMI_ERR_UNSUPPORTED,
               "%s must be float16/bfloat16/float32", what);
  return CTMI_OK;
}

extern "C" int ctmi_pack_fp4_to_uint8(const void* x, int32_t x_dtype, uint8_t* out, int64_t rows,
                                      int64_t cols, void* stream) {
  CTMI_REQUIRE(rows >= 0 && cols >= 0, CTMI_ERR_VALUE, "negative shape");
  CTMI_REQUIRE(cols % 2 == 0, CTMI_ERR_VALUE,
               "tensor must have an even number of columns for nvfp4 compression");
  int rc = check_float3(x_dtype, "fp4 input");
  if (rc) return rc;
  if (rows == 0 || cols == 0) return CTMI_OK;
  CTMI_REQUIRE(x && out, CTMI_ERR_VALUE, "NULL tensor pointer");
  hipStream_t st = (hipStream_t)stream;
  const int64_t n = rows * cols;
  if (n % 8 == 0 && (uintptr_t)x % (8 * dtype_size(x_dtype)) == 0 && (uintptr_t)out % 4 == 0) {
    const int64_t nvec = n / 8;
    const unsigned grid = (unsigned)cdiv(nvec, 256 * kFp4Vecs);
    if (x_dtype == CTMI_BF16) hipLaunchKernelGGL(fp4_pack_vec_kernel<BF16>, grid, 256, 0, st, (const uint16_t*)x, (uint32_t*)out, nvec);
    else if (x_dtype == CTMI_F16) hipLaunchKernelGGL(fp4_pack_vec_kernel<F16>, grid, 256, 0, st, (const uint16_t*)x, (uint32_t*)out, nvec);
    else hipLaunchKernelGGL(fp4_pack_vec_kernel<F32>, grid, 256, 0, st, (const float*)x, (uint32_t*)out, nvec);
  } else {
    hipLaunchKernelGGL(fp4_pack_kernel, grid_for(n / 2, 256), 256, 0, st, x, x_dtype, out, n / 2);
  }
  return check_launch("ctmi_pack_fp4_to_uint8");
}

extern "C" int ctmi_unpack_fp4_from_uint8(const uint8_t* in, void* out, int32_t out_dtype,
                                          int64_t rows, int64_t cols, void* stream) {
  CTMI_REQUIRE(rows >= 0 && cols >= 0, CTMI_ERR_VALUE, "negative shape");
  CTMI_REQUIRE(cols % 2 == 0, CTMI_ERR_VALUE, "unpacked fp4 column count must be even");
  int rc = check_float3(out_dtype, "fp4 output");
  if (rc) return rc;
  if (rows == 0 || cols == 0) return CTMI_OK;
  CTMI_REQUIRE(in && out, CTMI_ERR_VALUE, "NULL tensor pointer");
  hipStream_t st = (hipStream_t)stream;
  const int64_t n = rows * cols;
  if (n % 8 == 0 && (uintptr_t)out % (8 * dtype_size(out_dtype)) == 0 && (uintptr_t)in % 4 == 0) {
    const int64_t nvec = n / 8;
    const unsigned grid = (unsigned)cdiv(nvec, 256 * kFp4Vecs);
    if (out_dtype == CTMI_BF16) hipLaunchKernelGGL(fp4_unpack_vec_kernel<BF16>, grid, 256, 0, st, (const uint32_t*)in, (uint16_t*)out, nvec);
    else if (out_dtype == CTMI_F16) hipLaunchKernelGGL(fp4_unpack_vec_kernel<F16>, grid, 256, 0, st, (const uint32_t*)in, (uint16_t*)out, nvec);
    else hipLaunchKernelGGL(fp4_unpack_vec_kernel<F32>, grid, 256, 0, st, (const uint32_t*)in, (float*)out, nvec);
  } else {
    hipLaunchKernelGGL(fp4_unpack_kernel, grid_for(n / 2, 256), 256, 0, st, in, out, out_dtype, n / 2);
  }
  return check_launch("ctmi_unpack_fp4_from_uint8");
}

extern "C" int ctmi_nvfp4_compress(const void* x, int32_t x_dtype, uint8_t* out, int64_t rows,
                                   int64_t cols, const ctmi_qparams* qp, void* stream) {
  CTMI_REQUIRE(rows >= 0 && cols >= 0, CTMI_ERR_VALUE, "negative shape");
  int rc = check_float3(x_dtype, "quantize input");
  if (rc) return rc;
  rc = check_qparams(qp, rows, cols);
  if (rc) return rc;
  CTMI_REQUIRE(qp->qtype == CTMI_QTYPE_FLOAT && qp->num_bits == 4, CTMI_ERR_VALUE,
               "nvfp4 compression needs float 4-bit quantization args");
  CTMI_REQUIRE(cols % 2 == 0, CTMI_ERR_VALUE,
               "tensor must have an even number of columns for nvfp4 compression");
  if (rows == 0 || cols == 0) return CTMI_OK;
  CTMI_REQUIRE(x && out, CTMI_ERR_VALUE, "NULL tensor pointer");
  hipStream_t st = (hipStream_t)stream;

  VecGeom g;
  const bool zp_ok = qp->zero_point == nullptr || qp->zp_dtype == CTMI_F8E4M3;
  if (qp->scale_dtype == CTMI_F8E4M3 && qp->global_scale && zp_ok &&
      (uintptr_t)x % (8 * dtype_size(x_dtype)) == 0 && (uintptr_t)out % 4 == 0 &&
      vec_geometry(qp, rows, cols, &g, true)) {
    const unsigned grid = (unsigned)cdiv(g.nvec, kFp4Block * kFp4Unroll);
    const auto* sc = (const uint8_t*)qp->scale;
    const auto* zp = (const uint8_t*)qp->zero_point;
#define CTMI_LAUNCH(XT, RAW)                                                                      \
  if (zp) hipLaunchKernelGGL((nvfp4_compress_vec_kernel<XT, true>), grid, kFp4Block, 0, st, (const RAW*)x, sc, zp, qp->global_scale, (uint32_t*)out, g); \
  else hipLaunchKernelGGL((nvfp4_compress_vec_kernel<XT, false>), grid, kFp4Block, 0, st, (const RAW*)x, sc, zp, qp->global_scale, (uint32_t*)out, g);
    if (x_dtype == CTMI_BF16) { CTMI_LAUNCH(BF16, uint16_t) }
    else if (x_dtype == CTMI_F16) { CTMI_LAUNCH(F16, uint16_t) }
    else { CTMI_LAUNCH(F32, float) }
#undef CTMI_LAUNCH
    return check_launch("ctmi_nvfp4_compress");
  }

  Fp4Args a;
  fill_fp4(&a, qp, rows, cols);
  a.x = x;
  a.out = out;
  a.x_dtype = x_dtype;
  a.out_dtype = CTMI_U8;
  a.q.ct = promote_float(x_dtype, a.q.dt);
  hipLaunchKernelGGL(nvfp4_compress_generic_kernel, grid_for(rows * cols / 2, 256), 256, 0, st, a);
  return check_launch("ctmi_nvfp4_compress");
}

extern "C" int ctmi_nvfp4_decompress(const uint8_t* packed, void* out, int32_t out_dtype,
                                     int64_t rows, int64_t cols, const ctmi_qparams* qp,
                                     void* stream) {
  CTMI_REQUIRE(rows >= 0 && cols >= 0, CTMI_ERR_VALUE, "negative shape");
  int rc = check_float3(out_dtype, "dequantize output");
  if (rc) return rc;
  rc = check_qparams(qp, rows, cols);
  if (rc) return rc;
  CTMI_REQUIRE(cols % 2 == 0, CTMI_ERR_VALUE, "unpacked fp4 column count must be even");
  if (rows == 0 || cols == 0) return CTMI_OK;
  CTMI_REQUIRE(packed && out, CTMI_ERR_VALUE, "NULL tensor pointer");
  hipStream_t st = (hipStream_t)stream;

  VecGeom g;
  if (qp->scale_dtype == CTMI_F8E4M3 && qp->global_scale && qp->zero_point == nullptr &&
      (uintptr_t)out % (8 * dtype_size(out_dtype)) == 0 && (uintptr_t)packed % 4 == 0 &&
      vec_geometry(qp, rows, cols, &g, true)) {
    const unsigned grid = (unsigned)cdiv(g.nvec, kFp4Block * kFp4Unroll);
    const auto* sc = (const uint8_t*)qp->scale;
    if (out_dtype == CTMI_BF16) hipLaunchKernelGGL(nvfp4_decompress_vec_kernel<BF16>, grid, kFp4Block, 0, st, (const uint32_t*)packed, sc, qp->global_scale, (uint16_t*)out, g);
    else if (out_dtype == CTMI_F16) hipLaunchKernelGGL(nvfp4_decompress_vec_kernel<F16>, grid, kFp4Block, 0, st, (const uint32_t*)packed, sc, qp->global_scale, (uint16_t*)out, g);
    else hipLaunchKernelGGL(nvfp4_decompress_vec_kernel<F32>, grid, kFp4Block, 0, st, (const uint32_t*)packed, sc, qp->global_scale, (float*)out, g);
    return check_launch("ctmi_nvfp4_decompress");
  }

  Fp4Args a;
  fill_fp4(&a, qp, rows, cols);
  a.x = packed;
  a.out = out;
  a.x_dtype = CTMI_U8;
  a.out_dtype = out_dtype;
  a.q.ct = a.q.dt;
  hipLaunchKernelGGL(nvfp4_decompress_generic_kernel, grid_for(rows * cols, 256), 256, 0, st, a);
  return check_launch("ctmi_nvfp4_decompress");
}

// Can this weight go into a chained launch?  (the fast path of the single-call entry
// points, with scales numbered like the items and no zero point)
static bool fp4_chainable(const ctmi_weight_job& j, bool compress, VecGeom* g) {
  const ctmi_qparams* qp = &j.qp;
  const uintptr_t dense = (uintptr_t)(compress ? j.src : j.dst);
  const uintptr_t packed = (uintptr_t)(compress ? j.dst : j.src);
  return j.rows > 0 && j.cols > 0 && qp->scale_dtype == CTMI_F8E4M3 && qp->global_scale &&
         qp->zero_point == nullptr && dense % (8 * dtype_size(j.dense_dtype)) == 0 &&
         packed % 4 == 0 && vec_geometry(qp, j.rows, j.cols, g, true) && flat_geometry(*g);
}

static int fp4_many(const ctmi_weight_job* jobs, int64_t n, bool compress, void* stream,
                    const char* what) {
  CTMI_REQUIRE(n >= 0 && (jobs || n == 0), CTMI_ERR_VALUE, "bad job list");
  if (n == 0) return CTMI_OK;
  hipStream_t st = (hipStream_t)stream;
  constexpr uint32_t per = kFp4Block * kFp4Unroll;
  // validate everything before anything is enqueued
  for (int64_t i = 0; i < n; ++i) {
    const ctmi_weight_job& j = jobs[i];
    CTMI_REQUIRE(j.rows >= 0 && j.cols >= 0, CTMI_ERR_VALUE, "job %lld: negative shape", (long long)i);
    int rc = check_float3(j.dense_dtype, "dense side");
    if (rc) return rc;
    rc = check_qparams(&j.qp, j.rows, j.cols);
    if (rc) return rc;
    CTMI_REQUIRE(j.cols % 2 == 0, CTMI_ERR_VALUE,
                 "tensor must have an even number of columns for nvfp4 compression");
    CTMI_REQUIRE(!compress || (j.qp.qtype == CTMI_QTYPE_FLOAT && j.qp.num_bits == 4), CTMI_ERR_VALUE,
                 "nvfp4 compression needs float 4-bit quantization args");
    CTMI_REQUIRE((j.src && j.dst) || j.rows == 0 || j.cols == 0, CTMI_ERR_VALUE,
                 "job %lld: NULL tensor pointer", (long long)i);
  }
  // chain per dense dtype, kMaxJobs weights per launch; the rest one call each
  const int dts[3] = {CTMI_BF16, CTMI_F16, CTMI_F32};
  for (int d = 0; d < 3; ++d) {
    ChainTable t;
    auto reset = [&]() {
      t.n = 0;
      for (int k = 0; k < kMaxJobs; ++k) { t.chunk_end[k] = 0xFFFFFFFFu; t.nvec[k] = 0; }
    };
    auto flush = [&]() {
      if (t.n == 0) return;
      const unsigned grid = t.chunk_end[t.n - 1];
      if (compress) {
        if (dts[d] == CTMI_BF16) hipLaunchKernelGGL(nvfp4_compress_chain_kernel<BF16>, grid, kFp4Block, 0, st, t);
        else if (dts[d] == CTMI_F16) hipLaunchKernelGGL(nvfp4_compress_chain_kernel<F16>, grid, kFp4Block, 0, st, t);
        else hipLaunchKernelGGL(nvfp4_compress_chain_kernel<F32>, grid, kFp4Block, 0, st, t);
      } else {
        if (dts[d] == CTMI_BF16) hipLaunchKernelGGL(nvfp4_decompress_chain_kernel<BF16>, grid, kFp4Block, 0, st, t);
        else if (dts[d] == CTMI_F16) hipLaunchKernelGGL(nvfp4_decompress_chain_kernel<F16>, grid, kFp4Block, 0, st, t);
        else hipLaunchKernelGGL(nvfp4_decompress_chain_kernel<F32>, grid, kFp4Block, 0, st, t);
      }
      reset();
    };
    reset();
    for (int64_t i = 0; i < n; ++i) {
      const ctmi_weight_job& j = jobs[i];
      VecGeom g;
      if (j.dense_dtype != dts[d] || !fp4_chainable(j, compress, &g)) continue;
      const uint64_t chunks = cdiv(g.nvec, per);
      const uint64_t before = t.n ? t.chunk_end[t.n - 1] : 0;
      if (t.n == kMaxJobs || before + chunks >= 0x7FFFFFFFull) flush();
      VecJob vj;
      vj.src = j.src;
      vj.dst = j.dst;
      vj.scale = j.qp.scale;
      vj.zp = reinterpret_cast<const int8_t*>(j.qp.global_scale);
      vj.g = g;
      t.job[t.n] = make_chain_job(vj);
      t.nvec[t.n] = g.nvec;
      t.chunk_end[t.n] = (uint32_t)((t.n ? t.chunk_end[t.n - 1] : 0) + chunks);
      ++t.n;
    }
    flush();
  }
  int rc = check_launch(what);
  if (rc) return rc;
  for (int64_t i = 0; i < n; ++i) {
    const ctmi_weight_job& j = jobs[i];
    VecGeom g;
    if (j.rows == 0 || j.cols == 0 || fp4_chainable(j, compress, &g)) continue;
    rc = compress ? ctmi_nvfp4_compress(j.src, j.dense_dtype, (uint8_t*)j.dst, j.rows, j.cols, &j.qp, stream)
                  : ctmi_nvfp4_decompress((const uint8_t*)j.src, j.dst, j.dense_dtype, j.rows, j.cols,
                                          &j.qp, stream);
    if (rc) return rc;
  }
  return CTMI_OK;
}

extern "C" int ctmi_nvfp4_compress_many(const ctmi_weight_job* jobs, int64_t n, void* stream) {
  return fp4_many(jobs, n, true, stream, "ctmi_nvfp4_compress_many");
}

extern "C" int ctmi_nvfp4_decompress_many(const ctmi_weight_job* jobs, int64_t n, void* stream) {
  return fp4_many(jobs, n, false, stream, "ctmi_nvfp4_decompress_many");
}

extern "C" int ctmi_observe_nvfp4_compress(const void* x, int32_t x_dtype, int64_t rows,
                                           int64_t cols, const float* global_scale,
                                           uint8_t* packed, uint8_t* scale, void* stream) {
  CTMI_REQUIRE(rows >= 1 && cols >= 1, CTMI_ERR_VALUE, "cannot observe an empty tensor");
  int rc = check_float3(x_dtype, "nvfp4 input");
  if (rc) return rc;
  CTMI_REQUIRE(cols % 16 == 0, CTMI_ERR_UNSUPPORTED, "columns must come in groups of 16");
  CTMI_REQUIRE(x && global_scale && packed && scale, CTMI_ERR_VALUE, "NULL tensor pointer");
  CTMI_REQUIRE((uintptr_t)x % (8 * dtype_size(x_dtype)) == 0 && (uintptr_t)packed % 4 == 0,
               CTMI_ERR_VALUE, "tensors must be aligned to 8 elements");
  const int64_t nvec = rows * cols / 8;
  const int64_t grid = cdiv(nvec, kFp4Block * kFp4ObserveU);
  CTMI_REQUIRE(nvec < (1ll << 32) && grid < (1ll << 31), CTMI_ERR_UNSUPPORTED, "tensor too large");
  hipStream_t st = (hipStream_t)stream;
  auto* out = (uint32_t*)packed;
  if (x_dtype == CTMI_BF16) hipLaunchKernelGGL(nvfp4_observe_compress_kernel<BF16>, (unsigned)grid, kFp4Block, 0, st, (const uint16_t*)x, global_scale, out, scale, (uint32_t)nvec);
  else if (x_dtype == CTMI_F16) hipLaunchKernelGGL(nvfp4_observe_compress_kernel<F16>, (unsigned)grid, kFp4Block, 0, st, (const uint16_t*)x, global_scale, out, scale, (uint32_t)nvec);
  else hipLaunchKernelGGL(nvfp4_observe_compress_kernel<F32>, (unsigned)grid, kFp4Block, 0, st, (const float*)x, global_scale, out, scale, (uint32_t)nvec);
  return check_launch("ctmi_observe_nvfp4_compress");
}

extern "C" int ctmi_observe_nvfp4_compress_many(const ctmi_observe_nvfp4_job* jobs, int64_t n,
                                                void* stream) {
  CTMI_REQUIRE(n >= 0 && (jobs || n == 0), CTMI_ERR_VALUE, "bad job list");
  // everything is checked before anything is enqueued
  for (int64_t i = 0; i < n; ++i) {
    const ctmi_observe_nvfp4_job& j = jobs[i];
    CTMI_REQUIRE(j.rows >= 1 && j.cols >= 1, CTMI_ERR_VALUE, "job %lld: cannot observe an empty tensor",
                 (long long)i);
    int rc = check_float3(j.x_dtype, "nvfp4 input");
    if (rc) return rc;
    CTMI_REQUIRE(j.cols % 16 == 0, CTMI_ERR_UNSUPPORTED, "job %lld: columns must come in groups of 16",
                 (long long)i);
    CTMI_REQUIRE(j.x && j.global_scale && j.packed && j.scale, CTMI_ERR_VALUE,
                 "job %lld: NULL tensor pointer", (long long)i);
    CTMI_REQUIRE((uintptr_t)j.x % (8 * dtype_size(j.x_dtype)) == 0 && (uintptr_t)j.packed % 4 == 0,
                 CTMI_ERR_VALUE, "job %lld: tensors must be aligned to 8 elements", (long long)i);
    CTMI_REQUIRE(j.rows * j.cols / 8 < (1ll << 31), CTMI_ERR_UNSUPPORTED, "job %lld: tensor too large",
                 (long long)i);
  }
  hipStream_t st = (hipStream_t)stream;
  const int dts[3] = {CTMI_BF16, CTMI_F16, CTMI_F32};
  for (int d = 0; d < 3; ++d) {
    ChainTable t;
    int filled = 0;
    uint32_t total = 0;
    auto flush = [&]() {
      for (int k = filled; k < kMaxJobs; ++k) {
        t.chunk_end[k] = 0xFFFFFFFFu;
        t.nvec[k] = 0;
        t.job[k] = ChainJob{};
      }
      t.n = filled;
      t.qmin = t.qmax = 0.0f;
      if (dts[d] == CTMI_BF16)
        hipLaunchKernelGGL(nvfp4_observe_compress_chain_kernel<BF16>, total, kFp4Block, 0, st, t);
      else if (dts[d] == CTMI_F16)
        hipLaunchKernelGGL(nvfp4_observe_compress_chain_kernel<F16>, total, kFp4Block, 0, st, t);
      else
        hipLaunchKernelGGL(nvfp4_observe_compress_chain_kernel<F32>, total, kFp4Block, 0, st, t);
      filled = 0;
      total = 0;
    };
    for (int64_t i = 0; i < n; ++i) {
      const ctmi_observe_nvfp4_job& j = jobs[i];
      if (j.x_dtype != dts[d]) continue;
      const uint32_t nvec = (uint32_t)(j.rows * j.cols / 8);
      const uint32_t chunks = (uint32_t)cdiv((int64_t)nvec, kFp4Block * kFp4ObserveU);
      if (filled && (uint64_t)total + chunks >= (1ull << 31)) flush();
      ChainJob cj{};
      cj.src = j.x;
      cj.dst = j.packed;
      cj.scale = j.scale;
      cj.zp = reinterpret_cast<const int8_t*>(j.global_scale);
      t.job[filled] = cj;
      t.nvec[filled] = nvec;
      total += chunks;
      t.chunk_end[filled] = total;
      if (++filled == kMaxJobs) flush();
    }
    if (filled) flush();
  }
  return n ? check_launch("ctmi_observe_nvfp4_compress_many") : CTMI_OK;
}
