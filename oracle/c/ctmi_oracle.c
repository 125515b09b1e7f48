/*
 * C restatement of the scalar arithmetic on the compress / decompress path —
 * TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).  It exists to pin the
 * torch-CPU oracle from an independent direction: every routine here is
 * written from the number formats' definitions, not from torch's code.
 *
 *   bf16 / fp8-e4m3fn rounding   the casts inside quantization/lifecycle/forward.py:471-485
 *                                and quantization/quant_args.py:398
 *   quantize / dequantize chain  forward.py:455-514
 *   fp4 buckets                  quant_args.py:55-68
 *   int32 packing                compressors/quantized_compressors/pack_quantized.py:220-241, 285-307
 *   fp4 nibble packing           compressors/quantized_compressors/fp4_quantized.py:159-178, 206-218
 *   bit packing                  utils/helpers.py:310 (numpy.packbits, bitorder="little")
 *
 * Build: make -C oracle   ->  oracle/_build/libctmi_oracle.so
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* ---------------------------------------------------------------- bf16 */
float oracle_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

/* nearest bf16, ties to the even mantissa; derived with exact integer arithmetic
 * on the fp32 bit pattern (adjacent bf16 values differ by 0x10000 there) */
uint16_t oracle_f32_to_bf16(float f) {
  uint32_t u = f2u(f);
  if (isnan(f)) return 0x7FC0;
  uint32_t lower = u & 0xFFFF0000u;      /* truncation toward zero */
  uint32_t rem = u & 0xFFFFu;
  uint32_t upper = lower + 0x10000u;     /* next magnitude (may become inf: correct) */
  if (rem > 0x8000u) return (uint16_t)(upper >> 16);
  if (rem < 0x8000u) return (uint16_t)(lower >> 16);
  return (uint16_t)(((lower >> 16) & 1u) ? (upper >> 16) : (lower >> 16));
}

static float rbf16(float f) { return oracle_bf16_to_f32(oracle_f32_to_bf16(f)); }

/* ---------------------------------------------------------------- fp8 e4m3fn */
double oracle_f8e4m3_value(uint8_t code) { /* magnitude codes 0..0x7E */
  int e = (code >> 3) & 0xF, m = code & 7;
  double v = e == 0 ? ldexp((double)m, -9) : ldexp(1.0 + m / 8.0, e - 7);
  return (code & 0x80) ? -v : v;
}

float oracle_f8e4m3_to_f32(uint8_t code) {
  if ((code & 0x7F) == 0x7F) return (code & 0x80) ? -NAN : NAN;
  return (float)oracle_f8e4m3_value(code);
}

/* nearest representable magnitude by exhaustive search over the 127 finite
 * codes, ties to the even code; values beyond the midpoint between 448 and the
 * (non-existent) next value 480 — i.e. > 464 — and NaN give 0x7F (the tie at
 * 464 itself goes to the even code, 448). */
uint8_t oracle_f32_to_f8e4m3(float f) {
  uint8_t sign = (f2u(f) >> 31) ? 0x80 : 0;
  if (isnan(f)) return sign | 0x7F;
  double a = fabs((double)f);
  if (a > 464.0) return sign | 0x7F;
  int best = 0;
  double bd = a;
  for (int c = 1; c <= 0x7E; ++c) {
    double d = fabs(a - oracle_f8e4m3_value((uint8_t)c));
    if (d < bd || (d == bd && (c & 1) == 0 && (best & 1) == 1)) { bd = d; best = c; }
  }
  return sign | (uint8_t)best;
}

/* ---------------------------------------------------------------- fp4 e2m1 */
static const float kE2M1[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};

/* nearest e2m1 magnitude, ties to the code with even mantissa bit
 * (.25->0, .75->1, 1.25->1, 1.75->2, 2.5->2, 3.5->4, 5->4), times sign(x);
 * sign(+-0) = 0 makes exact zeros positive. */
float oracle_cast_to_fp4(float x) {
  if (isnan(x)) return x;
  float a = fabsf(x);
  int best = 0;
  for (int c = 1; c < 8; ++c) {
    float d = fabsf(a - kE2M1[c]), bd = fabsf(a - kE2M1[best]);
    if (d < bd || (d == bd && (c & 1) == 0)) best = c;
  }
  float sgn = x > 0 ? 1.0f : (x < 0 ? -1.0f : 0.0f);
  return kE2M1[best] * sgn;
}

uint8_t oracle_fp4_code(float v) { /* v on the e2m1 grid */
  int c = 0;
  for (int k = 0; k < 8; ++k) if (fabsf(v) == kE2M1[k]) c = k;
  return (uint8_t)(c | ((f2u(v) >> 31) << 3));
}

float oracle_fp4_decode(uint8_t code) {
  float m = kE2M1[code & 7];
  return (code & 8) ? -m : m;
}

/* ---------------------------------------------------------------- quantize chain
 * compute dtype: 0 = fp32, 2 = bf16 (every op rounded to it). */
static float rct(float v, int ct) { return ct == 2 ? rbf16(v) : v; }

static float clampf(float v, float lo, float hi) {
  if (isnan(v)) return v;
  return v < lo ? lo : (v > hi ? hi : v);
}

/* qkind: 0 = int(num_bits), 1 = fp8 e4m3fn, 2 = fp4 e2m1.  Returns the quantized
 * VALUE (an integer, an fp8-representable or an e2m1 number). */
float oracle_quantize(float x, float scale, float zp, int has_zp, int qkind, int num_bits, int ct) {
  float v = rct(x / scale, ct);
  if (has_zp) v = rct(v + zp, ct);
  if (qkind == 0) {
    float half = ldexpf(1.0f, num_bits - 1);
    return nearbyintf(clampf(v, -half, half - 1.0f));
  }
  if (qkind == 1) return oracle_f8e4m3_to_f32(oracle_f32_to_f8e4m3(clampf(v, -448.0f, 448.0f)));
  return oracle_cast_to_fp4(clampf(v, -6.0f, 6.0f));
}

float oracle_dequantize(float q, float scale, float zp, int has_zp, int dt) {
  float v = rct(q, dt);
  if (has_zp) v = rct(v - zp, dt);
  return rct(v * scale, dt);
}

/* vector forms over raw bf16 buffers, group-wise scales along the last dim */
void oracle_quantize_int_bf16(const uint16_t* x, const uint16_t* scale, const int8_t* zp,
                              int8_t* out, int64_t rows, int64_t cols, int64_t group,
                              int num_bits) {
  int64_t ng = cols / group;
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t c = 0; c < cols; ++c) {
      int64_t si = r * ng + c / group;
      float q = oracle_quantize(oracle_bf16_to_f32(x[r * cols + c]), oracle_bf16_to_f32(scale[si]),
                                zp ? (float)zp[si] : 0.0f, zp != 0, 0, num_bits, 2);
      out[r * cols + c] = (int8_t)q;
    }
}

void oracle_dequantize_int_bf16(const int8_t* q, const uint16_t* scale, const int8_t* zp,
                                uint16_t* out, int64_t rows, int64_t cols, int64_t group) {
  int64_t ng = cols / group;
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t c = 0; c < cols; ++c) {
      int64_t si = r * ng + c / group;
      float v = oracle_dequantize((float)q[r * cols + c], oracle_bf16_to_f32(scale[si]),
                                  zp ? (float)zp[si] : 0.0f, zp != 0, 2);
      out[r * cols + c] = oracle_f32_to_bf16(v);
    }
}

/* ---------------------------------------------------------------- int32 packing */
void oracle_pack_to_int32(const int8_t* in, int32_t* out, int64_t rows, int64_t cols,
                          int num_bits) {
  int pf = 32 / num_bits;
  int64_t pcols = (cols + pf - 1) / pf;
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t j = 0; j < pcols; ++j) {
      uint32_t acc = 0;
      for (int i = 0; i < pf; ++i) {
        int64_t c = j * pf + i;
        uint32_t u = c < cols ? (uint8_t)(in[r * cols + c] + (1 << (num_bits - 1))) : 0u;
        acc += u << (num_bits * i);
      }
      out[r * pcols + j] = (int32_t)acc;
    }
}

void oracle_unpack_from_int32(const int32_t* in, int8_t* out, int64_t rows, int64_t cols,
                              int num_bits) {
  int pf = 32 / num_bits;
  int64_t pcols = (cols + pf - 1) / pf;
  uint32_t mask = (1u << num_bits) - 1u;
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t c = 0; c < cols; ++c) {
      uint32_t w = (uint32_t)in[r * pcols + c / pf];
      out[r * cols + c] = (int8_t)((int)((w >> (num_bits * (c % pf))) & mask) - (1 << (num_bits - 1)));
    }
}

/* ---------------------------------------------------------------- bit packing */
void oracle_packbits_little(const uint8_t* mask, uint8_t* out, int64_t rows, int64_t cols) {
  int64_t pc = (cols + 7) / 8;
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t b = 0; b < pc; ++b) {
      uint8_t v = 0;
      for (int j = 0; j < 8; ++j) {
        int64_t c = b * 8 + j;
        if (c < cols && mask[r * cols + c]) v |= (uint8_t)(1u << j);
      }
      out[r * pc + b] = v;
    }
}

/* sparse-bitmask compress of a 2-byte-element tensor: returns nnz */
int64_t oracle_bitmask_compress_u16(const uint16_t* x, int64_t rows, int64_t cols,
                                    uint16_t* values, uint8_t* bitmask, int64_t* row_offsets) {
  int64_t pc = (cols + 7) / 8, n = 0;
  memset(bitmask, 0, (size_t)(rows * pc));
  for (int64_t r = 0; r < rows; ++r) {
    row_offsets[r] = n;
    for (int64_t c = 0; c < cols; ++c) {
      uint16_t v = x[r * cols + c];
      if ((v & 0x7FFF) != 0) { /* value != 0: -0.0 is zero, NaN is not */
        values[n++] = v;
        bitmask[r * pc + c / 8] |= (uint8_t)(1u << (c % 8));
      }
    }
  }
  return n;
}
