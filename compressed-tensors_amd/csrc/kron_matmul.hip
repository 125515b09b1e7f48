// Transforms whose matrix is an explicit h x h factor, alone or beside a Sylvester factor.
//
//   apply_transform_weight / _multihead_matmul   transform/utils/matrix.py:65-171
//   _matmul_hadU, random_hadamard_matrix         transform/utils/hadamard.py:65-163
//
// The reference's Hadamard matrices of size n = K * 2^m (K from its table of known
// matrices: 12, 20, 28 ... 224, e.g. 14336 = 224 * 64) are
//     diag(Q) * (H_K^T (x) Sylvester(2^m)),
// which no power-of-two kernel covers.  This kernel applies
//     W = diag(sign_in) * (w (x) S_b) * diag(sign_out) * scale
// to every run of n = h * b elements x: with X = reshape(x * sign_in, [h, b]),
//     y = vec(w^T X S_b) * scale,    S_b = Sylvester(b) or, without it, the identity.
// Plain Sylvester transforms up to 512 (h = 1) stay inside a wavefront's registers
// (fwht_wave_kernel).  Otherwise a workgroup holds one run in LDS as fp32, runs the butterflies of S_b in place and
// then the product with w on the vector ALUs: a lane owns an inner index j, a wavefront
// a range of output rows, so that the entries of w it needs are wave-uniform and come
// through the scalar cache.  One rounding, at the end.  h = 224, b = 64: 3.2 M
// multiply-adds per run of 14336 elements; a rotation of a weight with 4096 such rows
// takes a fraction of a millisecond, once per weight.
#include "ctmi_device.h"
#include "ctmi_host.h"
#include "fwht.h"

namespace ctmi {
namespace {

constexpr int kKmThreads = 256;
constexpr int kKmAcc = 16;  // output rows a thread accumulates at a time

struct KronArgs {
  const void* x;
  void* out;
  const float* w;         // [h, h], row-major
  const float* sign_in;   // [h * b] or NULL
  const float* sign_out;  // [h * b] or NULL
  int64_t n_runs;
  int h, b, log2b, log2r, sylvester;
  float scale;
};

// A workgroup takes R runs at a time (R a power of two, R * b <= 256 lanes, R * n floats of
// LDS): short runs (n = 256, 512 ...) still fill its 256 threads.
// UNIFORM: R * b >= 64, every lane of a wavefront has the same output rows
template <typename IO, bool UNIFORM>
__global__ void __launch_bounds__(kKmThreads) kron_matmul_kernel(KronArgs a) {
  extern __shared__ float xs[];  // [R][h * b]
  const int n = a.h * a.b;
  const int R = 1 << a.log2r;
  const auto* __restrict__ x = static_cast<const typename IO::raw*>(a.x);
  auto* __restrict__ out = static_cast<typename IO::raw*>(a.out);
  const int tid = threadIdx.x;
  for (int64_t run0 = (int64_t)blockIdx.x * R; run0 < a.n_runs; run0 += (int64_t)gridDim.x * R) {
    __syncthreads();  // the previous runs' readers are done
    const int64_t left = a.n_runs - run0;
    const int live_runs = left < R ? (int)left : R;
    const int live = live_runs * n;
    for (int i = tid; i < R * n; i += kKmThreads) {
      float v = 0.0f;
      if (i < live) {
        v = IO::to_f32(x[run0 * n + i]);
        if (a.sign_in) v *= a.sign_in[R == 1 ? i : i % n];
      }
      xs[i] = v;
    }
    __syncthreads();
    if (a.sylvester) {
      // in-place butterflies along the inner index: strides 1, 2, ... b/2 give the
      // natural (Sylvester) order; a pair never leaves its row of b elements
      for (int st = 1; st < a.b; st <<= 1) {
        for (int p = tid; p < R * n / 2; p += kKmThreads) {
          const int i = (p / st) * 2 * st + (p % st);
          const float u = xs[i], v = xs[i + st];
          xs[i] = u + v;
          xs[i + st] = u - v;
        }
        __syncthreads();
      }
    }
    // y[k', j] = sum_k X[k, j] * w[k, k'] for each of the R runs
    const int log2l = a.log2b + a.log2r;
    const int lane = tid & ((1 << log2l) - 1);
    const int r = lane >> a.log2b;
    const int j = lane & (a.b - 1);
    int g = tid >> log2l;                    // which range of output rows
    if (UNIFORM) g = __builtin_amdgcn_readfirstlane(g);
    const int groups = kKmThreads >> log2l;  // >= 1: R * b <= 256, checked on the host
    const float* xr = xs + r * n + j;
    for (int k0 = g * kKmAcc; k0 < a.h; k0 += groups * kKmAcc) {
      float acc[kKmAcc];
#pragma unroll
      for (int i = 0; i < kKmAcc; ++i) acc[i] = 0.0f;
      const int cnt = a.h - k0 < kKmAcc ? a.h - k0 : kKmAcc;
      if (cnt == kKmAcc) {
        for (int k = 0; k < a.h; ++k) {
          const float xv = xr[k * a.b];
          const float* wr = a.w + (size_t)k * a.h + k0;
#pragma unroll
          for (int i = 0; i < kKmAcc; ++i) acc[i] = fmaf(xv, wr[i], acc[i]);
        }
      } else {
        for (int k = 0; k < a.h; ++k) {
          const float xv = xr[k * a.b];
          const float* wr = a.w + (size_t)k * a.h + k0;
#pragma unroll
          for (int i = 0; i < kKmAcc; ++i)
            if (i < cnt) acc[i] = fmaf(xv, wr[i], acc[i]);
        }
      }
      if (r < live_runs) {
#pragma unroll
        for (int i = 0; i < kKmAcc; ++i) {
          if (i < cnt) {
            const int o = (k0 + i) * a.b + j;
            float v = acc[i] * a.scale;
            if (a.sign_out) v *= a.sign_out[o];
            out[(run0 + r) * n + o] = IO::from_f32(v);
          }
        }
      }
    }
  }
}

// b = 1 (a block-diagonal matrix of explicit h x h blocks): 64 runs make one tile, a lane
// owns a run, so the product has the same shape as above with the run index as the inner
// one.  Loads and stores walk the tile linearly (full lines); the transposition happens in
// LDS, whose rows are padded to 65 words.
constexpr int kKmTile = 64;
constexpr int kKmPitch = kKmTile + 1;

template <typename IO>
__global__ void __launch_bounds__(kKmThreads) block_tile_kernel(KronArgs a) {
  extern __shared__ float xs[];  // x: [h][65], then y: [h][65]
  const int h = a.h;
  float* ys = xs + (size_t)h * kKmPitch;
  const auto* __restrict__ x = static_cast<const typename IO::raw*>(a.x);
  auto* __restrict__ out = static_cast<typename IO::raw*>(a.out);
  const int tid = threadIdx.x;
  const int64_t n_tiles = (a.n_runs + kKmTile - 1) / kKmTile;
  for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
    __syncthreads();
    const int64_t base = tile * kKmTile * h;
    const int64_t left = a.n_runs - tile * kKmTile;
    const int live = (int)(left < kKmTile ? left : kKmTile) * h;  // elements of this tile
    for (int i = tid; i < kKmTile * h; i += kKmThreads) {
      const int r = i / h, k = i - r * h;
      float v = 0.0f;
      if (i < live) {
        v = IO::to_f32(x[base + i]);
        if (a.sign_in) v *= a.sign_in[k];
      }
      xs[k * kKmPitch + r] = v;
    }
    __syncthreads();
    const int j = tid & (kKmTile - 1);
    const int g = __builtin_amdgcn_readfirstlane(tid >> 6);
    constexpr int groups = kKmThreads / kKmTile;
    for (int k0 = g * kKmAcc; k0 < h; k0 += groups * kKmAcc) {
      float acc[kKmAcc];
#pragma unroll
      for (int i = 0; i < kKmAcc; ++i) acc[i] = 0.0f;
      const int cnt = h - k0 < kKmAcc ? h - k0 : kKmAcc;
      if (cnt == kKmAcc) {
        for (int k = 0; k < h; ++k) {
          const float xv = xs[k * kKmPitch + j];
          const float* wr = a.w + (size_t)k * h + k0;
#pragma unroll
          for (int i = 0; i < kKmAcc; ++i) acc[i] = fmaf(xv, wr[i], acc[i]);
        }
      } else {
        for (int k = 0; k < h; ++k) {
          const float xv = xs[k * kKmPitch + j];
          const float* wr = a.w + (size_t)k * h + k0;
#pragma unroll
          for (int i = 0; i < kKmAcc; ++i)
            if (i < cnt) acc[i] = fmaf(xv, wr[i], acc[i]);
        }
      }
#pragma unroll
      for (int i = 0; i < kKmAcc; ++i)
        if (i < cnt) ys[(k0 + i) * kKmPitch + j] = acc[i] * a.scale;
    }
    __syncthreads();
    for (int i = tid; i < live; i += kKmThreads) {
      const int r = i / h, k = i - r * h;
      float v = ys[k * kKmPitch + r];
      if (a.sign_out) v *= a.sign_out[k];
      out[base + i] = IO::from_f32(v);
    }
  }
}

// h = 1 with the Sylvester factor, b <= 512: the butterflies never leave a wavefront.  A lane
// holds 8 neighbouring elements (three stages in registers), the strides 8 ... 256 pair it
// with the lanes xor 1 ... 32; a wavefront covers 512 elements = 512 / b runs.  No LDS, one
// 16-byte access per lane each way (two for float32).
constexpr int kFwhtPer = 8;
constexpr int kFwhtChunk = kWave * kFwhtPer;

// the value of lane (l ^ m): a data-parallel-primitive move where one exists (neighbours in
// a quad, the other half of a row of 16), the LDS crossbar otherwise.  m is a constant after
// unrolling.
__device__ __forceinline__ float lane_xor(float v, int m) {
  const int bits = __builtin_bit_cast(int, v);
  int r;
  if (m == 1) r = __builtin_amdgcn_update_dpp(bits, bits, 0xB1, 0xF, 0xF, false);        // quad_perm [1,0,3,2]
  else if (m == 2) r = __builtin_amdgcn_update_dpp(bits, bits, 0x4E, 0xF, 0xF, false);   // quad_perm [2,3,0,1]
  else if (m == 8) r = __builtin_amdgcn_update_dpp(bits, bits, 0x128, 0xF, 0xF, false);  // row_ror:8
  else r = wave_shfl_xor(bits, m);
  return __builtin_bit_cast(float, r);
}

template <typename IO>
__global__ void __launch_bounds__(kKmThreads) fwht_wave_kernel(KronArgs a, int64_t numel,
                                                                int vector_ok) {
  using R = typename IO::raw;
  constexpr int VE = 16 / (int)sizeof(R);
  const auto* __restrict__ x = static_cast<const R*>(a.x);
  auto* __restrict__ out = static_cast<R*>(a.out);
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave = ((int64_t)blockIdx.x * kKmThreads + threadIdx.x) / kWave;
  const int64_t n_waves = (int64_t)gridDim.x * (kKmThreads / kWave);
  const int64_t n_chunks = (numel + kFwhtChunk - 1) / kFwhtChunk;
  const float factor = a.w[0] * a.scale;
  for (int64_t chunk = wave; chunk < n_chunks; chunk += n_waves) {
    const int64_t e0 = chunk * kFwhtChunk + (int64_t)lane * kFwhtPer;
    const bool full = vector_ok && e0 + kFwhtPer <= numel;
    float v[kFwhtPer];
    if (full) {
#pragma unroll
      for (int q = 0; q < kFwhtPer / VE; ++q) {
        const Vec<R, VE> r = ldg_nt<R, VE>(x + e0 + q * VE);
#pragma unroll
        for (int i = 0; i < VE; ++i) v[q * VE + i] = IO::to_f32(r.v[i]);
      }
    } else {
#pragma unroll
      for (int i = 0; i < kFwhtPer; ++i) v[i] = e0 + i < numel ? IO::to_f32(x[e0 + i]) : 0.0f;
    }
    const int pos = (int)(e0 & (a.b - 1));  // b divides the chunk size or is a multiple of 8
    if (a.sign_in) {
#pragma unroll
      for (int i = 0; i < kFwhtPer; ++i) v[i] *= a.sign_in[(pos + i) & (a.b - 1)];
    }
    // strides 1, 2, 4: inside the lane (runs shorter than 8 stop early)
#pragma unroll
    for (int st = 1; st < kFwhtPer; st <<= 1) {
      if (st < a.b) {
#pragma unroll
        for (int i = 0; i < kFwhtPer; ++i) {
          if ((i & st) == 0) {
            const float u = v[i], w = v[i + st];
            v[i] = u + w;
            v[i + st] = u - w;
          }
        }
      }
    }
    // strides 8 ... b / 2: between lanes
#pragma unroll
    for (int m = 1; m < kWave; m <<= 1) {
      if (m * kFwhtPer < a.b) {
        const bool upper = (lane & m) != 0;
#pragma unroll
        for (int i = 0; i < kFwhtPer; ++i) {
          const float other = lane_xor(v[i], m);
          v[i] = upper ? other - v[i] : v[i] + other;
        }
      }
    }
#pragma unroll
    for (int i = 0; i < kFwhtPer; ++i) {
      v[i] *= factor;
      if (a.sign_out) v[i] *= a.sign_out[(pos + i) & (a.b - 1)];
    }
    if (full) {
      if constexpr (VE == 8) {
        stg_nt<R, 8>(out + e0, pack8_from_f32<IO>(v));
      } else {
#pragma unroll
        for (int q = 0; q < kFwhtPer / VE; ++q) {
          Vec<R, VE> r;
#pragma unroll
          for (int i = 0; i < VE; ++i) r.v[i] = IO::from_f32(v[q * VE + i]);
          stg_nt<R, VE>(out + e0 + q * VE, r);
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < kFwhtPer; ++i)
        if (e0 + i < numel) out[e0 + i] = IO::from_f32(v[i]);
    }
  }
}

constexpr size_t kKmLdsMax = 160 * 1024 - 1024;

size_t kron_lds_bytes(int h, int b) {
  return b == 1 ? (size_t)h * kKmPitch * 2 * sizeof(float) : (size_t)h * b * sizeof(float);
}

template <typename IO>
int launch_kron(const KronArgs& a, hipStream_t st) {
  if (a.h == 1 && a.sylvester && fwht_size_supported(a.b)) {
    FwhtJob job;
    job.x = a.x;
    job.out = a.out;
    job.packed = nullptr;
    job.scale = nullptr;
    job.rows = a.n_runs;
    return fwht_launch(&job, 1, IO::id, a.b, a.sign_in, a.sign_out, a.w, a.scale, nullptr, st);
  }
  if (a.h == 1 && a.sylvester && a.b <= kFwhtChunk) {
    const int64_t numel = a.n_runs * a.b;
    const int64_t n_chunks = (numel + kFwhtChunk - 1) / kFwhtChunk;
    const int64_t n_wg = (n_chunks + kKmThreads / kWave - 1) / (kKmThreads / kWave);
    const unsigned grid = (unsigned)(n_wg < 256 * 16 ? n_wg : 256 * 16);
    const int vector_ok = (uintptr_t)a.x % 16 == 0 && (uintptr_t)a.out % 16 == 0;
    hipLaunchKernelGGL(fwht_wave_kernel<IO>, grid, kKmThreads, 0, st, a, numel, vector_ok);
    return CTMI_OK;
  }
  if (a.b == 1) {
    const size_t lds = kron_lds_bytes(a.h, 1);
    auto kern = block_tile_kernel<IO>;
    if (lds > 48 * 1024) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e != hipSuccess)
        return set_error(CTMI_ERR_HIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    }
    const int64_t n_tiles = (a.n_runs + kKmTile - 1) / kKmTile;
    const unsigned grid = (unsigned)(n_tiles < 256 * 8 ? n_tiles : 256 * 8);
    hipLaunchKernelGGL(kern, grid, kKmThreads, lds, st, a);
    return CTMI_OK;
  }
  // runs per workgroup: up to 256 lanes and 32 KB of LDS, never more runs than there are
  KronArgs k = a;
  k.log2r = 0;
  const size_t run_bytes = (size_t)a.h * a.b * sizeof(float);
  while ((2 << k.log2r) * a.b <= kKmThreads && (run_bytes << (k.log2r + 1)) <= 32 * 1024 &&
         (int64_t)(2 << k.log2r) <= a.n_runs)
    ++k.log2r;
  const size_t lds = run_bytes << k.log2r;
  auto uniform = kron_matmul_kernel<IO, true>;
  auto mixed = kron_matmul_kernel<IO, false>;
  auto kern = (a.b << k.log2r) >= 64 ? uniform : mixed;
  if (lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess)
      return set_error(CTMI_ERR_HIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  }
  const int64_t n_wg = (a.n_runs + (1 << k.log2r) - 1) >> k.log2r;
  const unsigned grid = (unsigned)(n_wg < 256 * 8 ? n_wg : 256 * 8);
  hipLaunchKernelGGL(kern, grid, kKmThreads, lds, st, k);
  return CTMI_OK;
}

}  // namespace
}  // namespace ctmi

using namespace ctmi;

extern "C" int ctmi_kron_matmul_supported(int32_t h, int32_t b, int32_t io_dtype) {
  if (!(io_dtype == CTMI_BF16 || io_dtype == CTMI_F16 || io_dtype == CTMI_F32)) return 0;
  if (h < 1 || b < 1 || (b & (b - 1)) != 0) return 0;
  if (h == 1 && (b <= 512 || fwht_size_supported(b))) return 1;  // butterflies in registers
  if (b > 256) return 0;
  return kron_lds_bytes(h, b) <= kKmLdsMax ? 1 : 0;  // a run (b = 1: a tile of 64) as fp32 in LDS
}

extern "C" int ctmi_kron_matmul(const void* x, void* out, int32_t io_dtype, int64_t numel, int32_t h,
                                int32_t b, const float* w, const float* sign_in,
                                const float* sign_out, int32_t sylvester, float scale,
                                void* stream) {
  CTMI_REQUIRE(numel >= 0, CTMI_ERR_VALUE, "negative size");
  CTMI_REQUIRE(io_dtype == CTMI_BF16 || io_dtype == CTMI_F16 || io_dtype == CTMI_F32,
               CTMI_ERR_UNSUPPORTED, "transforms take float16/bfloat16/float32 tensors");
  CTMI_REQUIRE(h >= 1 && b >= 1, CTMI_ERR_VALUE, "empty transform");
  CTMI_REQUIRE(ctmi_kron_matmul_supported(h, b, io_dtype), CTMI_ERR_UNSUPPORTED,
               "a run of %d x %d elements does not fit the kernel (inner size a power of two up "
               "to 256 and %d x %d x 4 bytes within 159 KB; for inner size 1, h up to 313)",
               h, b, h, b);
  CTMI_REQUIRE(b <= 256 || (h == 1 && sylvester), CTMI_ERR_UNSUPPORTED,
               "an inner size of %d runs only as a plain Sylvester transform (h = 1)", b);
  CTMI_REQUIRE(numel % ((int64_t)h * b) == 0, CTMI_ERR_VALUE,
               "tensor size %lld is not a multiple of the transform size %lld", (long long)numel,
               (long long)h * b);
  if (numel == 0) return CTMI_OK;
  CTMI_REQUIRE(x && out && w, CTMI_ERR_VALUE, "NULL tensor pointer");
  KronArgs a;
  a.x = x;
  a.out = out;
  a.w = w;
  a.sign_in = sign_in;
  a.sign_out = sign_out;
  a.n_runs = numel / ((int64_t)h * b);
  a.h = h;
  a.b = b;
  a.log2b = 0;
  while ((1 << a.log2b) < b) ++a.log2b;
  a.log2r = 0;
  a.sylvester = sylvester ? 1 : 0;
  a.scale = scale;
  hipStream_t st = (hipStream_t)stream;
  int rc;
  if (io_dtype == CTMI_BF16) rc = launch_kron<BF16>(a, st);
  else if (io_dtype == CTMI_F16) rc = launch_kron<F16>(a, st);
  else rc = launch_kron<F32>(a, st);
  if (rc) return rc;
  return check_launch("ctmi_kron_matmul");
}

// A24 for an explicit matrix: the case b = 1 of the kernel above
extern "C" int ctmi_block_matmul(const void* x, void* out, int32_t io_dtype, int64_t numel,
                                 int32_t h, const float* w, void* stream) {
  CTMI_REQUIRE(h >= 1, CTMI_ERR_VALUE, "empty block");
  return ctmi_kron_matmul(x, out, io_dtype, numel, h, 1, w, nullptr, nullptr, 0,
                          1.0f / sqrtf((float)h), stream);
}
