// quantize / dequantize / fake-quantize kernels.
//
// Numerics contract: the reference evaluates an op chain in torch, one op at a
// time, each op computed in fp32 and rounded to the tensor dtype torch's type
// promotion picked.  The kernels here replay the same chain per element in
// registers: every intermediate is rounded to that dtype (`round_to`) before
// the next op, so results are bit-identical while the tensor is read once and
// written once.
//
//   _quantize   (quantization/lifecycle/forward.py:455-487)
//   _dequantize (forward.py:491-514)
//   round_to_quantized_type / cast_to_fp4 (quantization/quant_args.py:55-68, 384-408)
#include "ctmi_device.h"
#include "ctmi_host.h"
#include "quant_core.h"
#include "vec_geom.h"
#include "job_table.h"

#include <cstring>
#include <vector>

namespace ctmi {

// ------------------------------------------------------------------ generic kernel
// One element per thread, any dtype / strategy combination.  Used whenever no
// vectorised specialisation applies.
struct QdqArgs {
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
  int do_q, do_dq;
};

__global__ void __launch_bounds__(256) qdq_generic_kernel(QdqArgs a) {
  const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= a.cols) return;
  const int64_t scol = a.col_group ? (int64_t)a.col_group[c] : c / a.blk_cols;
  const float gs = a.gscale ? a.gscale[0] : 1.0f;
  for (int64_t r = blockIdx.y; r < a.rows; r += gridDim.y) {
    const int64_t srow = (r / a.blk_rows) % a.s_rows;
    const int64_t si = srow * a.s_cols + scol;
    float s = load_f32(a.scale, a.scale_dtype, si);
    if (a.gscale) s = s / gs;  // scale.to(float32) / global_scale
    float zq = 0.0f, zd = 0.0f;
    if (a.zp) {
      float z = load_f32(a.zp, a.zp_dtype, si);
      zq = round_to(z, a.x_dtype);   // zero_point.to(x.dtype)
      zd = round_to(z, a.q.dt);      // zero_point.to(scale.dtype)
    }
    const int64_t i = r * a.cols + c;
    float v = load_f32(a.x, a.x_dtype, i);
    if (a.do_q) v = quantize_value(v, s, zq, a.zp != nullptr, a.q);
    if (a.do_dq) v = dequantize_value(v, s, zd, a.zp != nullptr, a.q.dt);
    store_from_f32(a.out, a.out_dtype, i, v);
  }
}

struct QdqKey {
  int sd, in_kind, out_kind, qk, has_zp, flat;
  bool operator==(const QdqKey& o) const {
    return sd == o.sd && in_kind == o.in_kind && out_kind == o.out_kind && qk == o.qk &&
           has_zp == o.has_zp && flat == o.flat;
  }
};
bool qdq_classify(const void* x, int x_dtype, const void* out, int out_dtype, int64_t rows,
                  int64_t cols, const ctmi_qparams* qp, int do_q, int do_dq, QdqKey* key,
                  VecGeom* g, float* qmin, float* qmax);
void qdq_launch_chain(const QdqKey& k, const ChainTable& t, unsigned grid, hipStream_t st);
int qdq_chunk_items();
bool qdq_try_vectorised(const void* x, int x_dtype, void* out, int out_dtype, int64_t rows,
                        int64_t cols, const ctmi_qparams* qp, int do_q, int do_dq, hipStream_t st);
bool nvfp4_qdq_try_vectorised(const void* x, int x_dtype, void* out, int out_dtype, int64_t rows,
                              int64_t cols, const ctmi_qparams* qp, hipStream_t st);
bool qdq_gidx_try(const void* x, int x_dtype, void* out, int out_dtype, int64_t rows, int64_t cols,
                  const ctmi_qparams* qp, int do_q, int do_dq, hipStream_t st);

// ------------------------------------------------------------------ round_to_quantized_type
// quant_args.py:384-408 on its own: every element to the nearest value of the quantized
// type, in the tensor's dtype, no scale and no clamp.  MODE 0: torch.round (ties to
// even); 1: to float8_e4m3fn and back; 2: FP4_E2M1_DATA.cast_to_fp4.
template <typename XT, int MODE>
__global__ void __launch_bounds__(256)
round_to_type_kernel(const typename XT::raw* __restrict__ x, typename XT::raw* __restrict__ out,
                     int64_t n) {
  constexpr int VE = 16 / (int)sizeof(typename XT::raw);
  const auto one = [](float v) {
    if constexpr (MODE == 0) return rintf(v);
    else if constexpr (MODE == 1) {
      // the hardware converter: nearest even, NaN beyond the largest value's rounding range,
      // as torch's cast (checked on every 16-bit pattern)
      return __builtin_amdgcn_cvt_f32_fp8(__builtin_amdgcn_cvt_pk_fp8_f32(v, v, 0, false), 0);
    }
    else return cast_to_fp4(v);
  };
  // 4 vectors a lane, all of them asked for before any is used; the tensor is read and
  // written once: streaming loads and stores
  constexpr int U = 4;
  const int64_t nvec = n / VE;
  const int64_t v0 = (int64_t)blockIdx.x * (256 * U) + threadIdx.x;
  Vec<typename XT::raw, VE> a[U];
  if (nvec > 0) {
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const int64_t v = v0 + k * 256;
      a[k] = ldg_nt<typename XT::raw, VE>(x + (v < nvec ? v : nvec - 1) * VE);  // past the end: re-read, not stored
    }
#pragma unroll
    for (int k = 0; k < U; ++k) {
      const int64_t v = v0 + k * 256;
#pragma unroll
      for (int j = 0; j < VE; ++j) a[k].v[j] = XT::from_f32(one(XT::to_f32(a[k].v[j])));
      if (v < nvec) stg_nt<typename XT::raw, VE>(out + v * VE, a[k]);
    }
  }
  if (blockIdx.x == 0 && threadIdx.x < n - nvec * VE) {
    const int64_t i = nvec * VE + threadIdx.x;
    out[i] = XT::from_f32(one(XT::to_f32(x[i])));
  }
}

template <typename XT>
static void round_to_type_launch(const void* x, void* out, int64_t n, int mode, hipStream_t st) {
  using R = typename XT::raw;
  constexpr int VE = 16 / (int)sizeof(R);
  const int64_t want = cdiv(n / VE, 256 * 4);
  const unsigned grid = (unsigned)(want < 1 ? 1 : want);
  if (mode == 0)
    hipLaunchKernelGGL((round_to_type_kernel<XT, 0>), grid, 256, 0, st, (const R*)x, (R*)out, n);
  else if (mode == 1)
    hipLaunchKernelGGL((round_to_type_kernel<XT, 1>), grid, 256, 0, st, (const R*)x, (R*)out, n);
  else
    hipLaunchKernelGGL((round_to_type_kernel<XT, 2>), grid, 256, 0, st, (const R*)x, (R*)out, n);
}

// ------------------------------------------------------------------ host side
static int fill_cfg(const ctmi_qparams* qp, int x_dtype, QuantCfg* q) {
  int rc = quant_range(qp->qtype, qp->num_bits, &q->qmin, &q->qmax);
  if (rc) return rc;
  q->qtype = qp->qtype;
  q->num_bits = qp->num_bits;
  const int sdt = qp->global_scale ? CTMI_F32 : qp->scale_dtype;
  q->dt = sdt;
  q->ct = is_float_dtype(x_dtype) && x_dtype != CTMI_F8E4M3 ? promote_float(x_dtype, sdt) : sdt;
  return CTMI_OK;
}

}  // namespace ctmi

using namespace ctmi;

static int qdq_validate(const void* x, int32_t x_dtype, const void* out, int32_t out_dtype,
                        int64_t rows, int64_t cols, const ctmi_qparams* qp, int32_t do_quantize,
                        int32_t do_dequantize) {
  CTMI_REQUIRE(rows >= 0 && cols >= 0, CTMI_ERR_VALUE, "negative shape");
  CTMI_REQUIRE(do_quantize || do_dequantize, CTMI_ERR_VALUE, "nothing to do");
  CTMI_REQUIRE(dtype_size(x_dtype) > 0 && x_dtype != CTMI_I64, CTMI_ERR_UNSUPPORTED,
               "unsupported input dtype %d", x_dtype);
  CTMI_REQUIRE(dtype_size(out_dtype) > 0 && out_dtype != CTMI_I64 && out_dtype != CTMI_BOOL,
               CTMI_ERR_UNSUPPORTED, "unsupported output dtype %d", out_dtype);
  if (do_quantize) {
    CTMI_REQUIRE(x_dtype == CTMI_F32 || x_dtype == CTMI_F16 || x_dtype == CTMI_BF16,
                 CTMI_ERR_UNSUPPORTED, "quantize needs a float16/bfloat16/float32 input");
  }
  int rc = check_qparams(qp, rows, cols);
  if (rc) return rc;
  if (rows == 0 || cols == 0) return CTMI_OK;
  CTMI_REQUIRE(x != nullptr && out != nullptr, CTMI_ERR_VALUE, "NULL tensor pointer");
  QuantCfg q;
  return fill_cfg(qp, x_dtype, &q);
}

// the any-layout kernel, for a validated problem
static void qdq_enqueue_generic(const void* x, int32_t x_dtype, void* out, int32_t out_dtype,
                                int64_t rows, int64_t cols, const ctmi_qparams* qp,
                                int32_t do_quantize, int32_t do_dequantize, hipStream_t st) {
  QdqArgs a;
  a.x = x;
  a.out = out;
  a.scale = qp->scale;
  a.zp = qp->zero_point;
  a.gscale = qp->global_scale;
  a.col_group = qp->col_group;
  a.rows = rows;
  a.cols = cols;
  a.s_rows = qp->s_rows;
  a.s_cols = qp->s_cols;
  a.blk_rows = qp->blk_rows;
  a.blk_cols = qp->blk_cols;
  a.x_dtype = x_dtype;
  a.out_dtype = out_dtype;
  a.scale_dtype = qp->scale_dtype;
  a.zp_dtype = qp->zp_dtype;
  a.do_q = do_quantize;
  a.do_dq = do_dequantize;
  fill_cfg(qp, x_dtype, &a.q);
  dim3 block(256);
  dim3 grid((unsigned)cdiv(cols, 256), (unsigned)(rows < 32768 ? rows : 32768));
  hipLaunchKernelGGL(qdq_generic_kernel, grid, block, 0, st, a);
}

extern "C" int ctmi_round_to_quantized_type(const void* x, void* out, int32_t dtype, int64_t n,
                                           int32_t qtype, int32_t num_bits, void* stream) {
  CTMI_REQUIRE(n >= 0, CTMI_ERR_VALUE, "negative size");
  CTMI_REQUIRE(dtype == CTMI_F32 || dtype == CTMI_F16 || dtype == CTMI_BF16, CTMI_ERR_UNSUPPORTED,
               "round_to_quantized_type needs a float16/bfloat16/float32 tensor");
  CTMI_REQUIRE(qtype == CTMI_QTYPE_INT || qtype == CTMI_QTYPE_FLOAT, CTMI_ERR_VALUE,
               "Invalid quantization type %d", qtype);
  CTMI_REQUIRE(qtype == CTMI_QTYPE_INT || num_bits == 4 || num_bits == 8, CTMI_ERR_UNSUPPORTED,
               "Only num_bits in (4, 8) are supported");
  if (n == 0) return CTMI_OK;
  CTMI_REQUIRE(x != nullptr && out != nullptr, CTMI_ERR_VALUE, "NULL tensor pointer");
  CTMI_REQUIRE((uintptr_t)x % 16 == 0 && (uintptr_t)out % 16 == 0, CTMI_ERR_VALUE,
               "tensors must be 16-byte aligned");
  const int mode = qtype == CTMI_QTYPE_INT ? 0 : num_bits == 8 ? 1 : 2;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == CTMI_BF16) round_to_type_launch<BF16>(x, out, n, mode, st);
  else if (dtype == CTMI_F16) round_to_type_launch<F16>(x, out, n, mode, st);
  else round_to_type_launch<F32>(x, out, n, mode, st);
  return check_launch("ctmi_round_to_quantized_type");
}

extern "C" int ctmi_qdq(const void* x, int32_t x_dtype, void* out, int32_t out_dtype, int64_t rows,
                        int64_t cols, const ctmi_qparams* qp, int32_t do_quantize,
                        int32_t do_dequantize, void* stream) {
  int rc = qdq_validate(x, x_dtype, out, out_dtype, rows, cols, qp, do_quantize, do_dequantize);
  if (rc) return rc;
  if (rows == 0 || cols == 0) return CTMI_OK;
  hipStream_t st = (hipStream_t)stream;
  if (qdq_try_vectorised(x, x_dtype, out, out_dtype, rows, cols, qp, do_quantize, do_dequantize, st))
    return check_launch("ctmi_qdq");
  if (do_quantize && do_dequantize &&
      nvfp4_qdq_try_vectorised(x, x_dtype, out, out_dtype, rows, cols, qp, st))
    return check_launch("ctmi_qdq");
  if (qdq_gidx_try(x, x_dtype, out, out_dtype, rows, cols, qp, do_quantize, do_dequantize, st))
    return check_launch("ctmi_qdq");
  qdq_enqueue_generic(x, x_dtype, out, out_dtype, rows, cols, qp, do_quantize, do_dequantize, st);
  return check_launch("ctmi_qdq");
}

// Every job is validated before anything is enqueued; jobs the vectorised
// kernels take are chained, kMaxJobs per launch and kernel instance, the others
// run as ctmi_qdq would run them.
extern "C" int ctmi_qdq_many(const ctmi_qdq_job* jobs, int64_t n, int32_t do_quantize,
                             int32_t do_dequantize, void* stream) {
  CTMI_REQUIRE(n >= 0 && (jobs || n == 0), CTMI_ERR_VALUE, "bad job list");
  for (int64_t i = 0; i < n; ++i) {
    const ctmi_qdq_job& j = jobs[i];
    int rc = qdq_validate(j.x, j.x_dtype, j.out, j.out_dtype, j.rows, j.cols, &j.qp, do_quantize,
                          do_dequantize);
    if (rc) return rc;
  }
  hipStream_t st = (hipStream_t)stream;
  struct Plan {
    bool vec;
    QdqKey key;
    VecJob job;
    float qmin, qmax;
  };
  std::vector<Plan> plans((size_t)n);
  std::vector<char> done((size_t)n, 0);
  for (int64_t i = 0; i < n; ++i) {
    const ctmi_qdq_job& j = jobs[i];
    Plan& p = plans[i];
    if (j.rows == 0 || j.cols == 0) { done[i] = 1; continue; }
    p.vec = qdq_classify(j.x, j.x_dtype, j.out, j.out_dtype, j.rows, j.cols, &j.qp, do_quantize,
                         do_dequantize, &p.key, &p.job.g, &p.qmin, &p.qmax);
    if (p.vec) {
      p.job.src = j.x;
      p.job.dst = j.out;
      p.job.scale = j.qp.scale;
      p.job.zp = (const int8_t*)j.qp.zero_point;
      continue;
    }
    if (!(do_quantize && do_dequantize &&
          nvfp4_qdq_try_vectorised(j.x, j.x_dtype, j.out, j.out_dtype, j.rows, j.cols, &j.qp, st)) &&
        !qdq_gidx_try(j.x, j.x_dtype, j.out, j.out_dtype, j.rows, j.cols, &j.qp, do_quantize,
                      do_dequantize, st))
      qdq_enqueue_generic(j.x, j.x_dtype, j.out, j.out_dtype, j.rows, j.cols, &j.qp, do_quantize,
                          do_dequantize, st);
    done[i] = 1;
  }
  const int per_chunk = qdq_chunk_items();
  for (int64_t i = 0; i < n; ++i) {
    if (done[i]) continue;
    const QdqKey key = plans[i].key;
    ChainTable t;
    std::memset(&t, 0, sizeof(t));
    uint64_t chunks = 0;
    auto reset = [&]() {
      t.n = 0;
      chunks = 0;
      for (int k = 0; k < kMaxJobs; ++k) t.chunk_end[k] = 0xFFFFFFFFu;
    };
    reset();
    t.qmin = plans[i].qmin;
    t.qmax = plans[i].qmax;
    auto flush = [&]() {
      if (t.n == 0) return;
      qdq_launch_chain(key, t, (unsigned)chunks, st);
      reset();
    };
    for (int64_t j = i; j < n; ++j) {
      // quantization range is part of the key: it follows from qk only for fp8, not for ints
      if (done[j] || !(plans[j].key == key) || plans[j].qmin != t.qmin || plans[j].qmax != t.qmax)
        continue;
      const uint64_t c = (uint64_t)cdiv(plans[j].job.g.nvec, per_chunk);
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
  return check_launch("ctmi_qdq_many");
}
