// Chained launches: one kernel launch that covers several tensors.
//
// A kernel start costs about 3 us on this GPU (dispatch ramp and drain), as much
// as streaming a 1024 x 4096 bf16 weight, so the streaming kernels take up to
// kMaxJobs tensors per launch.  The job table travels in the kernel arguments; a
// workgroup finds its tensor by a scan over the running chunk counts, all on
// wave-uniform values.
#pragma once

#include <cstddef>

#include "ctmi_device.h"
#include "vec_geom.h"

namespace ctmi {

constexpr int kMaxJobs = 8;

struct VecJob {
  const void* src;
  void* dst;
  const void* scale;
  const int8_t* zp;
  VecGeom g;
};

// What a workgroup needs of its weight, 64 bytes so that one scalar load brings
// it in.  Scale of item v (8 elements): `v >> shift` when scales are numbered
// like the items (FLAT), else row r = v / vpr, column block (v - r*vpr) / vpb,
// index (r >> row_shift) * s_stride + block (s_stride 0 when all rows share one
// scale row; row_shift > 0 for blocks several rows tall).
struct alignas(64) ChainJob {
  const void* src;
  void* dst;
  const void* scale;
  const int8_t* zp;
  uint32_t shift, row_shift;
  uint32_t vpr_d, vpr_m, vpr_s;
  uint32_t vpb_m, vpb_s;
  uint32_t s_stride;
};
static_assert(sizeof(ChainJob) == 64, "one scalar load per job");

// Kernel argument of a chained launch.  What decides which job a workgroup
// belongs to and whether a lane has work comes first, in one scalar load; unused
// chunk_end entries hold 0xFFFFFFFF.
struct ChainTable {
  uint32_t chunk_end[kMaxJobs];  // running total of chunks, job 0 .. j
  uint32_t nvec[kMaxJobs];       // items of job j
  ChainJob job[kMaxJobs];
  float qmin, qmax;
  int32_t n;
};

static inline bool flat_geometry(const VecGeom& g) { return g.mode == 0; }

static inline ChainJob make_chain_job(const VecJob& j) {
  ChainJob o;
  o.src = j.src;
  o.dst = j.dst;
  o.scale = j.scale;
  o.zp = j.zp;
  o.shift = j.g.shift;
  o.row_shift = j.g.row_shift;
  o.vpr_d = j.g.vpr.d;
  o.vpr_m = j.g.vpr.m;
  o.vpr_s = j.g.vpr.s;
  o.vpb_m = j.g.vpb.m;
  o.vpb_s = j.g.vpb.s;
  o.s_stride = j.g.row_scaled ? j.g.s_cols : 0u;
  return o;
}

static_assert(kMaxJobs == 8 && offsetof(ChainTable, chunk_end) == 0 &&
                  offsetof(ChainTable, nvec) == 32,
              "find_job reads chunk_end and nvec as the first 16 dwords of the kernel argument");

// The job of workgroup `chunk` (its index), the chunk's number within that job and the
// job's item count, for any table that is the kernel's only argument and starts with
// chunk_end[8] and the item counts [8].  This head is fetched with one 64-byte scalar
// load written out by hand: left to itself the compiler turns the search into a chain of
// dependent loads, and a wave of these kernels lives too short to hide several scalar
// round trips.  The search itself is then compares and selects on registers.
__device__ __forceinline__ uint32_t find_job_index(uint32_t chunk, uint32_t* local, uint32_t* nvec) {
  typedef uint32_t u32x16 __attribute__((ext_vector_type(16)));
  u32x16 head;
  asm volatile("s_load_dwordx16 %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)"
               : "=s"(head)
               : "s"(__builtin_amdgcn_kernarg_segment_ptr()));
  uint32_t j = 0, first = 0, nv = head[8];
#pragma unroll
  for (int i = 0; i < kMaxJobs - 1; ++i) {
    const uint32_t e = head[i];
    const bool past = chunk >= e;
    j = past ? (uint32_t)(i + 1) : j;  // chunk_end ascends: the last hit wins
    first = past ? e : first;
    nv = past ? head[9 + i] : nv;
  }
  *local = chunk - first;
  *nvec = nv;
  return j;
}

// ... and the job's 64 bytes, one more batch of scalar loads
__device__ __forceinline__ ChainJob find_job(const ChainTable& t, uint32_t chunk, uint32_t* local,
                                          uint32_t* nvec) {
  return t.job[find_job_index(chunk, local, nvec)];
}

template <bool FLAT>
__device__ __forceinline__ uint32_t chain_scale_index(uint32_t v, const ChainJob& job) {
  if constexpr (FLAT) {
    return v >> job.shift;
  } else {
    const uint32_t r = (uint32_t)(((uint64_t)v * job.vpr_m) >> 31) >> job.vpr_s;
    const uint32_t cv = v - r * job.vpr_d;
    return (r >> job.row_shift) * job.s_stride +
           ((uint32_t)(((uint64_t)cv * job.vpb_m) >> 31) >> job.vpb_s);
  }
}

}  // namespace ctmi
