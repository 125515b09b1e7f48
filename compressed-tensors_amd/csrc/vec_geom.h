// Geometry shared by the vectorised streaming kernels: a work item is 8
// neighbouring elements of one row that share one scale; items are numbered
// row-major and mapped to their scale with two invariant-divisor divisions.
#pragma once

#include "ctmi_device.h"
#include "ctmi_host.h"

namespace ctmi {

// 32-bit division by an invariant divisor: q = (n * m) >> (31 + s), exact for
// n < 2^31 and 1 <= d < 2^31.
struct FastDiv {
  uint32_t d, m, s;
};
static inline FastDiv make_fastdiv(uint32_t d) {
  FastDiv f;
  f.d = d;
  uint32_t s = 0;
  while ((1ull << s) < d) ++s;
  f.s = s;
  f.m = (uint32_t)(((1ull << (31 + s)) + d - 1) / d);
  return f;
}
__device__ __forceinline__ uint32_t fdiv(uint32_t n, const FastDiv& f) {
  return (uint32_t)(((uint64_t)n * f.m) >> 31) >> f.s;
}

struct VecGeom {
  FastDiv vpr;        // items per row
  FastDiv vpb;        // items per scale block (blk_cols / 8)
  uint32_t nvec;      // total items
  uint32_t s_cols;
  uint32_t row_scaled;  // 1: scale row = tensor row >> row_shift; 0: a single scale row
  uint32_t row_shift;   // log2 of the rows that share a scale row (blocks: 2^k rows tall)
  // When every row has its own scales and scale blocks tile the rows exactly,
  // scales are numbered like the items: index = item / vpb, a shift if vpb is a
  // power of two.  mode 0: shift, 1: one division, 2: row/column split.
  uint32_t mode, shift;
};

__device__ __forceinline__ uint32_t scale_index(uint32_t v, const VecGeom& g) {
  if (g.mode == 0) return v >> g.shift;
  if (g.mode == 1) return fdiv(v, g.vpb);
  const uint32_t r = fdiv(v, g.vpr);
  const uint32_t cv = v - r * g.vpr.d;
  return (g.row_scaled ? (r >> g.row_shift) * g.s_cols : 0u) + fdiv(cv, g.vpb);
}

template <int A, int B>
struct Promote {
  static constexpr int value = (A == B) ? A : CTMI_F32;
};

constexpr int kU = 4;

static inline int grid_for(int64_t work_items, int per_block) {
  int64_t b = cdiv(work_items, per_block);
  const int64_t cap = 256 * 16;  // 16 resident workgroups per CU is plenty for streaming
  if (b > cap) b = cap;
  if (b < 1) b = 1;
  return (int)b;
}

// Can the vectorised kernels take this problem?
static inline bool vec_geometry(const ctmi_qparams* qp, int64_t rows, int64_t cols, VecGeom* g,
                                bool allow_gscale = false) {
  if (qp->col_group || (qp->global_scale && !allow_gscale)) return false;
  if (cols % 8 || qp->blk_cols % 8) return false;
  if (rows * cols / 8 >= (1ll << 31) || cols / 8 < 1) return false;
  if (cols % qp->blk_cols) return false;
  const bool single_row = (qp->s_rows == 1 && qp->blk_rows >= rows);
  // every row its own scales, or blocks a power of two rows tall
  const bool pow2_rows = qp->blk_rows >= 1 && (qp->blk_rows & (qp->blk_rows - 1)) == 0;
  const bool row_scaled = pow2_rows && qp->s_rows == cdiv(rows, qp->blk_rows);
  if (!row_scaled && !single_row) return false;
  if (qp->s_cols >= (1ll << 31) || rows * qp->s_cols >= (1ll << 31)) return false;
  g->vpr = make_fastdiv((uint32_t)(cols / 8));
  g->vpb = make_fastdiv((uint32_t)(qp->blk_cols / 8));
  g->nvec = (uint32_t)(rows * cols / 8);
  g->s_cols = (uint32_t)qp->s_cols;
  g->row_scaled = row_scaled ? 1u : 0u;
  g->row_shift = 0;
  if (row_scaled)
    while ((1ll << g->row_shift) < qp->blk_rows) ++g->row_shift;
  g->mode = 2;
  g->shift = 0;
  if (row_scaled && g->row_shift == 0 && g->vpr.d % g->vpb.d == 0 &&
      qp->s_cols == cols / qp->blk_cols) {
    const uint32_t d = g->vpb.d;
    if ((d & (d - 1)) == 0) {
      g->mode = 0;
      while ((1u << g->shift) < d) ++g->shift;
    } else {
      g->mode = 1;
    }
  } else if (single_row && qp->s_cols == 1) {
    g->mode = 0;  // one scale for everything: items are < 2^31, so the index is 0
    g->shift = 31;
  }
  return true;
}


}  // namespace ctmi
