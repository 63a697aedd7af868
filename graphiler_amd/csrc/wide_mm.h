// Typed GEMM for wide bf16 outputs on gfx950 (wide_mm.hip): one pass over the rows of
// X for several groups of 128 output columns.
#pragma once
#include "common.h"

namespace ga {

constexpr int kWideGroupCols = 128;   // columns of a group
constexpr int kWideMaxGroups = 4;

// Y_g[r, 0:128] = X[r, :] @ W_g[type(r)][:, 0:128] for every group g.  The groups may
// be column ranges of one weight tensor (pointers 128 columns apart, the same strides)
// or different tensors (stacked projections of the same rows).
struct WideMm {
  const int32_t *tp;          // type pointer over the rows, or null: one type
  int n_types;
  int64_t rows;
  const bf16_t *X;            // (rows, K), rows K elements apart
  int K;                      // multiple of 8 up to 256, or of 4 up to 128 (two groups at most)
  int n_groups;
  const bf16_t *W[kWideMaxGroups];      // first column of the group in W[type 0]
  int64_t w_type_stride[kWideMaxGroups];
  int64_t ldw[kWideMaxGroups];          // elements between rows k and k + 1
  bf16_t *Y[kWideMaxGroups];            // first column of the group in row 0
  int64_t ldy[kWideMaxGroups];
  // attention terms (all null: none): el / er[r, head] = <Y[r, head, :], a_l / a_r[head, :]>
  // on the fp32 accumulators; a_l / a_r / el / er point at the group's first column / head
  const float *a_l[kWideMaxGroups], *a_r[kWideMaxGroups];
  float *el[kWideMaxGroups], *er[kWideMaxGroups];
  const float *row_scale;     // Y[r, :] of every group times row_scale[r]; null: 1 (not with a_l / a_r)
  const float *type_gate;     // Y[r, :] times g(type_gate[type(r)]); null: 1 (not with a_l / a_r)
  bool gate_sigmoid;          // g = 1 / (1 + exp(-x)) instead of the identity
  int64_t ldd;                // heads per row of el / er
  int dph;                    // columns per head: 32, 64 or 128
  bool w_wide;                // set by wide_mm_launch: rows of every W are 16-byte aligned
};

// True when the kernel takes this shape (the caller still checks pointers).
bool wide_mm_fits(int K, int n_groups);
// GA_OK, GA_EUNSUPPORTED (shape or alignment outside the kernel) or a launch error.
int wide_mm_launch(const WideMm &p, hipStream_t s);

}  // namespace ga
