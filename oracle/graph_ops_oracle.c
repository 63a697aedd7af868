/*
 * CPU oracle for the sparse graph-primitive layer.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, what the reference's operators compute
 * (xiezhq-hermann/graphiler, src/ops).  It exists so the HIP kernels can be
 * checked against an independent implementation.  Only tests, the smoke check
 * and the benchmark's cpu_baseline leg may load it; the product never does.
 *
 * Conventions
 *   - graphs use the reference's container layout (include/dglgraph.h:54-74):
 *     int32 row pointer (N+1), int32 neighbour ids (E), int32 edge ids (E),
 *     int64 COO endpoints in edge-id order.
 *   - floating point inputs/outputs are fp32.  Reductions accumulate in fp64
 *     and round once, so the oracle is the "mathematical" answer the fp32 and
 *     bf16 device results are judged against.  Single fp32 operations
 *     (u_add_v, row copies) are done in fp32 and are bit-exact.
 *   - every function returns 0, or a negative code for bad arguments.
 *
 * Parity pinning: the reference ships no golden vectors for these operators, so
 * each function here is pinned by the CPU test-suite against closed forms and
 * library routines (scipy.sparse products, numpy fancy indexing,
 * scipy.special.softmax, per-type numpy matmul, brute-force Python loops on the
 * reference's two debug graphs).  Summation order of the reference's cuSPARSE /
 * cuBLAS calls is not recoverable offline: parity with those is "unpinned"
 * beyond the mathematical definition.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_OK 0
#define ORC_EINVAL (-1)

enum {
  ORC_OP_COPY_U = 0, ORC_OP_COPY_E = 1, ORC_OP_U_MUL_E = 2,
  ORC_OP_U_ADD_E = 3, ORC_OP_U_SUB_E = 4, ORC_OP_U_DIV_E = 5 /* functor.cuh:19-72 */
};
enum { ORC_RED_SUM = 0, ORC_RED_MAX = 1, ORC_RED_MIN = 2 };

int orc_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

void orc_set_num_threads(int n) {
#ifdef _OPENMP
  if (n > 0) omp_set_num_threads(n);
#else
  (void)n;
#endif
}

/*
 * Grouped adjacency from an edge list.
 * Follows python/graphiler/utils/setup.py:116-146 (prepare_graph): for every
 * node, its incident edges grouped together, `pointer` the running sum of the
 * degrees, `nbr` the other endpoint and `eid` the edge id.  Inside a group the
 * edges keep ascending edge-id order (stable grouping), which is the order the
 * reference's debug graph yields (setup.py:41-42).
 *   key   : endpoint the edges are grouped by (dst for the in-CSR, src for out)
 *   other : the opposite endpoint
 */
int orc_group_edges(int64_t n_nodes, int64_t n_edges, const int64_t *key,
                    const int64_t *other, int32_t *pointer, int32_t *nbr,
                    int32_t *eid) {
  if (n_nodes < 0 || n_edges < 0 || n_edges > INT32_MAX) return ORC_EINVAL;
  int64_t *cursor = (int64_t *)calloc((size_t)n_nodes + 1, sizeof(int64_t));
  if (!cursor) return ORC_EINVAL;
  for (int64_t e = 0; e < n_edges; ++e) {
    if (key[e] < 0 || key[e] >= n_nodes) {
      free(cursor);
      return ORC_EINVAL;
    }
    cursor[key[e] + 1]++;
  }
  for (int64_t v = 0; v < n_nodes; ++v) cursor[v + 1] += cursor[v];
  for (int64_t v = 0; v <= n_nodes; ++v) pointer[v] = (int32_t)cursor[v];
  for (int64_t e = 0; e < n_edges; ++e) {
    int64_t slot = cursor[key[e]]++;
    nbr[slot] = (int32_t)other[e];
    eid[slot] = (int32_t)e;
  }
  free(cursor);
  return ORC_OK;
}

/*
 * Type pointer: running sum of the number of items per type, for items whose
 * type ids are already non-decreasing (include/dglgraph.h:68-71;
 * setup.py:149-161 builds it with cumsum).  Returns ORC_EINVAL when the type
 * column is not sorted.
 */
int orc_type_pointer(int64_t n_items, int64_t n_types, const int64_t *type_of,
                     int32_t *pointer) {
  memset(pointer, 0, sizeof(int32_t) * (size_t)(n_types + 1));
  for (int64_t i = 0; i < n_items; ++i) {
    if (type_of[i] < 0 || type_of[i] >= n_types) return ORC_EINVAL;
    if (i > 0 && type_of[i] < type_of[i - 1]) return ORC_EINVAL;
    pointer[type_of[i] + 1]++;
  }
  for (int64_t t = 0; t < n_types; ++t) pointer[t + 1] += pointer[t];
  return ORC_OK;
}

/*
 * Generalised SpMM over a grouped adjacency.
 *   out[v, h, d] = reduce_{i in [ptr[v], ptr[v+1])} msg_i[h, d]
 *   msg_i = u[nbr[i]]                      (copy_u : spmm.cu:375-389 SpMMSrc)
 *         = e[eid[i]]                      (copy_e : spmm.cu:359-373 SpMMEdge)
 *         = u[nbr[i], h, d] * w[eid[i], h] (u_mul_e: spmm.cu:192-211, 286-356)
 * feat = heads * d_per_head.  The reference's u_mul_e has one scalar per edge
 * (heads == 1); heads > 1 is the multi-head generalisation with one scalar per
 * edge and head.  eid may be NULL, meaning eid[i] == i.
 * reduce: sum (empty group -> 0), max / min following functor.cuh:125-213:
 * start at -inf / +inf, strict comparison so the first extremum in group order
 * wins, an empty group keeps the start value.  arg_u / arg_e (may be NULL)
 * receive the neighbour id / edge id of the winning message per output element
 * (0 for an empty group, spmm.cuh:47).
 */
int orc_spmm(int64_t n_rows, const int32_t *ptr, const int32_t *nbr,
             const int32_t *eid, const float *u, const float *w, float *out,
             int32_t *arg_u, int32_t *arg_e, int64_t feat, int64_t heads,
             int op, int reduce) {
  if (feat <= 0 || heads <= 0 || feat % heads) return ORC_EINVAL;
  if (op < 0 || op > 5 || reduce < 0 || reduce > 2) return ORC_EINVAL;
  const int64_t dph = feat / heads;
#pragma omp parallel
  {
    double *acc = (double *)malloc(sizeof(double) * (size_t)feat);
#pragma omp for schedule(dynamic, 256)
    for (int64_t v = 0; v < n_rows; ++v) {
      const double start = reduce == ORC_RED_SUM
                               ? 0.0
                               : (reduce == ORC_RED_MAX ? -INFINITY : INFINITY);
      for (int64_t f = 0; f < feat; ++f) acc[f] = start;
      if (arg_u)
        for (int64_t f = 0; f < feat; ++f) arg_u[v * feat + f] = 0;
      if (arg_e)
        for (int64_t f = 0; f < feat; ++f) arg_e[v * feat + f] = 0;
      for (int32_t i = ptr[v]; i < ptr[v + 1]; ++i) {
        const int64_t e = eid ? eid[i] : i;
        const int64_t c = nbr ? nbr[i] : 0;
        for (int64_t f = 0; f < feat; ++f) {
          double m;
          if (op == ORC_OP_COPY_U)
            m = u[c * feat + f];
          else if (op == ORC_OP_COPY_E)
            m = u[e * feat + f];
          else if (op == ORC_OP_U_MUL_E)
            m = (double)u[c * feat + f] * (double)w[e * heads + f / dph];
          else if (op == ORC_OP_U_ADD_E)
            m = (double)u[c * feat + f] + (double)w[e * heads + f / dph];
          else if (op == ORC_OP_U_SUB_E)
            m = (double)u[c * feat + f] - (double)w[e * heads + f / dph];
          else
            m = (double)u[c * feat + f] / (double)w[e * heads + f / dph];
          if (reduce == ORC_RED_SUM) {
            acc[f] += m;
          } else if ((reduce == ORC_RED_MAX && acc[f] < m) ||
                     (reduce == ORC_RED_MIN && acc[f] > m)) {
            acc[f] = m;
            if (arg_u) arg_u[v * feat + f] = (int32_t)c;
            if (arg_e) arg_e[v * feat + f] = (int32_t)e;
          }
        }
      }
      for (int64_t f = 0; f < feat; ++f) out[v * feat + f] = (float)acc[f];
    }
    free(acc);
  }
  return ORC_OK;
}

/*
 * Same contraction as orc_spmm(sum) but accumulating in fp32 in group order,
 * one lane per feature, exactly like the reference's u_mul_e_sum_kernel
 * (spmm.cu:192-211).  Used as the timed CPU baseline and to show how far a
 * sequential fp32 sum sits from the fp64 answer.
 */
int orc_spmm_sum_f32(int64_t n_rows, const int32_t *ptr, const int32_t *nbr,
                     const int32_t *eid, const float *u, const float *w,
                     float *out, int64_t feat, int64_t heads, int op) {
  if (feat <= 0 || heads <= 0 || feat % heads) return ORC_EINVAL;
  const int64_t dph = feat / heads;
#pragma omp parallel for schedule(dynamic, 256)
  for (int64_t v = 0; v < n_rows; ++v) {
    float *o = out + v * feat;
    for (int64_t f = 0; f < feat; ++f) o[f] = 0.0f;
    for (int32_t i = ptr[v]; i < ptr[v + 1]; ++i) {
      const int64_t e = eid ? eid[i] : i;
      if (op == ORC_OP_COPY_U) {
        const float *x = u + (int64_t)nbr[i] * feat;
        for (int64_t f = 0; f < feat; ++f) o[f] += x[f];
      } else if (op == ORC_OP_COPY_E) {
        const float *x = u + e * feat;
        for (int64_t f = 0; f < feat; ++f) o[f] += x[f];
      } else {
        const float *x = u + (int64_t)nbr[i] * feat;
        const float *a = w + e * heads;
        for (int64_t f = 0; f < feat; ++f) o[f] += x[f] * a[f / dph];
      }
    }
  }
  return ORC_OK;
}

/*
 * SDDMM u_add_v in edge-id order: out[e, k] = u[src[e], k] + v[dst[e], k].
 * Follows sddmm.cu:118-129 (SDDMMCoo "add", lhs target 0 = source, rhs target
 * 2 = destination; sddmm.cuh:34-71).  The reference accepts and ignores alpha.
 */
int orc_sddmm_u_add_v(int64_t n_edges, const int64_t *src, const int64_t *dst,
                      const float *u, const float *v, float *out,
                      int64_t feat) {
  if (feat <= 0) return ORC_EINVAL;
#pragma omp parallel for schedule(static)
  for (int64_t e = 0; e < n_edges; ++e)
    for (int64_t k = 0; k < feat; ++k)
      out[e * feat + k] = u[src[e] * feat + k] + v[dst[e] * feat + k];
  return ORC_OK;
}

/*
 * The same with the other binary functors (functor.cuh:19-72): op 0 add, 1 sub,
 * 2 mul, 3 div; one fp32 operation per element, as SDDMMCooKernel computes it
 * (sddmm.cuh:34-71).
 */
int orc_sddmm_u_op_v(int64_t n_edges, const int64_t *src, const int64_t *dst,
                     const float *u, const float *v, float *out, int64_t feat,
                     int op) {
  if (feat <= 0 || op < 0 || op > 3) return ORC_EINVAL;
#pragma omp parallel for schedule(static)
  for (int64_t e = 0; e < n_edges; ++e)
    for (int64_t k = 0; k < feat; ++k) {
      const float a = u[src[e] * feat + k], b = v[dst[e] * feat + k];
      out[e * feat + k] = op == 0 ? a + b : op == 1 ? a - b : op == 2 ? a * b : a / b;
    }
  return ORC_OK;
}

/*
 * SDDMM u_dot_v: out[e, h] = sum_k u[src[e], h, k] * v[dst[e], h, k].
 * Follows the Dot functor (functor.cuh:103-116) with the reduction over the
 * last feature dimension (bcast.cc:37-39, 57-60).
 */
int orc_sddmm_u_dot_v(int64_t n_edges, const int64_t *src, const int64_t *dst,
                      const float *u, const float *v, float *out,
                      int64_t heads, int64_t dim) {
  if (heads <= 0 || dim <= 0) return ORC_EINVAL;
#pragma omp parallel for schedule(static)
  for (int64_t e = 0; e < n_edges; ++e)
    for (int64_t h = 0; h < heads; ++h) {
      const float *a = u + (src[e] * heads + h) * dim;
      const float *b = v + (dst[e] * heads + h) * dim;
      double s = 0.0;
      for (int64_t k = 0; k < dim; ++k) s += (double)a[k] * (double)b[k];
      out[e * heads + h] = (float)s;
    }
  return ORC_OK;
}

/*
 * Edge softmax over each destination's incoming edges, per head:
 *   y[e, h] = exp(x[e, h] - m) / sum_{e' in group} exp(x[e', h] - m)
 * with e ranging over eid[ptr[v] .. ptr[v+1]).  Follows
 * segment_softmax.cu:3-24 and segment_softmax_kernel.cu:4-49.
 * zero_floor != 0 reproduces the reference's choice m = max(0, max x) (its
 * running maximum starts at 0.0f, segment_softmax_kernel.cu:9) in fp32 with
 * expf; zero_floor == 0 uses the true maximum and fp64 arithmetic.  Edges that
 * belong to no group keep the value 0 (the reference's zeros_like output).
 * heads > 1 is the multi-head generalisation the reference leaves unimplemented.
 */
int orc_segment_softmax(int64_t n_rows, int64_t n_edges, const int32_t *ptr,
                        const int32_t *eid, const float *x, float *y,
                        int64_t heads, int zero_floor) {
  if (heads <= 0) return ORC_EINVAL;
  memset(y, 0, sizeof(float) * (size_t)(n_edges * heads));
#pragma omp parallel for schedule(dynamic, 256)
  for (int64_t v = 0; v < n_rows; ++v) {
    for (int64_t h = 0; h < heads; ++h) {
      if (zero_floor) {
        float m = 0.0f, s = 0.0f;
        for (int32_t i = ptr[v]; i < ptr[v + 1]; ++i) {
          const int64_t e = eid ? eid[i] : i;
          m = fmaxf(m, x[e * heads + h]);
        }
        for (int32_t i = ptr[v]; i < ptr[v + 1]; ++i) {
          const int64_t e = eid ? eid[i] : i;
          s += expf(x[e * heads + h] - m);
        }
        for (int32_t i = ptr[v]; i < ptr[v + 1]; ++i) {
          const int64_t e = eid ? eid[i] : i;
          y[e * heads + h] = expf(x[e * heads + h] - m) / s;
        }
      } else {
        double m = -INFINITY, s = 0.0;
        for (int32_t i = ptr[v]; i < ptr[v + 1]; ++i) {
          const int64_t e = eid ? eid[i] : i;
          if ((double)x[e * heads + h] > m) m = x[e * heads + h];
        }
        for (int32_t i = ptr[v]; i < ptr[v + 1]; ++i) {
          const int64_t e = eid ? eid[i] : i;
          s += exp((double)x[e * heads + h] - m);
        }
        for (int32_t i = ptr[v]; i < ptr[v + 1]; ++i) {
          const int64_t e = eid ? eid[i] : i;
          y[e * heads + h] = (float)(exp((double)x[e * heads + h] - m) / s);
        }
      }
    }
  }
  return ORC_OK;
}

/*
 * Typed linear: rows are sorted by type, type t owns rows [tp[t], tp[t+1]);
 *   Y[r, h, :] = X[r, h, :] @ W[t, h, :, :]      X (rows, heads, K)
 *                                                W (T, heads, K, M)
 * heads == 1 is the reference's SegmentMMBase (segment_mm.cu:4-21): a loop of
 * per-type matrix products concatenated in type order.  heads > 1 applies an
 * independent K x M block per head (block-diagonal typed linear).  Rows outside
 * [tp[0], tp[T]) are not written by the reference (its output only has
 * tp[T]-tp[0] rows); here tp[0] must be 0 and Y has tp[T] rows.
 */
int orc_segment_mm(int64_t n_types, const int32_t *tp, const float *X,
                   const float *W, float *Y, int64_t heads, int64_t K,
                   int64_t M) {
  if (heads <= 0 || K <= 0 || M <= 0 || n_types < 0) return ORC_EINVAL;
  if (n_types > 0 && tp[0] != 0) return ORC_EINVAL;
  for (int64_t t = 0; t < n_types; ++t) {
    if (tp[t + 1] < tp[t]) return ORC_EINVAL;
    const float *Wt = W + t * heads * K * M;
#pragma omp parallel
    {
      double *acc = (double *)malloc(sizeof(double) * (size_t)M);
#pragma omp for schedule(static)
      for (int64_t r = tp[t]; r < tp[t + 1]; ++r)
        for (int64_t h = 0; h < heads; ++h) {
          const float *x = X + (r * heads + h) * K;
          const float *w = Wt + h * K * M;
          for (int64_t m = 0; m < M; ++m) acc[m] = 0.0;
          for (int64_t k = 0; k < K; ++k) {
            const double xv = x[k];
            for (int64_t m = 0; m < M; ++m) acc[m] += xv * (double)w[k * M + m];
          }
          float *y = Y + (r * heads + h) * M;
          for (int64_t m = 0; m < M; ++m) y[m] = (float)acc[m];
        }
      free(acc);
    }
  }
  return ORC_OK;
}

/* fp32-accumulating typed linear (timed CPU baseline; same loop nest). */
int orc_segment_mm_f32(int64_t n_types, const int32_t *tp, const float *X,
                       const float *W, float *Y, int64_t heads, int64_t K,
                       int64_t M) {
  if (heads <= 0 || K <= 0 || M <= 0 || n_types < 0) return ORC_EINVAL;
  for (int64_t t = 0; t < n_types; ++t) {
    const float *Wt = W + t * heads * K * M;
#pragma omp parallel for schedule(static)
    for (int64_t r = tp[t]; r < tp[t + 1]; ++r)
      for (int64_t h = 0; h < heads; ++h) {
        const float *x = X + (r * heads + h) * K;
        const float *w = Wt + h * K * M;
        float *y = Y + (r * heads + h) * M;
        for (int64_t m = 0; m < M; ++m) y[m] = 0.0f;
        for (int64_t k = 0; k < K; ++k) {
          const float xv = x[k];
          for (int64_t m = 0; m < M; ++m) y[m] += xv * w[k * M + m];
        }
      }
  }
  return ORC_OK;
}

/*
 * Row gather y[i, :] = x[idx[i], :] on raw bytes (any dtype), the reference's
 * Broadcast* operators (broadcast.cu:58-100: features.index({COO_src | COO_dst
 * | ntype_COO | etype_COO})).  Out-of-range indices are rejected.
 */
int orc_gather_rows(int64_t n_out, int64_t n_in, const int64_t *idx,
                    const void *x, void *y, int64_t row_bytes) {
  if (row_bytes < 0) return ORC_EINVAL;
  for (int64_t i = 0; i < n_out; ++i)
    if (idx[i] < 0 || idx[i] >= n_in) return ORC_EINVAL;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n_out; ++i)
    memcpy((char *)y + i * row_bytes, (const char *)x + idx[i] * row_bytes,
           (size_t)row_bytes);
  return ORC_OK;
}

/*
 * One GAT attention + aggregation pass, the operator chain the reference's
 * optimised plan runs for examples/GAT/GAT.py:25-36 (fusion.cpp:37-47, 67-77):
 *   s_i   = leaky_relu(el[nbr[i], h] + er[v, h], slope)
 *   a_i   = softmax over the group of v
 *   out[v, h, :] = sum_i a_i * z[nbr[i], h, :]
 * fp64 throughout, rounded once.  Rows with no in-edges produce 0.
 */
int orc_gat_aggregate(int64_t n_rows, const int32_t *ptr, const int32_t *nbr,
                      const float *el, const float *er, const float *z,
                      float *out, int64_t heads, int64_t dim, double slope) {
  if (heads <= 0 || dim <= 0) return ORC_EINVAL;
  const int64_t feat = heads * dim;
#pragma omp parallel
  {
    double *acc = (double *)malloc(sizeof(double) * (size_t)dim);
#pragma omp for schedule(dynamic, 256)
    for (int64_t v = 0; v < n_rows; ++v)
      for (int64_t h = 0; h < heads; ++h) {
        double m = -INFINITY, s = 0.0;
        for (int32_t i = ptr[v]; i < ptr[v + 1]; ++i) {
          /* the logit itself is one fp32 add, as in orc_sddmm_u_add_v */
          float t = el[(int64_t)nbr[i] * heads + h] + er[v * heads + h];
          double q = t >= 0.0f ? (double)t : (double)t * slope;
          if (q > m) m = q;
        }
        for (int64_t d = 0; d < dim; ++d) acc[d] = 0.0;
        for (int32_t i = ptr[v]; i < ptr[v + 1]; ++i) {
          float t = el[(int64_t)nbr[i] * heads + h] + er[v * heads + h];
          double q = t >= 0.0f ? (double)t : (double)t * slope;
          double p = exp(q - m);
          s += p;
          const float *zr = z + (int64_t)nbr[i] * feat + h * dim;
          for (int64_t d = 0; d < dim; ++d) acc[d] += p * (double)zr[d];
        }
        float *o = out + v * feat + h * dim;
        for (int64_t d = 0; d < dim; ++d)
          o[d] = ptr[v + 1] > ptr[v] ? (float)(acc[d] / s) : 0.0f;
      }
    free(acc);
  }
  return ORC_OK;
}
