// General forms of the two binary graph operators: operands whose feature shapes
// broadcast against each other (numpy rules over the dimensions after the first)
// and, for SDDMM, operands that live on the source nodes, on the edges or on the
// destination nodes in any combination.
//
// These are the UseBcast = true instantiations of the reference's generic kernels
// (SpMMCsrKernel, spmm.cuh:30-71; SDDMMCooKernel and the dot-product kernel,
// sddmm.cuh:34-120, operand selection selector.h:30-60), which consume the offset
// tables of CalcBcastOff (bcast.cc:19-71): output element k of a row or an edge is
// op(lhs[lhs_off[k]], rhs[rhs_off[k]]).  The shapes the benchmark models use never
// broadcast (one value per head at most) and run on the specialised kernels of
// spmm.hip / edge_ops.hip; this file is the general path behind them: one thread
// per output element, edges of a row folded in adjacency order (so sums are
// deterministic and max / min report the first extremum, functor.cuh:148-213).
#include "common.h"

namespace ga {
namespace {

__device__ __forceinline__ float binary(int op, float a, float b) {
  switch (op) {
    case GA_BCAST_SUB: return a - b;
    case GA_BCAST_MUL: return a * b;
    case GA_BCAST_DIV: return a / b;
    case GA_BCAST_COPY_LHS: return a;
    case GA_BCAST_COPY_RHS: return b;
    default: return a + b;
  }
}

__global__ __launch_bounds__(kBlock) void spmm_bcast_kernel(
    const int32_t *__restrict__ pointer, const int32_t *__restrict__ nbr,
    const int32_t *__restrict__ eid, const float *__restrict__ u, const float *__restrict__ w,
    float *__restrict__ out, int32_t *__restrict__ arg_u, int32_t *__restrict__ arg_e,
    int64_t n_rows, const int64_t *__restrict__ u_off, const int64_t *__restrict__ w_off,
    int64_t u_len, int64_t w_len, int64_t out_len, int op, int reduce) {
  const int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (t >= n_rows * out_len) return;
  const int64_t row = t / out_len, k = t - row * out_len;
  const int64_t ua = u_off ? u_off[k] : k, wa = w_off ? w_off[k] : k;
  const bool use_u = op != GA_BCAST_COPY_RHS, use_w = op != GA_BCAST_COPY_LHS;
  float acc = reduce == GA_SUM ? 0.0f : (reduce == GA_MAX ? -INFINITY : INFINITY);
  int best_u = 0, best_e = 0;
  for (int32_t i = pointer[row]; i < pointer[row + 1]; ++i) {
    const int32_t c = nbr[i], e = eid ? eid[i] : i;
    const float a = use_u ? u[(int64_t)c * u_len + ua] : 0.0f;
    const float b = use_w ? w[(int64_t)e * w_len + wa] : 0.0f;
    const float m = binary(op, a, b);
    if (reduce == GA_SUM) {
      acc += m;
    } else if (reduce == GA_MAX ? acc < m : acc > m) {   // strict: the first extremum stays
      acc = m;
      best_u = c;
      best_e = e;
    }
  }
  out[t] = acc;
  if (arg_u) arg_u[t] = best_u;
  if (arg_e) arg_e[t] = best_e;
}

__device__ __forceinline__ int64_t pick(int target, int64_t src, int64_t edge, int64_t dst) {
  return target == 0 ? src : (target == 1 ? edge : dst);
}

__global__ __launch_bounds__(kBlock) void sddmm_bcast_kernel(
    const int64_t *__restrict__ src, const int64_t *__restrict__ dst,
    const float *__restrict__ lhs, const float *__restrict__ rhs, float *__restrict__ out,
    int64_t n_edges, int lhs_target, int rhs_target, const int64_t *__restrict__ lhs_off,
    const int64_t *__restrict__ rhs_off, int64_t lhs_len, int64_t rhs_len, int64_t out_len,
    int64_t reduce_size, int op) {
  const int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (t >= n_edges * out_len) return;
  const int64_t e = t / out_len, k = t - e * out_len;
  const int64_t s = src[e], d = dst[e];
  const int64_t la = (lhs_off ? lhs_off[k] : k) * reduce_size;
  const int64_t ra = (rhs_off ? rhs_off[k] : k) * reduce_size;
  const float *lp = lhs + pick(lhs_target, s, e, d) * lhs_len + la;
  const float *rp = rhs + pick(rhs_target, s, e, d) * rhs_len + ra;
  if (op == GA_BCAST_DOT) {
    float acc = 0.0f;
    for (int64_t j = 0; j < reduce_size; ++j) acc = fmaf(lp[j], rp[j], acc);
    out[t] = acc;
  } else {
    out[t] = binary(op, op == GA_BCAST_COPY_RHS ? 0.0f : lp[0], op == GA_BCAST_COPY_LHS ? 0.0f : rp[0]);
  }
}

}  // namespace
}  // namespace ga

extern "C" {

int ga_spmm_csr_bcast(const int32_t *pointer, const int32_t *nbr, const int32_t *eid,
                      const float *u, const float *w, float *out, int32_t *arg_u,
                      int32_t *arg_e, int64_t n_rows, int64_t n_edges, const int64_t *u_off,
                      const int64_t *w_off, int64_t u_len, int64_t w_len, int64_t out_len,
                      int op, int reduce, ga_stream_t stream) {
  using namespace ga;
  if (n_rows < 0 || n_edges < 0 || n_rows > 0x7fffffff || n_edges > 0x7fffffff) return GA_EINVAL;
  if (u_len <= 0 || w_len <= 0 || out_len <= 0) return GA_EINVAL;
  if (op < GA_BCAST_ADD || op > GA_BCAST_COPY_RHS) return GA_EINVAL;
  if (reduce != GA_SUM && reduce != GA_MAX && reduce != GA_MIN) return GA_EINVAL;
  if ((arg_u || arg_e) && reduce == GA_SUM) return GA_EINVAL;
  if (n_rows == 0) return GA_OK;
  if (!pointer || !out) return GA_EINVAL;
  const bool use_u = op != GA_BCAST_COPY_RHS, use_w = op != GA_BCAST_COPY_LHS;
  if (n_edges > 0 && (!nbr || (use_u && !u) || (use_w && !w))) return GA_EINVAL;
  if (!aligned(out, 4) || (u && !aligned(u, 4)) || (w && !aligned(w, 4)) ||
      (u_off && !aligned(u_off, 8)) || (w_off && !aligned(w_off, 8)))
    return GA_EALIGN;
  const int64_t blocks = (n_rows * out_len + kBlock - 1) / kBlock;
  if (blocks > 0x7fffffff) return GA_EUNSUPPORTED;
  hipLaunchKernelGGL(spmm_bcast_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, (hipStream_t)stream,
                     pointer, nbr, eid, u, w, out, arg_u, arg_e, n_rows, u_off, w_off, u_len, w_len,
                     out_len, op, reduce);
  return launch_status();
}

int ga_sddmm_bcast(const int64_t *src, const int64_t *dst, const float *lhs, const float *rhs,
                   float *out, int64_t n_edges, int lhs_target, int rhs_target,
                   const int64_t *lhs_off, const int64_t *rhs_off, int64_t lhs_len,
                   int64_t rhs_len, int64_t out_len, int64_t reduce_size, int op,
                   ga_stream_t stream) {
  using namespace ga;
  if (n_edges < 0 || n_edges > 0x7fffffff) return GA_EINVAL;
  if (lhs_len <= 0 || rhs_len <= 0 || out_len <= 0 || reduce_size <= 0) return GA_EINVAL;
  if (op < GA_BCAST_ADD || op > GA_BCAST_DOT) return GA_EINVAL;
  if (reduce_size != 1 && op != GA_BCAST_DOT) return GA_EINVAL;
  if (lhs_target < 0 || lhs_target > 2 || rhs_target < 0 || rhs_target > 2) return GA_EINVAL;
  if (n_edges == 0) return GA_OK;
  if (!src || !dst || !lhs || !rhs || !out) return GA_EINVAL;
  if (!aligned(src, 8) || !aligned(dst, 8) || !aligned(lhs, 4) || !aligned(rhs, 4) ||
      !aligned(out, 4) || (lhs_off && !aligned(lhs_off, 8)) || (rhs_off && !aligned(rhs_off, 8)))
    return GA_EALIGN;
  const int64_t blocks = (n_edges * out_len + kBlock - 1) / kBlock;
  if (blocks > 0x7fffffff) return GA_EUNSUPPORTED;
  hipLaunchKernelGGL(sddmm_bcast_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, (hipStream_t)stream,
                     src, dst, lhs, rhs, out, n_edges, lhs_target, rhs_target, lhs_off, rhs_off,
                     lhs_len, rhs_len, out_len, reduce_size, op);
  return launch_status();
}

}  // extern "C"
