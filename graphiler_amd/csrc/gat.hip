// Fused GAT aggregation for gfx950: u_add_v -> leaky_relu -> edge softmax ->
// u_mul_e sum in one pass over the in-adjacency, nothing per-edge materialised.
//
// Same run-based schedule as the SpMM (equal runs of slots, one lane group per
// run, rows shared between runs combined by a second kernel), with an online
// softmax state per lane: running maximum m, running denominator l and the
// un-normalised weighted sum acc.  Two states merge as
//   M = max(m1, m2); l = l1 e^(m1-M) + l2 e^(m2-M); acc likewise,
// so partial rows combine exactly like partial sums, in run order.
#include "common.h"

namespace ga {
namespace {

constexpr int kUnroll = 8;

__device__ __forceinline__ float leaky(float t, float slope) {
  return t >= 0.0f ? t : t * slope;
}

template <typename T, int VEC>
__global__ __launch_bounds__(kBlock) void gat_runs_kernel(
    const int32_t *__restrict__ row_of_slot, const int32_t *__restrict__ nbr,
    const float *__restrict__ el, const float *__restrict__ er,
    const T *__restrict__ z, T *__restrict__ out, float *__restrict__ pacc,
    float *__restrict__ pml, int64_t n_edges, int64_t n_runs, int feat,
    int heads, int dph, float slope, int run_shift, int tpr_shift) {
  typedef Frag<T, VEC> IO;
  const int tpr = 1 << tpr_shift;
  const int64_t k = ((int64_t)blockIdx.x * kBlock + threadIdx.x) >> tpr_shift;
  const int f0 = ((int)blockIdx.y * tpr + (threadIdx.x & (tpr - 1))) * VEC;
  if (k >= n_runs || f0 >= feat) return;
  const int h = f0 / dph;
  const bool head_leader = f0 == h * dph;

  const int64_t a = k << run_shift;
  const int64_t b = min(a + ((int64_t)1 << run_shift), n_edges);

  int cur = row_of_slot[a];
  const bool began_before = a > 0 && row_of_slot[a - 1] == cur;
  bool first_seg = true;

  float m = -INFINITY, l = 0.0f;
  float acc[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) acc[v] = 0.0f;

  auto flush = [&](bool to_partial, int slot) {
    if (to_partial) {
      float *p = pacc + (k * 2 + slot) * feat + f0;
#pragma unroll
      for (int v = 0; v < VEC; ++v) p[v] = acc[v];
      if (head_leader) {
        float *q = pml + ((k * 2 + slot) * heads + h) * 2;
        q[0] = m;
        q[1] = l;
      }
    } else {
      const float inv = 1.0f / l;
      float o[VEC];
#pragma unroll
      for (int v = 0; v < VEC; ++v) o[v] = acc[v] * inv;
      IO::store(out + (int64_t)cur * feat + f0, o);
    }
  };

  for (int64_t j = a; j < b; j += kUnroll) {
    int r[kUnroll];
    int64_t g[kUnroll];
    float s[kUnroll];
    typename IO::raw_t x[kUnroll];
#pragma unroll
    for (int t = 0; t < kUnroll; ++t) {
      const int64_t jj = j + t < b ? j + t : b - 1;
      r[t] = row_of_slot[jj];
      g[t] = nbr[jj];
    }
#pragma unroll
    for (int t = 0; t < kUnroll; ++t) {
      x[t] = IO::load(z + g[t] * feat + f0);
      s[t] = leaky(el[g[t] * heads + h] + er[(int64_t)r[t] * heads + h], slope);
    }
    if (j + kUnroll <= b && r[0] == cur && r[kUnroll - 1] == cur) {
      // whole batch inside the open row (rows are sorted): one rescale
      float bm = s[0];
#pragma unroll
      for (int t = 1; t < kUnroll; ++t) bm = fmaxf(bm, s[t]);
      const float nm = fmaxf(m, bm);
      const float sc = __expf(m - nm);
      l *= sc;
#pragma unroll
      for (int v = 0; v < VEC; ++v) acc[v] *= sc;
      m = nm;
#pragma unroll
      for (int t = 0; t < kUnroll; ++t) {
        const float p = __expf(s[t] - nm);
        l += p;
        float xf[VEC];
        IO::widen(x[t], xf);
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[v] = fmaf(p, xf[v], acc[v]);
      }
    } else {
#pragma unroll
      for (int t = 0; t < kUnroll; ++t) {
        if (j + t < b) {
          if (r[t] != cur) {
            flush(first_seg && began_before, 0);
            first_seg = false;
            cur = r[t];
            m = -INFINITY;
            l = 0.0f;
#pragma unroll
            for (int v = 0; v < VEC; ++v) acc[v] = 0.0f;
          }
          const float nm = fmaxf(m, s[t]);
          const float sc = __expf(m - nm);
          const float p = __expf(s[t] - nm);
          l = l * sc + p;
          float xf[VEC];
          IO::widen(x[t], xf);
#pragma unroll
          for (int v = 0; v < VEC; ++v) acc[v] = fmaf(p, xf[v], acc[v] * sc);
          m = nm;
        }
      }
    }
  }
  const bool continues = b < n_edges && row_of_slot[b] == cur;
  if (first_seg)
    flush(began_before || continues, 0);
  else
    flush(continues, 1);
}

template <typename T, int VEC>
__global__ __launch_bounds__(kBlock) void gat_fixup_kernel(
    const int32_t *__restrict__ pointer, const int32_t *__restrict__ row_of_slot,
    const float *__restrict__ pacc, const float *__restrict__ pml,
    T *__restrict__ out, int64_t n_rows, int64_t n_edges, int64_t n_runs,
    int feat, int heads, int dph, int run_shift, int tpr_shift, int fix_blocks) {
  typedef Frag<T, VEC> IO;
  const int tpr = 1 << tpr_shift;
  const int f0 = ((int)blockIdx.y * tpr + (threadIdx.x & (tpr - 1))) * VEC;
  if (f0 >= feat) return;
  const int h = f0 / dph;
  float acc[VEC];
  if ((int)blockIdx.x < fix_blocks) {
    const int64_t k = ((int64_t)blockIdx.x * kBlock + threadIdx.x) >> tpr_shift;
    if (k >= n_runs) return;
    const int64_t a = k << run_shift;
    const int64_t b = min(a + ((int64_t)1 << run_shift), n_edges);
    const int row = row_of_slot[a];
    const int64_t s = pointer[row], e = pointer[row + 1];
    if (!(s < a && e <= b)) return;
    const int64_t k_lo = s >> run_shift;
    const int64_t first = k_lo * 2 + ((s == (k_lo << run_shift)) ? 0 : 1);
    const float *p = pacc + first * feat + f0;
    float m = pml[(first * heads + h) * 2], l = pml[(first * heads + h) * 2 + 1];
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = p[v];
    for (int64_t q = k_lo + 1; q <= k; ++q) {
      const float *pq = pacc + (q * 2) * feat + f0;
      const float mq = pml[((q * 2) * heads + h) * 2];
      const float lq = pml[((q * 2) * heads + h) * 2 + 1];
      const float nm = fmaxf(m, mq);
      const float sa = __expf(m - nm), sb = __expf(mq - nm);
      l = l * sa + lq * sb;
#pragma unroll
      for (int v = 0; v < VEC; ++v) acc[v] = acc[v] * sa + pq[v] * sb;
      m = nm;
    }
    const float inv = 1.0f / l;
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] *= inv;
    IO::store(out + (int64_t)row * feat + f0, acc);
  } else {
    const int64_t row =
        ((int64_t)(blockIdx.x - fix_blocks) * kBlock + threadIdx.x) >> tpr_shift;
    if (row >= n_rows || pointer[row] != pointer[row + 1]) return;
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = 0.0f;
    IO::store(out + row * feat + f0, acc);
  }
}

template <typename T, int VEC>
int launch_gat(const int32_t *pointer, const int32_t *row_of_slot,
               const int32_t *nbr, const float *el, const float *er,
               const void *z, void *out, int64_t n_rows, int64_t n_edges,
               int heads, int dim, float slope, float *ws, hipStream_t stream) {
  const int feat = heads * dim;
  const int lanes = (feat + VEC - 1) / VEC;
  const int tpr_shift = ilog2_ceil((uint64_t)(lanes > kWave ? kWave : lanes));
  const int tpr = 1 << tpr_shift;
  const int ftiles = (lanes + tpr - 1) / tpr;
  const int run_shift = run_shift_for(n_edges, feat);
  const int64_t n_runs = (n_edges + ((int64_t)1 << run_shift) - 1) >> run_shift;
  const int groups_per_block = kBlock >> tpr_shift;
  float *pacc = ws;
  float *pml = ws + n_runs * 2 * feat;
  const int64_t fix_blocks = (n_runs + groups_per_block - 1) / groups_per_block;
  const int64_t fill_blocks = (n_rows + groups_per_block - 1) / groups_per_block;
  if (fix_blocks + fill_blocks > 0x7fffffff) return GA_EUNSUPPORTED;
  if (n_runs > 0)
    hipLaunchKernelGGL((gat_runs_kernel<T, VEC>), dim3((unsigned)fix_blocks, ftiles),
                       dim3(kBlock), 0, stream, row_of_slot, nbr, el, er,
                       (const T *)z, (T *)out, pacc, pml, n_edges, n_runs, feat,
                       heads, dim, slope, run_shift, tpr_shift);
  if (fix_blocks + fill_blocks > 0)
    hipLaunchKernelGGL((gat_fixup_kernel<T, VEC>),
                       dim3((unsigned)(fix_blocks + fill_blocks), ftiles),
                       dim3(kBlock), 0, stream, pointer, row_of_slot, pacc, pml,
                       (T *)out, n_rows, n_edges, n_runs, feat, heads, dim,
                       run_shift, tpr_shift, (int)fix_blocks);
  return launch_status();
}

}  // namespace
}  // namespace ga

extern "C" {

size_t ga_gat_workspace_bytes(int64_t n_edges, int64_t feat, int64_t heads) {
  if (n_edges <= 0 || feat <= 0 || heads <= 0) return 0;
  const int run_shift = ga::run_shift_for(n_edges, feat);
  const int64_t n_runs = (n_edges + ((int64_t)1 << run_shift) - 1) >> run_shift;
  return (size_t)n_runs * 2 * (size_t)(feat + 2 * heads) * sizeof(float);
}

int ga_gat_aggregate(const int32_t *pointer, const int32_t *row_of_slot,
                     const int32_t *nbr, const float *el, const float *er,
                     const void *z, void *out, int64_t n_rows, int64_t n_edges,
                     int64_t heads, int64_t dim, float slope, int dtype,
                     void *workspace, size_t workspace_bytes,
                     ga_stream_t stream) {
  if (n_rows < 0 || n_edges < 0 || heads <= 0 || dim <= 0) return GA_EINVAL;
  if (n_rows > 0x7fffffff || n_edges > 0x7fffffff ||
      heads * dim > 0x7fffffff)
    return GA_EINVAL;
  if (dtype != GA_F32 && dtype != GA_BF16) return GA_EINVAL;
  if (n_rows == 0) return GA_OK;
  if (!pointer || !out) return GA_EINVAL;
  const int64_t feat = heads * dim;
  if (n_edges > 0) {
    if (!row_of_slot || !nbr || !el || !er || !z) return GA_EINVAL;
    if (!workspace || !ga::aligned(workspace, 16) ||
        ga_gat_workspace_bytes(n_edges, feat, heads) > workspace_bytes)
      return GA_EWORKSPACE;
  }
  const size_t esz = dtype == GA_F32 ? 4 : 2;
  if (!ga::aligned(out, esz) || (z && !ga::aligned(z, esz)) ||
      (el && !ga::aligned(el, 4)) || (er && !ga::aligned(er, 4)))
    return GA_EALIGN;
  const bool vec_ok = ga::aligned(out, 16) && (!z || ga::aligned(z, 16));
  hipStream_t s = (hipStream_t)stream;
  float *ws = (float *)workspace;
  if (dtype == GA_F32) {
    if (vec_ok && dim % 4 == 0)
      return ga::launch_gat<float, 4>(pointer, row_of_slot, nbr, el, er, z, out,
                                      n_rows, n_edges, (int)heads, (int)dim,
                                      slope, ws, s);
    return ga::launch_gat<float, 1>(pointer, row_of_slot, nbr, el, er, z, out,
                                    n_rows, n_edges, (int)heads, (int)dim, slope,
                                    ws, s);
  }
  if (vec_ok && dim % 8 == 0)
    return ga::launch_gat<ga::bf16_t, 8>(pointer, row_of_slot, nbr, el, er, z,
                                         out, n_rows, n_edges, (int)heads,
                                         (int)dim, slope, ws, s);
  return ga::launch_gat<ga::bf16_t, 1>(pointer, row_of_slot, nbr, el, er, z, out,
                                       n_rows, n_edges, (int)heads, (int)dim,
                                       slope, ws, s);
}

}  // extern "C"
