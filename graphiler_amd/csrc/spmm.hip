// Load-balanced CSR SpMM for gfx950 (copy_u / copy_e / u_mul_e x sum / max / min).
//
// Scheduling.  The adjacency's slots [0, E) are cut into equal runs of 2^s
// slots.  A group of `tpr` adjacent lanes (tpr * VEC features cover one feature
// row, 16 bytes per lane when VEC > 1) owns one run and walks it in slot order,
// eight gathers in flight per lane.  Rows that lie inside one run are written
// straight to the output; the (at most two) rows a run shares with its
// neighbours are written as fp32 partial rows to the workspace and combined by
// a second kernel in run order.  Work per lane group is therefore identical
// whatever the degree distribution, no atomics are used, and the summation
// order depends on the graph and sizes only.
#include "common.h"

namespace ga {

int run_shift_for(int64_t n_edges, int64_t feat) {
  // lanes a feature row occupies with 16-byte fp32 accesses
  int64_t lanes = (feat + 3) / 4;
  int lane_shift = ilog2_ceil((uint64_t)(lanes < 1 ? 1 : (lanes > 64 ? 64 : lanes)));
  // aim at >= 16k wavefronts of work, between 32 and 1024 slots per run
  int64_t per_run = (n_edges << lane_shift) / 64 / 16384;
  int shift = per_run < 1 ? 0 : ilog2_floor((uint64_t)per_run);
  if (shift < 5) shift = 5;
  if (shift > 10) shift = 10;
  return shift;
}

namespace {

constexpr int kUnroll = 8;

template <int RED>
__device__ __forceinline__ float red_init() {
  return RED == GA_SUM ? 0.0f : (RED == GA_MAX ? -INFINITY : INFINITY);
}
template <int RED>
__device__ __forceinline__ float red_apply(float acc, float m) {
  if (RED == GA_SUM) return acc + m;
  // strict comparison: the first extremum in slot order wins, NaN never does
  if (RED == GA_MAX) return acc < m ? m : acc;
  return acc > m ? m : acc;
}

// One lane group per run.  gidx: row of `u` gathered per slot (neighbour id, or
// edge id for copy_e); nullptr means the slot index itself.
template <typename T, int VEC, int RED, bool HASW>
__global__ __launch_bounds__(kBlock) void spmm_runs_kernel(
    const int32_t *__restrict__ row_of_slot, const int32_t *__restrict__ gidx,
    const int32_t *__restrict__ eid, const T *__restrict__ u,
    const float *__restrict__ w, T *__restrict__ out,
    float *__restrict__ partial, int64_t n_edges, int64_t n_runs, int feat,
    int heads, int dph, int run_shift, int tpr_shift) {
  typedef Frag<T, VEC> IO;
  const int tpr = 1 << tpr_shift;
  const int64_t k = ((int64_t)blockIdx.x * kBlock + threadIdx.x) >> tpr_shift;
  const int f0 = ((int)blockIdx.y * tpr + (threadIdx.x & (tpr - 1))) * VEC;
  if (k >= n_runs || f0 >= feat) return;
  const int h = HASW ? f0 / dph : 0;

  const int64_t a = k << run_shift;
  const int64_t b = min(a + ((int64_t)1 << run_shift), n_edges);

  int cur = row_of_slot[a];
  const bool began_before = a > 0 && row_of_slot[a - 1] == cur;
  bool first_seg = true;

  float acc[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) acc[v] = red_init<RED>();

  for (int64_t j = a; j < b; j += kUnroll) {
    int r[kUnroll];
    int64_t g[kUnroll];
    float ww[kUnroll];
    typename IO::raw_t x[kUnroll];
#pragma unroll
    for (int t = 0; t < kUnroll; ++t) {
      const int64_t jj = j + t < b ? j + t : b - 1;
      r[t] = row_of_slot[jj];
      g[t] = gidx ? (int64_t)gidx[jj] : jj;
      if (HASW) {
        const int64_t e = eid ? (int64_t)eid[jj] : jj;
        ww[t] = w[e * heads + h];
      }
    }
#pragma unroll
    for (int t = 0; t < kUnroll; ++t) x[t] = IO::load(u + g[t] * feat + f0);
#pragma unroll
    for (int t = 0; t < kUnroll; ++t) {
      if (j + t < b) {
        if (r[t] != cur) {
          // the open row ended inside this run
          if (first_seg && began_before) {
            float *p = partial + (k * 2) * feat + f0;
#pragma unroll
            for (int v = 0; v < VEC; ++v) p[v] = acc[v];
          } else {
            IO::store(out + (int64_t)cur * feat + f0, acc);
          }
          first_seg = false;
          cur = r[t];
#pragma unroll
          for (int v = 0; v < VEC; ++v) acc[v] = red_init<RED>();
        }
        float xf[VEC];
        IO::widen(x[t], xf);
#pragma unroll
        for (int v = 0; v < VEC; ++v)
          acc[v] = red_apply<RED>(acc[v], HASW ? xf[v] * ww[t] : xf[v]);
      }
    }
  }
  const bool continues = b < n_edges && row_of_slot[b] == cur;
  if (first_seg ? (began_before || continues) : continues) {
    float *p = partial + (k * 2 + (first_seg ? 0 : 1)) * feat + f0;
#pragma unroll
    for (int v = 0; v < VEC; ++v) p[v] = acc[v];
  } else {
    IO::store(out + (int64_t)cur * feat + f0, acc);
  }
}

// Blocks [0, fix_blocks): one lane group per run; the group whose run holds
// the END of a row that began in an earlier run combines that row's partials
// in run order.  Remaining blocks: one lane group per row, rows without edges
// receive the reducer's start value.
template <typename T, int VEC, int RED>
__global__ __launch_bounds__(kBlock) void spmm_fixup_kernel(
    const int32_t *__restrict__ pointer, const int32_t *__restrict__ row_of_slot,
    const float *__restrict__ partial, T *__restrict__ out, int64_t n_rows,
    int64_t n_edges, int64_t n_runs, int feat, int run_shift, int tpr_shift,
    int fix_blocks) {
  typedef Frag<T, VEC> IO;
  const int tpr = 1 << tpr_shift;
  const int f0 = ((int)blockIdx.y * tpr + (threadIdx.x & (tpr - 1))) * VEC;
  if (f0 >= feat) return;
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
    const int slot = (s == (k_lo << run_shift)) ? 0 : 1;
    const float *p = partial + (k_lo * 2 + slot) * feat + f0;
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = p[v];
    for (int64_t q = k_lo + 1; q <= k; ++q) {
      const float *pq = partial + (q * 2) * feat + f0;
#pragma unroll
      for (int v = 0; v < VEC; ++v) acc[v] = red_apply<RED>(acc[v], pq[v]);
    }
    IO::store(out + (int64_t)row * feat + f0, acc);
  } else {
    const int64_t row =
        ((int64_t)(blockIdx.x - fix_blocks) * kBlock + threadIdx.x) >> tpr_shift;
    if (row >= n_rows || pointer[row] != pointer[row + 1]) return;
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = red_init<RED>();
    IO::store(out + row * feat + f0, acc);
  }
}

template <typename T, int VEC, int RED, bool HASW>
int launch_spmm(const int32_t *pointer, const int32_t *row_of_slot,
                const int32_t *gidx, const int32_t *eid, const void *u,
                const float *w, void *out, int64_t n_rows, int64_t n_edges,
                int feat, int heads, float *partial, hipStream_t stream) {
  const int lanes = (feat + VEC - 1) / VEC;
  const int tpr_shift = ilog2_ceil((uint64_t)(lanes > kWave ? kWave : lanes));
  const int tpr = 1 << tpr_shift;
  const int ftiles = (lanes + tpr - 1) / tpr;
  const int run_shift = run_shift_for(n_edges, feat);
  const int64_t n_runs = (n_edges + ((int64_t)1 << run_shift) - 1) >> run_shift;
  const int groups_per_block = kBlock >> tpr_shift;
  if (n_runs > 0) {
    const int64_t blocks = (n_runs + groups_per_block - 1) / groups_per_block;
    if (blocks > 0x7fffffff) return GA_EUNSUPPORTED;
    hipLaunchKernelGGL((spmm_runs_kernel<T, VEC, RED, HASW>),
                       dim3((unsigned)blocks, ftiles), dim3(kBlock), 0, stream,
                       row_of_slot, gidx, eid, (const T *)u, w, (T *)out,
                       partial, n_edges, n_runs, feat, heads, feat / heads,
                       run_shift, tpr_shift);
  }
  const int64_t fix_blocks = (n_runs + groups_per_block - 1) / groups_per_block;
  const int64_t fill_blocks = (n_rows + groups_per_block - 1) / groups_per_block;
  if (fix_blocks + fill_blocks > 0x7fffffff) return GA_EUNSUPPORTED;
  if (fix_blocks + fill_blocks > 0)
    hipLaunchKernelGGL((spmm_fixup_kernel<T, VEC, RED>),
                       dim3((unsigned)(fix_blocks + fill_blocks), ftiles),
                       dim3(kBlock), 0, stream, pointer, row_of_slot, partial,
                       (T *)out, n_rows, n_edges, n_runs, feat, run_shift,
                       tpr_shift, (int)fix_blocks);
  return launch_status();
}

template <typename T, int VEC, int RED>
int pick_w(bool hasw, const int32_t *pointer, const int32_t *row_of_slot,
           const int32_t *gidx, const int32_t *eid, const void *u,
           const float *w, void *out, int64_t n_rows, int64_t n_edges, int feat,
           int heads, float *partial, hipStream_t stream) {
  return hasw ? launch_spmm<T, VEC, RED, true>(pointer, row_of_slot, gidx, eid,
                                                u, w, out, n_rows, n_edges, feat,
                                                heads, partial, stream)
              : launch_spmm<T, VEC, RED, false>(pointer, row_of_slot, gidx, eid,
                                                 u, w, out, n_rows, n_edges,
                                                 feat, heads, partial, stream);
}

template <typename T, int VEC>
int pick_red(int reduce, bool hasw, const int32_t *pointer,
             const int32_t *row_of_slot, const int32_t *gidx,
             const int32_t *eid, const void *u, const float *w, void *out,
             int64_t n_rows, int64_t n_edges, int feat, int heads,
             float *partial, hipStream_t stream) {
  switch (reduce) {
    case GA_SUM:
      return pick_w<T, VEC, GA_SUM>(hasw, pointer, row_of_slot, gidx, eid, u, w,
                                    out, n_rows, n_edges, feat, heads, partial,
                                    stream);
    case GA_MAX:
      return pick_w<T, VEC, GA_MAX>(hasw, pointer, row_of_slot, gidx, eid, u, w,
                                    out, n_rows, n_edges, feat, heads, partial,
                                    stream);
    default:
      return pick_w<T, VEC, GA_MIN>(hasw, pointer, row_of_slot, gidx, eid, u, w,
                                    out, n_rows, n_edges, feat, heads, partial,
                                    stream);
  }
}

__global__ __launch_bounds__(kBlock) void row_ids_kernel(
    const int32_t *__restrict__ pointer, int64_t n_rows, int64_t n_edges,
    int32_t *__restrict__ row_of_slot) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= n_edges) return;
  // largest v with pointer[v] <= i  (rows without edges are skipped over)
  int64_t lo = 0, hi = n_rows;  // invariant: pointer[lo] <= i < pointer[hi]
  while (hi - lo > 1) {
    const int64_t mid = (lo + hi) >> 1;
    if ((int64_t)pointer[mid] <= i) lo = mid; else hi = mid;
  }
  row_of_slot[i] = (int32_t)lo;
}

}  // namespace
}  // namespace ga

extern "C" {

int ga_csr_row_ids(const int32_t *pointer, int64_t n_rows, int64_t n_edges,
                   int32_t *row_of_slot, ga_stream_t stream) {
  if (n_rows < 0 || n_edges < 0 || n_rows > 0x7fffffff || n_edges > 0x7fffffff)
    return GA_EINVAL;
  if (n_edges == 0) return GA_OK;
  if (!pointer || !row_of_slot || n_rows == 0) return GA_EINVAL;
  const int64_t blocks = (n_edges + ga::kBlock - 1) / ga::kBlock;
  hipLaunchKernelGGL(ga::row_ids_kernel, dim3((unsigned)blocks),
                     dim3(ga::kBlock), 0, (hipStream_t)stream, pointer, n_rows,
                     n_edges, row_of_slot);
  return ga::launch_status();
}

size_t ga_spmm_workspace_bytes(int64_t n_edges, int64_t feat) {
  if (n_edges <= 0 || feat <= 0) return 0;
  const int run_shift = ga::run_shift_for(n_edges, feat);
  const int64_t n_runs = (n_edges + ((int64_t)1 << run_shift) - 1) >> run_shift;
  return (size_t)n_runs * 2 * (size_t)feat * sizeof(float);
}

int ga_spmm_csr(const int32_t *pointer, const int32_t *row_of_slot,
                const int32_t *nbr, const int32_t *eid, const void *u,
                const float *w, void *out, int64_t n_rows, int64_t n_edges,
                int64_t feat, int64_t heads, int op, int reduce, int dtype,
                void *workspace, size_t workspace_bytes, ga_stream_t stream) {
  if (n_rows < 0 || n_edges < 0 || feat <= 0 || heads <= 0 || feat % heads)
    return GA_EINVAL;
  if (n_rows > 0x7fffffff || n_edges > 0x7fffffff || feat > 0x7fffffff)
    return GA_EINVAL;
  if (op < GA_COPY_U || op > GA_U_MUL_E || reduce < GA_SUM || reduce > GA_MIN)
    return GA_EINVAL;
  if (dtype != GA_F32 && dtype != GA_BF16) return GA_EINVAL;
  if (n_rows == 0) return GA_OK;
  if (!pointer || !out) return GA_EINVAL;
  if (n_edges > 0) {
    if (!row_of_slot || !u) return GA_EINVAL;
    if (op != GA_COPY_E && !nbr) return GA_EINVAL;
    if (op == GA_U_MUL_E && !w) return GA_EINVAL;
    if (ga_spmm_workspace_bytes(n_edges, feat) > workspace_bytes || !workspace)
      return GA_EWORKSPACE;
    if (!ga::aligned(workspace, 16)) return GA_EWORKSPACE;
  }
  const size_t esz = dtype == GA_F32 ? 4 : 2;
  if (!ga::aligned(out, esz) || (u && !ga::aligned(u, esz)) ||
      (w && !ga::aligned(w, 4)))
    return GA_EALIGN;

  const bool hasw = op == GA_U_MUL_E;
  const int32_t *gidx = op == GA_COPY_E ? eid : nbr;
  const int64_t dph = feat / heads;
  const bool vec_ok = ga::aligned(out, 16) && (!u || ga::aligned(u, 16));
  hipStream_t s = (hipStream_t)stream;
  float *partial = (float *)workspace;
  if (dtype == GA_F32) {
    if (vec_ok && feat % 4 == 0 && (!hasw || dph % 4 == 0))
      return ga::pick_red<float, 4>(reduce, hasw, pointer, row_of_slot, gidx,
                                    eid, u, w, out, n_rows, n_edges, (int)feat,
                                    (int)heads, partial, s);
    return ga::pick_red<float, 1>(reduce, hasw, pointer, row_of_slot, gidx, eid,
                                  u, w, out, n_rows, n_edges, (int)feat,
                                  (int)heads, partial, s);
  }
  if (vec_ok && feat % 8 == 0 && (!hasw || dph % 8 == 0))
    return ga::pick_red<ga::bf16_t, 8>(reduce, hasw, pointer, row_of_slot, gidx,
                                       eid, u, w, out, n_rows, n_edges,
                                       (int)feat, (int)heads, partial, s);
  return ga::pick_red<ga::bf16_t, 1>(reduce, hasw, pointer, row_of_slot, gidx,
                                     eid, u, w, out, n_rows, n_edges, (int)feat,
                                     (int)heads, partial, s);
}

}  // extern "C"
