// Edge segment softmax for gfx950 (any number of heads), fp32.
//
// Rows are owned by lane groups: a group of S adjacent lanes (S a power of two
// picked from the average segment size) handles one destination row, keeps up
// to kCache elements per lane in registers so a typical segment is read once,
// and reduces max / sum with a fixed xor-shuffle tree.  Rows longer than
// kLongRow slots are skipped there and cut into chunks at the multiples of
// kLongRow, one workgroup per chunk (found without any list: the workgroup
// looks up the row of its first slot): pass A writes per-chunk (max, sum-exp)
// to the workspace, pass B merges them in chunk order and normalises.
// No atomics; the order of every reduction is fixed.
#include "common.h"

namespace ga {
namespace {

constexpr int kCache = 4;
constexpr int kLongRow = 1024;

// heads is a power of two <= S: lane -> fixed head (lane & (heads-1)).
__global__ __launch_bounds__(kBlock) void softmax_rows_pow2_kernel(
    const int32_t *__restrict__ pointer, const int32_t *__restrict__ eid,
    const float *__restrict__ x, float *__restrict__ y, int64_t n_rows,
    int head_shift, int s_shift) {
  const int S = 1 << s_shift;
  const int H = 1 << head_shift;
  const int lane = threadIdx.x & (S - 1);
  const int64_t row = ((int64_t)blockIdx.x * kBlock + threadIdx.x) >> s_shift;
  int64_t start = 0, n = 0;
  if (row < n_rows) {
    start = pointer[row];
    const int64_t deg = pointer[row + 1] - start;
    n = deg > kLongRow ? 0 : deg << head_shift;
  }
  const int hh = lane & (H - 1);
  float c[kCache];
  int64_t off[kCache];
  float m = -INFINITY;
#pragma unroll
  for (int t = 0; t < kCache; ++t) {
    const int64_t q = lane + (int64_t)t * S;
    c[t] = -INFINITY;
    off[t] = -1;
    if (q < n) {
      const int64_t slot = start + (q >> head_shift);
      const int64_t e = eid ? (int64_t)eid[slot] : slot;
      off[t] = (e << head_shift) + hh;
      c[t] = x[off[t]];
      m = fmaxf(m, c[t]);
    }
  }
  for (int64_t q = lane + (int64_t)kCache * S; q < n; q += S) {
    const int64_t slot = start + (q >> head_shift);
    const int64_t e = eid ? (int64_t)eid[slot] : slot;
    m = fmaxf(m, x[(e << head_shift) + hh]);
  }
  for (int o = S >> 1; o >= H; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
  float l = 0.0f;
#pragma unroll
  for (int t = 0; t < kCache; ++t) {
    if (off[t] >= 0) {
      c[t] = expf(c[t] - m);
      l += c[t];
    }
  }
  for (int64_t q = lane + (int64_t)kCache * S; q < n; q += S) {
    const int64_t slot = start + (q >> head_shift);
    const int64_t e = eid ? (int64_t)eid[slot] : slot;
    l += expf(x[(e << head_shift) + hh] - m);
  }
  for (int o = S >> 1; o >= H; o >>= 1) l += __shfl_xor(l, o);
#pragma unroll
  for (int t = 0; t < kCache; ++t)
    if (off[t] >= 0) y[off[t]] = c[t] / l;
  for (int64_t q = lane + (int64_t)kCache * S; q < n; q += S) {
    const int64_t slot = start + (q >> head_shift);
    const int64_t e = eid ? (int64_t)eid[slot] : slot;
    const int64_t o = (e << head_shift) + hh;
    y[o] = expf(x[o] - m) / l;
  }
}

// Any head count: the group runs the heads one after the other.
__global__ __launch_bounds__(kBlock) void softmax_rows_generic_kernel(
    const int32_t *__restrict__ pointer, const int32_t *__restrict__ eid,
    const float *__restrict__ x, float *__restrict__ y, int64_t n_rows,
    int heads, int s_shift) {
  const int S = 1 << s_shift;
  const int lane = threadIdx.x & (S - 1);
  const int64_t row = ((int64_t)blockIdx.x * kBlock + threadIdx.x) >> s_shift;
  int64_t start = 0, deg = 0;
  if (row < n_rows) {
    start = pointer[row];
    deg = pointer[row + 1] - start;
    if (deg > kLongRow) deg = 0;
  }
  for (int h = 0; h < heads; ++h) {
    float m = -INFINITY;
    for (int64_t q = lane; q < deg; q += S) {
      const int64_t e = eid ? (int64_t)eid[start + q] : start + q;
      m = fmaxf(m, x[e * heads + h]);
    }
    for (int o = S >> 1; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
    float l = 0.0f;
    for (int64_t q = lane; q < deg; q += S) {
      const int64_t e = eid ? (int64_t)eid[start + q] : start + q;
      l += expf(x[e * heads + h] - m);
    }
    for (int o = S >> 1; o > 0; o >>= 1) l += __shfl_xor(l, o);
    for (int64_t q = lane; q < deg; q += S) {
      const int64_t e = eid ? (int64_t)eid[start + q] : start + q;
      y[e * heads + h] = expf(x[e * heads + h] - m) / l;
    }
  }
}

template <bool IS_MAX>
__device__ __forceinline__ float block_reduce(float v, float *lds) {
  for (int o = kWave >> 1; o > 0; o >>= 1) {
    const float other = __shfl_xor(v, o);
    v = IS_MAX ? fmaxf(v, other) : v + other;
  }
  const int wave = threadIdx.x / kWave;
  __syncthreads();  // lds may still be read from the previous reduction
  if ((threadIdx.x & (kWave - 1)) == 0) lds[wave] = v;
  __syncthreads();
  float r = lds[0];
  for (int q = 1; q < kBlock / kWave; ++q)
    r = IS_MAX ? fmaxf(r, lds[q]) : r + lds[q];
  return r;
}

// Rows longer than kLongRow slots are cut at the multiples of kLongRow; the
// workgroup of chunk c owns the slots [c*kLongRow, (c+1)*kLongRow) of the long
// row that contains slot c*kLongRow, and the first chunk of a row also takes
// the row's slots before its first multiple.  Returns false when the chunk
// holds no part of a long row.
__device__ __forceinline__ bool long_chunk(const int32_t *pointer,
                                           const int32_t *row_of_slot,
                                           int64_t n_edges, int64_t &lo,
                                           int64_t &hi, int64_t &c_first,
                                           int64_t &c_last) {
  const int64_t c = blockIdx.x;
  const int row = row_of_slot[c * kLongRow];
  const int64_t start = pointer[row], end = pointer[row + 1];
  if (end - start <= kLongRow) return false;
  c_first = (start + kLongRow - 1) / kLongRow;
  c_last = (end - 1) / kLongRow;
  lo = c == c_first ? start : c * kLongRow;
  hi = min(end, (c + 1) * (int64_t)kLongRow);
  return true;
}

// Pass A: per chunk and head, (max, sum of exp(x - max)) -> stats[c][h][2].
__global__ __launch_bounds__(kBlock) void softmax_long_stats_kernel(
    const int32_t *__restrict__ pointer, const int32_t *__restrict__ row_of_slot,
    const int32_t *__restrict__ eid, const float *__restrict__ x,
    float *__restrict__ stats, int64_t n_edges, int heads) {
  __shared__ float lds[kBlock / kWave];
  int64_t lo, hi, c_first, c_last;
  if (!long_chunk(pointer, row_of_slot, n_edges, lo, hi, c_first, c_last)) return;
  for (int h = 0; h < heads; ++h) {
    float m = -INFINITY;
    for (int64_t q = lo + threadIdx.x; q < hi; q += kBlock) {
      const int64_t e = eid ? (int64_t)eid[q] : q;
      m = fmaxf(m, x[e * heads + h]);
    }
    m = block_reduce<true>(m, lds);
    float l = 0.0f;
    for (int64_t q = lo + threadIdx.x; q < hi; q += kBlock) {
      const int64_t e = eid ? (int64_t)eid[q] : q;
      l += expf(x[e * heads + h] - m);
    }
    l = block_reduce<false>(l, lds);
    if (threadIdx.x == 0) {
      stats[((int64_t)blockIdx.x * heads + h) * 2] = m;
      stats[((int64_t)blockIdx.x * heads + h) * 2 + 1] = l;
    }
  }
}

// Pass B: merge the row's chunk statistics in chunk order, then normalise.
__global__ __launch_bounds__(kBlock) void softmax_long_write_kernel(
    const int32_t *__restrict__ pointer, const int32_t *__restrict__ row_of_slot,
    const int32_t *__restrict__ eid, const float *__restrict__ x,
    const float *__restrict__ stats, float *__restrict__ y, int64_t n_edges,
    int heads) {
  int64_t lo, hi, c_first, c_last;
  if (!long_chunk(pointer, row_of_slot, n_edges, lo, hi, c_first, c_last)) return;
  for (int h = 0; h < heads; ++h) {
    float m = -INFINITY;
    for (int64_t c = c_first; c <= c_last; ++c)
      m = fmaxf(m, stats[(c * heads + h) * 2]);
    float l = 0.0f;
    for (int64_t c = c_first; c <= c_last; ++c)
      l += stats[(c * heads + h) * 2 + 1] * expf(stats[(c * heads + h) * 2] - m);
    for (int64_t q = lo + threadIdx.x; q < hi; q += kBlock) {
      const int64_t e = eid ? (int64_t)eid[q] : q;
      y[e * heads + h] = expf(x[e * heads + h] - m) / l;
    }
  }
}

}  // namespace
}  // namespace ga

extern "C" {

size_t ga_softmax_workspace_bytes(int64_t n_edges, int64_t heads) {
  if (n_edges <= ga::kLongRow || heads <= 0) return 0;
  const int64_t chunks = (n_edges + ga::kLongRow - 1) / ga::kLongRow;
  return (size_t)chunks * (size_t)heads * 2 * sizeof(float);
}

int ga_segment_softmax(const int32_t *pointer, const int32_t *row_of_slot,
                       const int32_t *eid, const float *x, float *y,
                       int64_t n_rows, int64_t n_edges, int64_t heads,
                       void *workspace, size_t workspace_bytes,
                       ga_stream_t stream) {
  using namespace ga;
  if (n_rows < 0 || n_edges < 0 || heads <= 0) return GA_EINVAL;
  if (n_rows > 0x7fffffff || n_edges > 0x7fffffff || heads > 65536)
    return GA_EINVAL;
  if (n_rows == 0 || n_edges == 0) return GA_OK;
  if (!pointer || !row_of_slot || !x || !y) return GA_EINVAL;
  if (!aligned(x, 4) || !aligned(y, 4)) return GA_EALIGN;
  const size_t need = ga_softmax_workspace_bytes(n_edges, heads);
  if (need && (!workspace || workspace_bytes < need || !aligned(workspace, 16)))
    return GA_EWORKSPACE;
  hipStream_t s = (hipStream_t)stream;

  // lanes per row: the register cache (kCache elements per lane) should cover
  // an average segment, so that it is read from memory once
  const bool pow2 = (heads & (heads - 1)) == 0 && heads <= kWave;
  const int64_t avg = (n_edges * (pow2 ? heads : 1) + n_rows - 1) / n_rows;
  int s_shift = ilog2_ceil((uint64_t)((avg + kCache - 1) / kCache));
  if (s_shift < 2) s_shift = 2;
  if (s_shift > 6) s_shift = 6;
  if (pow2 && (1 << s_shift) < heads) s_shift = ilog2_ceil((uint64_t)heads);
  const int64_t per_block = kBlock >> s_shift;
  const int64_t blocks = (n_rows + per_block - 1) / per_block;
  if (blocks > 0x7fffffff) return GA_EUNSUPPORTED;
  if (pow2)
    hipLaunchKernelGGL(softmax_rows_pow2_kernel, dim3((unsigned)blocks),
                       dim3(kBlock), 0, s, pointer, eid, x, y, n_rows,
                       ilog2_floor((uint64_t)heads), s_shift);
  else
    hipLaunchKernelGGL(softmax_rows_generic_kernel, dim3((unsigned)blocks),
                       dim3(kBlock), 0, s, pointer, eid, x, y, n_rows,
                       (int)heads, s_shift);
  if (n_edges > kLongRow) {
    const int64_t chunks = (n_edges + kLongRow - 1) / kLongRow;
    float *stats = (float *)workspace;
    hipLaunchKernelGGL(softmax_long_stats_kernel, dim3((unsigned)chunks),
                       dim3(kBlock), 0, s, pointer, row_of_slot, eid, x, stats,
                       n_edges, (int)heads);
    hipLaunchKernelGGL(softmax_long_write_kernel, dim3((unsigned)chunks),
                       dim3(kBlock), 0, s, pointer, row_of_slot, eid, x, stats, y,
                       n_edges, (int)heads);
  }
  return launch_status();
}

}  // extern "C"
