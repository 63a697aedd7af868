// Edge segment softmax for gfx950 (any number of heads), fp32.
//
// A segment is the run of (slot, head) elements of one destination row, n =
// degree * heads values that are contiguous in memory when edge ids are slot
// numbers.  Power-of-two head counts (<= 64) take three size classes, each with
// its own launch so that no lane group idles behind a long row:
//   small   n <= 4*S      a group of S adjacent lanes per row (S from the mean
//                         segment size), every element held in a register;
//   medium  n <= 1024     one wavefront per row, 16 elements per lane in
//                         registers.  Waves are not launched per row but per
//                         chunk of 1024 elements: a wave scans the rows that
//                         START in its chunk and takes the medium ones;
//   long    n  > 1024     cut at multiples of 1024/heads slots, one workgroup
//                         per chunk: pass A writes per-chunk (max, sum-exp) per
//                         head to the workspace, pass B merges them in chunk
//                         order and normalises.
// Every segment is read once (small, medium) or twice (long).  Other head
// counts use a generic lane-group kernel that runs the heads one after the
// other.  No atomics; the order of every reduction is fixed by the sizes.
#include "common.h"

namespace ga {
namespace {

constexpr int kSmallCache = 4;     // elements per lane, small rows
constexpr int kMediumCache = 16;   // elements per lane, medium rows
constexpr int kMediumMax = kWave * kMediumCache;   // 1024 elements
constexpr int kChunkElems = 1024;  // elements scanned per medium-kernel wave
constexpr int kLongRow = 1024;     // generic path: slots per long-row chunk

__device__ __forceinline__ int64_t elem_offset(const int32_t *__restrict__ eid,
                                               int64_t start, int64_t q,
                                               int head_shift) {
  const int64_t slot = start + (q >> head_shift);
  const int64_t e = eid ? (int64_t)eid[slot] : slot;
  return (e << head_shift) + (q & ((1 << head_shift) - 1));
}

// ---- small rows -----------------------------------------------------------
__global__ __launch_bounds__(kBlock) void softmax_small_kernel(
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
    n = (int64_t)(pointer[row + 1] - start) << head_shift;
    if (n > (int64_t)kSmallCache * S) n = 0;   // another class owns this row
  }
  float c[kSmallCache];
  int64_t off[kSmallCache];
  float m = -INFINITY;
#pragma unroll
  for (int t = 0; t < kSmallCache; ++t) {
    const int64_t q = lane + (int64_t)t * S;   // lane keeps one head: S % H == 0
    c[t] = -INFINITY;
    off[t] = -1;
    if (q < n) {
      off[t] = elem_offset(eid, start, q, head_shift);
      c[t] = x[off[t]];
      m = fmaxf(m, c[t]);
    }
  }
  for (int o = S >> 1; o >= H; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
  float l = 0.0f;
#pragma unroll
  for (int t = 0; t < kSmallCache; ++t) {
    c[t] = off[t] >= 0 ? expf(c[t] - m) : 0.0f;
    l += c[t];
  }
  for (int o = S >> 1; o >= H; o >>= 1) l += __shfl_xor(l, o);
#pragma unroll
  for (int t = 0; t < kSmallCache; ++t)
    if (off[t] >= 0) y[off[t]] = c[t] / l;
}

// ---- medium rows ----------------------------------------------------------
__global__ __launch_bounds__(kBlock) void softmax_medium_kernel(
    const int32_t *__restrict__ pointer, const int32_t *__restrict__ row_of_slot,
    const int32_t *__restrict__ eid, const float *__restrict__ x,
    float *__restrict__ y, int64_t n_rows, int64_t n_edges, int head_shift,
    int small_max) {
  const int H = 1 << head_shift;
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t chunk = ((int64_t)blockIdx.x * kBlock + threadIdx.x) / kWave;
  const int chunk_slots = kChunkElems >> head_shift;
  const int64_t c0 = chunk * chunk_slots;
  if (c0 >= n_edges) return;                       // whole wave
  const int64_t c1 = min(c0 + (int64_t)chunk_slots, n_edges);
  // first row that starts inside [c0, c1)
  int64_t r0 = row_of_slot[c0];
  if ((int64_t)pointer[r0] < c0) ++r0;
  for (;; r0 += kWave) {
    const int64_t r = r0 + lane;
    int64_t start = n_edges, end = n_edges;
    if (r < n_rows) {
      start = pointer[r];
      end = pointer[r + 1];
    }
    const bool starts_here = r < n_rows && start < c1;
    const int64_t n = (end - start) << head_shift;
    uint64_t todo = __ballot(starts_here && n > small_max && n <= kMediumMax);
    while (todo) {
      const int src = __ffsll((unsigned long long)todo) - 1;
      todo &= todo - 1;
      const int64_t rs = __shfl(start, src);
      const int64_t rn = __shfl(n, src);
      float c[kMediumCache];
      int64_t off[kMediumCache];
      float m = -INFINITY;
#pragma unroll
      for (int t = 0; t < kMediumCache; ++t) {
        const int64_t q = lane + (int64_t)t * kWave;
        c[t] = -INFINITY;
        off[t] = -1;
        if (q < rn) {
          off[t] = elem_offset(eid, rs, q, head_shift);
          c[t] = x[off[t]];
          m = fmaxf(m, c[t]);
        }
      }
      for (int o = kWave >> 1; o >= H; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
      float l = 0.0f;
#pragma unroll
      for (int t = 0; t < kMediumCache; ++t) {
        c[t] = off[t] >= 0 ? expf(c[t] - m) : 0.0f;
        l += c[t];
      }
      for (int o = kWave >> 1; o >= H; o >>= 1) l += __shfl_xor(l, o);
#pragma unroll
      for (int t = 0; t < kMediumCache; ++t)
        if (off[t] >= 0) y[off[t]] = c[t] / l;
    }
    // stop once a lane's row starts at or beyond the chunk end (rows ascend)
    if (__ballot(!starts_here)) break;
  }
}

// ---- long rows -------------------------------------------------------------
// Chunk c of L slots belongs to the long row that contains slot c*L; the first
// chunk of a row also takes the row's slots before its first multiple of L.
__device__ __forceinline__ bool long_chunk(const int32_t *pointer,
                                           const int32_t *row_of_slot, int L,
                                           int long_min_deg, int64_t &lo,
                                           int64_t &hi, int64_t &c_first,
                                           int64_t &c_last) {
  const int64_t c = blockIdx.x;
  const int row = row_of_slot[c * L];
  const int64_t start = pointer[row], end = pointer[row + 1];
  if (end - start < long_min_deg) return false;
  c_first = (start + L - 1) / L;
  c_last = (end - 1) / L;
  lo = c == c_first ? start : c * L;
  hi = min(end, (c + 1) * (int64_t)L);
  return true;
}

// reduce over the lanes of the workgroup that share (tid & (H-1))
template <bool IS_MAX>
__device__ __forceinline__ float block_reduce_heads(float v, int H, float *lds) {
  for (int o = kWave >> 1; o >= H; o >>= 1) {
    const float other = __shfl_xor(v, o);
    v = IS_MAX ? fmaxf(v, other) : v + other;
  }
  const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  __syncthreads();   // lds may still be read from the previous reduction
  if (lane < H) lds[wave * kWave + lane] = v;
  __syncthreads();
  const int h = lane & (H - 1);
  float r = lds[h];
  for (int w = 1; w < kBlock / kWave; ++w)
    r = IS_MAX ? fmaxf(r, lds[w * kWave + h]) : r + lds[w * kWave + h];
  return r;
}

// power-of-two heads: all heads of the chunk at once, read once
__global__ __launch_bounds__(kBlock) void softmax_long_stats_kernel(
    const int32_t *__restrict__ pointer, const int32_t *__restrict__ row_of_slot,
    const int32_t *__restrict__ eid, const float *__restrict__ x,
    float *__restrict__ stats, int head_shift, int L, int long_min_deg) {
  __shared__ float lds[kBlock];
  int64_t lo, hi, c_first, c_last;
  if (!long_chunk(pointer, row_of_slot, L, long_min_deg, lo, hi, c_first, c_last))
    return;
  const int H = 1 << head_shift;
  const int64_t n = (hi - lo) << head_shift;    // < 2 * 1024 elements
  float c[8];
  float m = -INFINITY;
#pragma unroll
  for (int t = 0; t < 8; ++t) {
    const int64_t q = threadIdx.x + (int64_t)t * kBlock;
    c[t] = q < n ? x[elem_offset(eid, lo, q, head_shift)] : -INFINITY;
    m = fmaxf(m, c[t]);
  }
  m = block_reduce_heads<true>(m, H, lds);
  float l = 0.0f;
#pragma unroll
  for (int t = 0; t < 8; ++t) l += expf(c[t] - m);   // exp(-inf) == 0
  l = block_reduce_heads<false>(l, H, lds);
  if (threadIdx.x < H) {
    stats[((int64_t)blockIdx.x * H + threadIdx.x) * 2] = m;
    stats[((int64_t)blockIdx.x * H + threadIdx.x) * 2 + 1] = l;
  }
}

__global__ __launch_bounds__(kBlock) void softmax_long_write_kernel(
    const int32_t *__restrict__ pointer, const int32_t *__restrict__ row_of_slot,
    const int32_t *__restrict__ eid, const float *__restrict__ x,
    const float *__restrict__ stats, float *__restrict__ y, int head_shift, int L,
    int long_min_deg) {
  int64_t lo, hi, c_first, c_last;
  if (!long_chunk(pointer, row_of_slot, L, long_min_deg, lo, hi, c_first, c_last))
    return;
  const int H = 1 << head_shift;
  const int h = threadIdx.x & (H - 1);
  // merge the row's chunk statistics in chunk order (every lane, its own head)
  float m = -INFINITY;
  for (int64_t c = c_first; c <= c_last; ++c)
    m = fmaxf(m, stats[(c * H + h) * 2]);
  float l = 0.0f;
  for (int64_t c = c_first; c <= c_last; ++c)
    l += stats[(c * H + h) * 2 + 1] * expf(stats[(c * H + h) * 2] - m);
  const int64_t n = (hi - lo) << head_shift;
  for (int64_t q = threadIdx.x; q < n; q += kBlock) {
    const int64_t o = elem_offset(eid, lo, q, head_shift);
    y[o] = expf(x[o] - m) / l;
  }
}

// ---- any head count ---------------------------------------------------------
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
  __syncthreads();
  if ((threadIdx.x & (kWave - 1)) == 0) lds[wave] = v;
  __syncthreads();
  float r = lds[0];
  for (int q = 1; q < kBlock / kWave; ++q)
    r = IS_MAX ? fmaxf(r, lds[q]) : r + lds[q];
  return r;
}

__global__ __launch_bounds__(kBlock) void softmax_long_stats_generic_kernel(
    const int32_t *__restrict__ pointer, const int32_t *__restrict__ row_of_slot,
    const int32_t *__restrict__ eid, const float *__restrict__ x,
    float *__restrict__ stats, int heads) {
  __shared__ float lds[kBlock / kWave];
  int64_t lo, hi, c_first, c_last;
  if (!long_chunk(pointer, row_of_slot, kLongRow, kLongRow + 1, lo, hi, c_first,
                  c_last))
    return;
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

__global__ __launch_bounds__(kBlock) void softmax_long_write_generic_kernel(
    const int32_t *__restrict__ pointer, const int32_t *__restrict__ row_of_slot,
    const int32_t *__restrict__ eid, const float *__restrict__ x,
    const float *__restrict__ stats, float *__restrict__ y, int heads) {
  int64_t lo, hi, c_first, c_last;
  if (!long_chunk(pointer, row_of_slot, kLongRow, kLongRow + 1, lo, hi, c_first,
                  c_last))
    return;
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

inline bool pow2_heads(int64_t heads) {
  return (heads & (heads - 1)) == 0 && heads <= kWave;
}
// slots per long-row chunk
inline int long_chunk_slots(int64_t heads) {
  return pow2_heads(heads) ? (int)(kMediumMax / heads) : kLongRow;
}

}  // namespace
}  // namespace ga

extern "C" {

size_t ga_softmax_workspace_bytes(int64_t n_edges, int64_t heads) {
  if (n_edges <= 0 || heads <= 0) return 0;
  // (max, sum-exp) per head for every chunk of a long row
  const int64_t L = ga::long_chunk_slots(heads);
  if (n_edges <= L) return 0;
  const int64_t chunks = (n_edges + L - 1) / L;
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
  float *stats = (float *)workspace;
  const int L = long_chunk_slots(heads);
  const int64_t lchunks = (n_edges + L - 1) / L;
  if (lchunks > 0x7fffffff) return GA_EUNSUPPORTED;

  if (pow2_heads(heads)) {
    const int head_shift = ilog2_floor((uint64_t)heads);
    // lanes per small row: the register cache covers the mean segment
    const int64_t avg = (n_edges * heads + n_rows - 1) / n_rows;
    int s_shift = ilog2_ceil((uint64_t)((avg + kSmallCache - 1) / kSmallCache));
    // at least 16 lanes: medium rows then have > 64 elements, so a wave of the
    // medium kernel (one per 1024 elements) never meets more than 16 of them
    if (s_shift < 4) s_shift = 4;
    if (s_shift > 6) s_shift = 6;
    if (s_shift < head_shift) s_shift = head_shift;
    const int small_max = kSmallCache << s_shift;
    const int64_t per_block = kBlock >> s_shift;
    const int64_t blocks = (n_rows + per_block - 1) / per_block;
    if (blocks > 0x7fffffff) return GA_EUNSUPPORTED;
    hipLaunchKernelGGL(softmax_small_kernel, dim3((unsigned)blocks), dim3(kBlock),
                       0, s, pointer, eid, x, y, n_rows, head_shift, s_shift);
    if (small_max < kMediumMax) {
      const int64_t chunk_slots = kChunkElems >> head_shift;
      const int64_t chunks = (n_edges + chunk_slots - 1) / chunk_slots;
      const int64_t mblocks = (chunks + kBlock / kWave - 1) / (kBlock / kWave);
      hipLaunchKernelGGL(softmax_medium_kernel, dim3((unsigned)mblocks),
                         dim3(kBlock), 0, s, pointer, row_of_slot, eid, x, y,
                         n_rows, n_edges, head_shift, small_max);
    }
    if (n_edges > L) {
      const int long_min_deg = L + 1;   // n > 1024 elements
      hipLaunchKernelGGL(softmax_long_stats_kernel, dim3((unsigned)lchunks),
                         dim3(kBlock), 0, s, pointer, row_of_slot, eid, x, stats,
                         head_shift, L, long_min_deg);
      hipLaunchKernelGGL(softmax_long_write_kernel, dim3((unsigned)lchunks),
                         dim3(kBlock), 0, s, pointer, row_of_slot, eid, x, stats,
                         y, head_shift, L, long_min_deg);
    }
    return launch_status();
  }

  const int64_t avg = (n_edges + n_rows - 1) / n_rows;
  int s_shift = ilog2_ceil((uint64_t)(avg < 1 ? 1 : avg));
  if (s_shift < 2) s_shift = 2;
  if (s_shift > 6) s_shift = 6;
  const int64_t per_block = kBlock >> s_shift;
  const int64_t blocks = (n_rows + per_block - 1) / per_block;
  if (blocks > 0x7fffffff) return GA_EUNSUPPORTED;
  hipLaunchKernelGGL(softmax_rows_generic_kernel, dim3((unsigned)blocks),
                     dim3(kBlock), 0, s, pointer, eid, x, y, n_rows, (int)heads,
                     s_shift);
  if (n_edges > kLongRow) {
    hipLaunchKernelGGL(softmax_long_stats_generic_kernel, dim3((unsigned)lchunks),
                       dim3(kBlock), 0, s, pointer, row_of_slot, eid, x, stats,
                       (int)heads);
    hipLaunchKernelGGL(softmax_long_write_generic_kernel, dim3((unsigned)lchunks),
                       dim3(kBlock), 0, s, pointer, row_of_slot, eid, x, stats, y,
                       (int)heads);
  }
  return launch_status();
}

}  // extern "C"
