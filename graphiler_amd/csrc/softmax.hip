// Edge segment softmax for gfx950 (any number of heads), fp32.
//
// Rows are owned by lane groups: a group of S adjacent lanes (S a power of two
// picked from the average segment size) handles one destination row, keeps up
// to kCache elements per lane in registers so a typical segment is read once,
// and reduces max / sum with a fixed xor-shuffle tree.  Rows longer than
// kLongRow slots are skipped there and handled by one whole workgroup each
// (found without any list: the workgroup whose first slot is the first multiple
// of kLongRow inside the row owns it).  No atomics; order is fixed.
#include "common.h"

namespace ga {
namespace {

constexpr int kCache = 4;
constexpr int kLongRow = 2048;

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

// One workgroup per row longer than kLongRow slots.
__global__ __launch_bounds__(kBlock) void softmax_long_rows_kernel(
    const int32_t *__restrict__ pointer, const int32_t *__restrict__ row_of_slot,
    const int32_t *__restrict__ eid, const float *__restrict__ x,
    float *__restrict__ y, int heads) {
  __shared__ float lds[kBlock / kWave];
  const int64_t first_slot = (int64_t)blockIdx.x * kLongRow;
  const int row = row_of_slot[first_slot];
  const int64_t start = pointer[row];
  const int64_t deg = pointer[row + 1] - start;
  // owner = the workgroup at the first multiple of kLongRow that is >= start
  if (deg <= kLongRow || (start + kLongRow - 1) / kLongRow != blockIdx.x) return;
  for (int h = 0; h < heads; ++h) {
    float m = -INFINITY;
    for (int64_t q = threadIdx.x; q < deg; q += kBlock) {
      const int64_t e = eid ? (int64_t)eid[start + q] : start + q;
      m = fmaxf(m, x[e * heads + h]);
    }
    m = block_reduce<true>(m, lds);
    float l = 0.0f;
    for (int64_t q = threadIdx.x; q < deg; q += kBlock) {
      const int64_t e = eid ? (int64_t)eid[start + q] : start + q;
      l += expf(x[e * heads + h] - m);
    }
    l = block_reduce<false>(l, lds);
    for (int64_t q = threadIdx.x; q < deg; q += kBlock) {
      const int64_t e = eid ? (int64_t)eid[start + q] : start + q;
      y[e * heads + h] = expf(x[e * heads + h] - m) / l;
    }
  }
}

}  // namespace
}  // namespace ga

extern "C" int ga_segment_softmax(const int32_t *pointer,
                                  const int32_t *row_of_slot,
                                  const int32_t *eid, const float *x, float *y,
                                  int64_t n_rows, int64_t n_edges,
                                  int64_t heads, ga_stream_t stream) {
  using namespace ga;
  if (n_rows < 0 || n_edges < 0 || heads <= 0) return GA_EINVAL;
  if (n_rows > 0x7fffffff || n_edges > 0x7fffffff || heads > 65536)
    return GA_EINVAL;
  if (n_rows == 0 || n_edges == 0) return GA_OK;
  if (!pointer || !row_of_slot || !x || !y) return GA_EINVAL;
  if (!aligned(x, 4) || !aligned(y, 4)) return GA_EALIGN;
  hipStream_t s = (hipStream_t)stream;

  const bool pow2 = (heads & (heads - 1)) == 0 && heads <= kWave;
  const int64_t avg = (n_edges * (pow2 ? heads : 1) + n_rows - 1) / n_rows;
  int s_shift = ilog2_ceil((uint64_t)(avg < 1 ? 1 : avg));
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
    const int64_t lblocks = (n_edges + kLongRow - 1) / kLongRow;
    hipLaunchKernelGGL(softmax_long_rows_kernel, dim3((unsigned)lblocks),
                       dim3(kBlock), 0, s, pointer, row_of_slot, eid, x, y,
                       (int)heads);
  }
  return launch_status();
}
