// Edge segment softmax for gfx950 (any number of heads), fp32.
//
// Up to 64 heads run a chunked, load-balanced scheme: the (slot, head) elements
// are cut into chunks of 1024 lane elements, one wavefront per chunk whatever the
// degree distribution.  Lane = (slot group g, head h) with the heads rounded up to a
// power of two (lanes of the padding heads idle); a lane owns 16 consecutive slots
// of its head, so
//   1. segments that lie inside one lane are reduced sequentially in registers;
//   2. segments shared by neighbouring lanes are combined with two segmented
//      shuffle scans over the lanes of a head (rows are sorted, so equal keys at
//      distance d imply equal keys in between);
//   3. rows that lie inside the chunk are normalised and written at once: their
//      logits are read exactly once;
//   4. the (at most two) rows a chunk shares with its neighbours leave their
//      per-head (max, sum-exp) in the workspace; a second launch merges the
//      partials of every such row once (one workgroup per row, so a row of any
//      length costs one pass over its partials), a third writes the elements.
// More than 64 heads use a lane-group kernel that runs the heads one after the
// other, with chunked two-pass handling of rows longer than 1024 slots.
// No atomics; the order of every reduction is fixed by the graph and sizes.
#include "common.h"

namespace ga {
namespace {

constexpr int kT = 16;                    // slots per lane
constexpr int kChunkElems = kWave * kT;   // 1024 elements per wavefront
constexpr int kLongRow = 1024;            // generic path: slots per long-row chunk

// exp(x) as exp2(x * log2 e) with the rounding error of the product fed back
// (x*log2e = t + r, exp2(t + r) ~ exp2(t) * (1 + r ln 2)): about 2 ulp, eight
// instructions instead of the library routine's thirty.  Arguments below -126
// (-inf included: a masked logit) are moved to -126, where the result is already
// 0 in fp32 -- the error term would be inf - inf there; NaN stays NaN.
__device__ __forceinline__ float exp_fast(float x) {
  x = x < -126.0f ? -126.0f : x;
  const float t = x * 1.44269502162933349609375f;
  const float r = fmaf(x, 1.44269502162933349609375f, -t) + x * 1.925963033e-8f;
  return __builtin_amdgcn_exp2f(t) * fmaf(r, 0.693147182464599609375f, 1.0f);
}

// The maximum of a piece of a row as the point its exponentials are taken from:
// a piece whose logits are all -inf (masked edges) has the maximum -inf, and
// exp(-inf - -inf) would be NaN; taken from 0 its elements weigh 0, and the
// piece's (max, sum) = (-inf, 0) merges as the empty state.
__device__ __forceinline__ float finite_or_zero(float m) {
  return m == -INFINITY ? 0.0f : m;
}

// Per-chunk partial statistics: [chunk][A|B][head][max, sum].  A = the chunk's
// first row when it began in an earlier chunk; B = its last row when that row
// started inside the chunk and continues in the next one.
__device__ __forceinline__ float *stat_ptr(float *stats, int64_t chunk, int which,
                                           int H, int h) {
  return stats + ((chunk * 2 + which) * H + h) * 2;
}

struct ChunkInfo {
  int64_t c0, c1;       // slot range of the chunk
  int row_first, row_last;
  bool began_before;    // first row started in an earlier chunk
  bool continues;       // last row goes on in the next chunk
};

__device__ __forceinline__ bool chunk_info(const int32_t *__restrict__ row_of_slot,
                                           int64_t n_edges, int head_shift,
                                           ChunkInfo &ci) {
  const int64_t chunk = ((int64_t)blockIdx.x * kBlock + threadIdx.x) / kWave;
  const int chunk_slots = kChunkElems >> head_shift;
  ci.c0 = chunk * chunk_slots;
  if (ci.c0 >= n_edges) return false;
  ci.c1 = min(ci.c0 + (int64_t)chunk_slots, n_edges);
  ci.row_first = row_of_slot[ci.c0];
  ci.row_last = row_of_slot[ci.c1 - 1];
  ci.began_before = ci.c0 > 0 && row_of_slot[ci.c0 - 1] == ci.row_first;
  ci.continues = ci.c1 < n_edges && row_of_slot[ci.c1] == ci.row_last;
  return true;
}

// Segmented scans over the lanes of one head (lanes at distance `step`
// multiples).  Keys ascend with the lane, so a match at distance d means every
// lane in between holds that key only.
template <bool IS_MAX>
__device__ __forceinline__ float scan_up(float v, int key, int lane, int step) {
  for (int off = step; off < kWave; off <<= 1) {
    const int pk = __shfl_up(key, off);
    const bool hit = lane >= off && pk == key;
    if (!__ballot(hit)) break;   // no match at this distance: none further away
    const float pv = __shfl_up(v, off);
    if (hit) v = IS_MAX ? fmaxf(v, pv) : v + pv;
  }
  return v;
}
template <bool IS_MAX>
__device__ __forceinline__ float scan_down(float v, int key, int lane, int step) {
  for (int off = step; off < kWave; off <<= 1) {
    const int nk = __shfl_down(key, off);
    const bool hit = lane + off < kWave && nk == key;
    if (!__ballot(hit)) break;
    const float nv = __shfl_down(v, off);
    if (hit) v = IS_MAX ? fmaxf(v, nv) : v + nv;
  }
  return v;
}

// Totals of a lane's first and last segment over the whole chunk, from the
// lane-local values vf (first segment) and vl (last segment).
template <bool IS_MAX>
__device__ __forceinline__ void chunk_totals(float vf, float vl, int kf, int kl,
                                             int lane, int H, float &tf, float &tl) {
  const float P = scan_up<IS_MAX>(vl, kl, lane, H);     // lanes <= me, key kl
  const float S = scan_down<IS_MAX>(vf, kf, lane, H);   // lanes >= me, key kf
  const int pk = __shfl_up(kl, H);
  const float pP = __shfl_up(P, H);
  const int nk = __shfl_down(kf, H);
  const float nS = __shfl_down(S, H);
  const float none = IS_MAX ? -INFINITY : 0.0f;
  const float prev = (lane >= H && pk == kf) ? pP : none;
  const float next = (lane + H < kWave && nk == kl) ? nS : none;
  tf = IS_MAX ? fmaxf(S, prev) : S + prev;
  tl = IS_MAX ? fmaxf(P, next) : P + next;
}

// Pass 1: one wavefront per chunk.  DIRECT: edge ids are slot numbers, so the
// chunk is one contiguous piece of x / y; it is moved with fully coalesced
// 16-byte accesses and re-distributed to the owning lanes through a padded,
// wave-private LDS tile.  Otherwise every element is gathered through eid.
// FULL: the chunk holds all 1024 elements (every chunk but the last), so no
// element needs a validity test.
template <bool DIRECT, bool FULL>
__device__ __forceinline__ void softmax_chunk_body(
    const int32_t *__restrict__ row_of_slot, const int32_t *__restrict__ eid,
    const float *__restrict__ x, float *__restrict__ y, float *__restrict__ stats,
    int64_t n_edges, int head_shift, int heads, int64_t chunk_id, int64_t c0, int64_t c1,
    float (*lds_v)[kChunkElems + kChunkElems / kT]) {
  const int H = 1 << head_shift;              // lanes per slot; heads <= H of them are live
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int g = lane >> head_shift, h = lane & (H - 1);
  const int64_t s0 = c0 + (int64_t)g * kT;   // first slot of this lane

  int key[kT];
  int64_t off[kT];
  float v[kT];
  const int64_t base_elem = c0 << head_shift;
  const int n_elem = (int)((c1 - c0) << head_shift);
  // LDS word of element q = (i*64 + lane)*4 + c of the chunk, as seen by the
  // lane that loads / stores it from global memory
  int lds_at[kChunkElems / (kWave * 4)][4];
  if (DIRECT) {
#pragma unroll
    for (int i = 0; i < kChunkElems / (kWave * 4); ++i)
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int q = (i * kWave + lane) * 4 + c;
        const int slot = q >> head_shift, hd = q & (H - 1);
        lds_at[i][c] = (((slot >> 4) << head_shift) + hd) * (kT + 1) + (slot & 15);
      }
    float *tv = lds_v[wave];
    int *tk = reinterpret_cast<int *>(lds_v[wave]);
    const int n_slots = (int)(c1 - c0);
    // all global loads first (keys and logits), then the two redistributions
    int4 kk[kChunkElems / (kWave * 4)];
    float4 xv[kChunkElems / (kWave * 4)];
#pragma unroll
    for (int i = 0; i < kChunkElems / (kWave * 4); ++i) {
      const int q = (i * kWave + lane) * 4;
      kk[i] = make_int4(-1, -1, -1, -1);
      if (FULL ? q < n_slots : q + 3 < n_slots) {
        kk[i] = *reinterpret_cast<const int4 *>(row_of_slot + c0 + q);
      } else if (!FULL && q < n_slots) {
        kk[i].x = row_of_slot[c0 + q];
        if (q + 1 < n_slots) kk[i].y = row_of_slot[c0 + q + 1];
        if (q + 2 < n_slots) kk[i].z = row_of_slot[c0 + q + 2];
      }
      xv[i] = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
      if (FULL || q + 3 < n_elem) {
        xv[i] = *reinterpret_cast<const float4 *>(x + base_elem + q);
      } else if (q < n_elem) {
        xv[i].x = x[base_elem + q];
        if (q + 1 < n_elem) xv[i].y = x[base_elem + q + 1];
        if (q + 2 < n_elem) xv[i].z = x[base_elem + q + 2];
      }
    }
#pragma unroll
    for (int i = 0; i < kChunkElems / (kWave * 4); ++i) {
      const int q = (i * kWave + lane) * 4;
      if (q < n_slots) {          // keys: one per slot, word slot + slot/16
        const int w = q + (q >> 4);
        tk[w] = kk[i].x; tk[w + 1] = kk[i].y; tk[w + 2] = kk[i].z; tk[w + 3] = kk[i].w;
      }
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int j = 0; j < kT; ++j)
      key[j] = (FULL || s0 + j < c1) ? tk[g * (kT + 1) + j] : -1;
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int i = 0; i < kChunkElems / (kWave * 4); ++i) {
      tv[lds_at[i][0]] = xv[i].x; tv[lds_at[i][1]] = xv[i].y;
      tv[lds_at[i][2]] = xv[i].z; tv[lds_at[i][3]] = xv[i].w;
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int j = 0; j < kT; ++j) {
      v[j] = (FULL || key[j] >= 0) ? tv[lane * (kT + 1) + j] : -INFINITY;
      off[j] = 0;
    }
    __builtin_amdgcn_wave_barrier();
  } else {
#pragma unroll
    for (int j = 0; j < kT; ++j) {
      const int64_t slot = s0 + j;
      const bool valid = FULL || (slot < c1 && h < heads);
      key[j] = valid ? row_of_slot[slot] : -1;
      const int64_t e = (valid && eid) ? (int64_t)eid[slot] : slot;
      off[j] = e * heads + h;
      v[j] = valid ? x[off[j]] : -INFINITY;
    }
  }
  // which rows does the chunk share with its neighbours?  (needed last)
  ChunkInfo ci;
  chunk_info(row_of_slot, n_edges, head_shift, ci);
  // ---- maxima ------------------------------------------------------------
  float m[kT];
  m[0] = v[0];
#pragma unroll
  for (int j = 1; j < kT; ++j)
    m[j] = key[j] == key[j - 1] ? fmaxf(m[j - 1], v[j]) : v[j];
#pragma unroll
  for (int j = kT - 2; j >= 0; --j)
    if (key[j] == key[j + 1]) m[j] = m[j + 1];
  const int kf = key[0], kl = key[kT - 1];
  float mf, ml;
  chunk_totals<true>(m[0], m[kT - 1], kf, kl, lane, H, mf, ml);
#pragma unroll
  for (int j = 0; j < kT; ++j) m[j] = key[j] == kf ? mf : (key[j] == kl ? ml : m[j]);
  // ---- sums of exponentials ------------------------------------------------
  float p[kT], l[kT];
#pragma unroll
  for (int j = 0; j < kT; ++j)
    p[j] = (FULL || key[j] >= 0) ? exp_fast(v[j] - finite_or_zero(m[j])) : 0.0f;
  l[0] = p[0];
#pragma unroll
  for (int j = 1; j < kT; ++j) l[j] = key[j] == key[j - 1] ? l[j - 1] + p[j] : p[j];
#pragma unroll
  for (int j = kT - 2; j >= 0; --j)
    if (key[j] == key[j + 1]) l[j] = l[j + 1];
  float lf, ll;
  chunk_totals<false>(l[0], l[kT - 1], kf, kl, lane, H, lf, ll);
  // ---- rows inside the chunk: done; boundary rows: leave their statistics --
  // (pass 2 rewrites every element of a boundary row, so DIRECT stores all)
  const float rf = __builtin_amdgcn_rcpf(lf), rl = __builtin_amdgcn_rcpf(ll);
  if (DIRECT) {
    float *tv = lds_v[wave];
#pragma unroll
    for (int j = 0; j < kT; ++j) {
      const float rt = key[j] == kf ? rf : (key[j] == kl ? rl : __builtin_amdgcn_rcpf(l[j]));
      tv[lane * (kT + 1) + j] = p[j] * rt;
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int i = 0; i < kChunkElems / (kWave * 4); ++i) {
      const int q = (i * kWave + lane) * 4;
      const float4 o = make_float4(tv[lds_at[i][0]], tv[lds_at[i][1]],
                                   tv[lds_at[i][2]], tv[lds_at[i][3]]);
      if (FULL || q + 3 < n_elem) {
        *reinterpret_cast<float4 *>(y + base_elem + q) = o;
      } else if (q < n_elem) {
        y[base_elem + q] = o.x;
        if (q + 1 < n_elem) y[base_elem + q + 1] = o.y;
        if (q + 2 < n_elem) y[base_elem + q + 2] = o.z;
      }
    }
  } else {
    const int skip_a = ci.began_before ? ci.row_first : -2;
    const int skip_b = ci.continues ? ci.row_last : -2;
#pragma unroll
    for (int j = 0; j < kT; ++j) {
      const float rt = key[j] == kf ? rf : (key[j] == kl ? rl : __builtin_amdgcn_rcpf(l[j]));
      if ((FULL || key[j] >= 0) && key[j] != skip_a && key[j] != skip_b)
        y[off[j]] = p[j] * rt;
    }
  }
  const int64_t chunk = chunk_id;
  if (ci.began_before && g == 0) {           // lanes 0..H-1 start with row_first
    float *st = stat_ptr(stats, chunk, 0, H, h);
    st[0] = mf;
    st[1] = lf;
  }
  if (ci.continues && !(ci.began_before && ci.row_first == ci.row_last) &&
      g == (kWave >> head_shift) - 1) {      // a continuing chunk is full
    float *st = stat_ptr(stats, chunk, 1, H, h);
    st[0] = ml;
    st[1] = ll;
  }
}

template <bool DIRECT>
__global__ __launch_bounds__(kBlock) void softmax_chunks_kernel(
    const int32_t *__restrict__ row_of_slot, const int32_t *__restrict__ eid,
    const float *__restrict__ x, float *__restrict__ y, float *__restrict__ stats,
    int64_t n_edges, int head_shift, int heads) {
  // per wave: one tile of 1024 words (+ one pad word per 16), used in turn for
  // the keys, the logits and the results
  __shared__ float lds_v[kBlock / kWave][kChunkElems + kChunkElems / kT];
  const int chunk_slots = kChunkElems >> head_shift;
  const int64_t chunk_id = ((int64_t)blockIdx.x * kBlock + threadIdx.x) / kWave;
  const int64_t c0 = chunk_id * chunk_slots;
  if (c0 >= n_edges) return;                                        // whole wave
  const int64_t c1 = min(c0 + (int64_t)chunk_slots, n_edges);
  // the variant without validity tests needs every lane live: a whole chunk and as
  // many heads as lanes per slot
  if (c1 - c0 == chunk_slots && heads == (1 << head_shift))
    softmax_chunk_body<DIRECT, true>(row_of_slot, eid, x, y, stats, n_edges,
                                     head_shift, heads, chunk_id, c0, c1, lds_v);
  else
    softmax_chunk_body<DIRECT, false>(row_of_slot, eid, x, y, stats, n_edges,
                                      head_shift, heads, chunk_id, c0, c1, lds_v);
}

// Pass 2: every row that starts in one chunk and continues into later ones gets its
// partials -- B of its first chunk, A of the following ones -- merged once, as
// (max, sum-exp) pairs: the chunk list is split over the lanes of a head, each lane
// folds its chunks in ascending order (four loads in flight), and a fixed tree
// combines the lanes.  The row's pair is left in the A slot of the row's second
// chunk, which nothing else reads.  Rows of up to kWaveMergeChunks chunks are merged
// by the wavefront of their first chunk (softmax_row_totals_kernel, same grid as
// pass 1); longer rows by a workgroup of 1024 lanes each (softmax_long_row_totals_
// kernel), so that a row of any length costs one parallel pass over its partials.
constexpr int kWaveMergeShift = 9;
constexpr int kWaveMergeChunks = 1 << kWaveMergeShift;
constexpr int kTotalsBlock = 1024;

// (m, l) <- (m, l) (+) (sm, sl).  The side that holds the maximum keeps its sum
// unscaled (also when both maxima are -inf: the sums are then 0 or NaN and stay
// so); the empty state (-inf, 0) scales by 0 (exp_fast has no value at -inf).
__device__ __forceinline__ void pair_merge(float &m, float &l, float sm, float sl) {
  const float nm = fmaxf(m, sm);
  const float a = m == nm ? 1.0f : (m == -INFINITY ? 0.0f : exp_fast(m - nm));
  const float b = sm == nm ? 1.0f : (sm == -INFINITY ? 0.0f : exp_fast(sm - nm));
  l = l * a + sl * b;
  m = nm;
}

// Lane (g, h) of G lane groups folds chunks k_lo + g, k_lo + g + G, ... <= k_hi of head h.
__device__ __forceinline__ void fold_row_partials(const float *__restrict__ stats, int64_t k_lo,
                                                  int64_t k_hi, int g, int G, int H, int h,
                                                  float &m, float &l) {
  m = -INFINITY;
  l = 0.0f;
  int64_t c = k_lo + g;
  if (g == 0) {                               // the B partial of the row's first chunk
    const float *st = stats + ((k_lo * 2 + 1) * H + h) * 2;
    m = st[0];
    l = st[1];
    c += G;
  }
  const int64_t step = (int64_t)2 * H * 2;    // floats from one chunk's A slot to the next
  const float *p = stats + ((c * 2) * H + h) * 2;
  for (; c + 3 * (int64_t)G <= k_hi; c += 4 * (int64_t)G, p += 4 * G * step) {
    float2 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = *reinterpret_cast<const float2 *>(p + u * G * step);
#pragma unroll
    for (int u = 0; u < 4; ++u) pair_merge(m, l, v[u].x, v[u].y);
  }
  for (; c <= k_hi; c += G, p += G * step) {
    const float2 v = *reinterpret_cast<const float2 *>(p);
    pair_merge(m, l, v.x, v.y);
  }
}

__global__ __launch_bounds__(kBlock) void softmax_row_totals_kernel(
    const int32_t *__restrict__ pointer, const int32_t *__restrict__ row_of_slot,
    float *__restrict__ stats, int64_t n_edges, int head_shift) {
  ChunkInfo ci;
  if (!chunk_info(row_of_slot, n_edges, head_shift, ci)) return;
  if (!ci.continues) return;
  const int cs_shift = 10 - head_shift;       // chunk_slots = 1024 >> head_shift
  const int64_t s = pointer[ci.row_last], e = pointer[ci.row_last + 1];
  if (s < ci.c0) return;                      // the row started in an earlier chunk
  const int64_t chunk = ci.c0 >> cs_shift, k_hi = (e - 1) >> cs_shift;
  if (k_hi - chunk >= kWaveMergeChunks) return;   // left to the workgroup kernel
  const int H = 1 << head_shift;
  const int lane = threadIdx.x & (kWave - 1);
  float m, l;
  fold_row_partials(stats, chunk, k_hi, lane >> head_shift, kWave >> head_shift, H,
                    lane & (H - 1), m, l);
  // butterfly over the lane groups; partner pairs are merged lower group first
  for (int o = H; o < kWave; o <<= 1) {
    const float pm = __shfl_xor(m, o), pl = __shfl_xor(l, o);
    if (lane & o) {
      float qm = pm, ql = pl;
      pair_merge(qm, ql, m, l);
      m = qm;
      l = ql;
    } else {
      pair_merge(m, l, pm, pl);
    }
  }
  if (lane < H) *reinterpret_cast<float2 *>(stat_ptr(stats, chunk + 1, 0, H, lane)) = make_float2(m, l);
}

// Workgroup j (>= 1) looks at the row that covers the first slot of chunk
// j * kWaveMergeChunks and merges it when it is longer than kWaveMergeChunks chunks
// and that chunk is the first multiple of kWaveMergeChunks after the row's first
// chunk -- every such row contains exactly one.
__global__ __launch_bounds__(kTotalsBlock) void softmax_long_row_totals_kernel(
    const int32_t *__restrict__ pointer, const int32_t *__restrict__ row_of_slot,
    float *__restrict__ stats, int head_shift) {
  __shared__ float2 red[kTotalsBlock];
  const int cs_shift = 10 - head_shift;
  const int64_t mark = ((int64_t)blockIdx.x + 1) << kWaveMergeShift;
  const int row = row_of_slot[mark << cs_shift];
  const int64_t s = pointer[row], e = pointer[row + 1];
  const int64_t k_lo = s >> cs_shift, k_hi = (e - 1) >> cs_shift;
  if (k_hi - k_lo < kWaveMergeChunks) return;
  if (((k_lo >> kWaveMergeShift) + 1) << kWaveMergeShift != mark) return;
  const int H = 1 << head_shift;
  const int h = threadIdx.x & (H - 1);
  float m, l;
  fold_row_partials(stats, k_lo, k_hi, threadIdx.x >> head_shift, kTotalsBlock >> head_shift,
                    H, h, m, l);
  red[threadIdx.x] = make_float2(m, l);
  __syncthreads();                            // also: every partial has been read
  for (int o = kTotalsBlock >> 1; o >= H; o >>= 1) {
    if ((int)threadIdx.x < o) {
      float2 p = red[threadIdx.x];
      const float2 q = red[threadIdx.x + o];
      pair_merge(p.x, p.y, q.x, q.y);
      red[threadIdx.x] = p;
    }
    __syncthreads();
  }
  if ((int)threadIdx.x < H)
    *reinterpret_cast<float2 *>(stat_ptr(stats, k_lo + 1, 0, H, h)) = red[h];
}

// Pass 3: the rows a chunk shares with its neighbours (A = first row, begun in
// an earlier chunk; B = last row, started here and continuing) are normalised with
// their merged statistics.  Both rows are handled side by side so their dependent
// loads overlap.
__global__ __launch_bounds__(kBlock) void softmax_boundary_kernel(
    const int32_t *__restrict__ pointer, const int32_t *__restrict__ row_of_slot,
    const int32_t *__restrict__ eid, const float *__restrict__ x,
    float *__restrict__ y, float *__restrict__ stats, int64_t n_edges,
    int head_shift, int heads) {
  ChunkInfo ci;
  if (!chunk_info(row_of_slot, n_edges, head_shift, ci)) return;
  const bool has_b = ci.continues && !(ci.began_before && ci.row_first == ci.row_last);
  if (!ci.began_before && !has_b) return;
  const int H = 1 << head_shift;
  const int G = kWave >> head_shift;
  const int lane = threadIdx.x & (kWave - 1);
  const int g = lane >> head_shift, h = lane & (H - 1);
  const int cs_shift = 10 - head_shift;       // chunk_slots = 1024 >> head_shift

  int64_t s[2] = {0, 0}, e[2] = {0, 0};
  if (ci.began_before) { s[0] = pointer[ci.row_first]; e[0] = pointer[ci.row_first + 1]; }
  if (has_b) { s[1] = pointer[ci.row_last]; e[1] = pointer[ci.row_last + 1]; }
  int64_t lo[2], hi[2], o0[2];
  float x0[2];
#pragma unroll
  for (int w = 0; w < 2; ++w) {            // first element of each row, early
    lo[w] = max(s[w], ci.c0);
    hi[w] = min(e[w], ci.c1);
    o0[w] = -1;
    x0[w] = 0.0f;
    if (lo[w] + g < hi[w] && h < heads) {
      const int64_t slot = lo[w] + g;
      const int64_t ed = eid ? (int64_t)eid[slot] : slot;
      o0[w] = ed * heads + h;
      x0[w] = x[o0[w]];
    }
  }
  float m[2], rcp_l[2];
#pragma unroll
  for (int w = 0; w < 2; ++w) {
    m[w] = 0.0f;
    rcp_l[w] = 0.0f;
    if (e[w] > s[w]) {      // totals of the row: A slot of its second chunk
      const float *t = stat_ptr(stats, (s[w] >> cs_shift) + 1, 0, H, h);
      m[w] = t[0];
      rcp_l[w] = __builtin_amdgcn_rcpf(t[1]);
    }
  }
#pragma unroll
  for (int w = 0; w < 2; ++w) {
    if (o0[w] >= 0) y[o0[w]] = exp_fast(x0[w] - m[w]) * rcp_l[w];
    // the rest of the row's slots in this chunk, eight loads in flight
    for (int64_t base = lo[w] + g + G; base < hi[w]; base += 8 * (int64_t)G) {
      int64_t o[8];
      float xv[8];
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const int64_t slot = base + (int64_t)t * G;
        o[t] = -1;
        xv[t] = 0.0f;
        if (slot < hi[w] && h < heads) {
          const int64_t ed = eid ? (int64_t)eid[slot] : slot;
          o[t] = ed * heads + h;
          xv[t] = x[o[t]];
        }
      }
#pragma unroll
      for (int t = 0; t < 8; ++t)
        if (o[t] >= 0) y[o[t]] = exp_fast(xv[t] - m[w]) * rcp_l[w];
    }
  }
}

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
    const float ref = finite_or_zero(m);
    float l = 0.0f;
    for (int64_t q = lo + threadIdx.x; q < hi; q += kBlock) {
      const int64_t e = eid ? (int64_t)eid[q] : q;
      l += expf(x[e * heads + h] - ref);
    }
    l = block_reduce<false>(l, lds);
    if (threadIdx.x == 0) {
      stats[((int64_t)blockIdx.x * heads + h) * 2] = m;
      stats[((int64_t)blockIdx.x * heads + h) * 2 + 1] = l;
    }
  }
}

// One workgroup per long row (the one that owns the row's first chunk) merges the
// row's per-chunk statistics and leaves the totals in the first chunk's place.
__global__ __launch_bounds__(kBlock) void softmax_long_totals_generic_kernel(
    const int32_t *__restrict__ pointer, const int32_t *__restrict__ row_of_slot,
    float *__restrict__ stats, int heads) {
  __shared__ float lds[kBlock / kWave];
  int64_t lo, hi, c_first, c_last;
  if (!long_chunk(pointer, row_of_slot, kLongRow, kLongRow + 1, lo, hi, c_first,
                  c_last))
    return;
  if ((int64_t)blockIdx.x != c_first) return;
  for (int h = 0; h < heads; ++h) {
    float m = -INFINITY;
    for (int64_t c = c_first + threadIdx.x; c <= c_last; c += kBlock)
      m = fmaxf(m, stats[(c * heads + h) * 2]);
    m = block_reduce<true>(m, lds);
    float l = 0.0f;
    for (int64_t c = c_first + threadIdx.x; c <= c_last; c += kBlock)
      l += stats[(c * heads + h) * 2 + 1] * expf(stats[(c * heads + h) * 2] - m);
    l = block_reduce<false>(l, lds);   // its barriers: every partial has been read
    if (threadIdx.x == 0) {
      stats[(c_first * heads + h) * 2] = m;
      stats[(c_first * heads + h) * 2 + 1] = l;
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
    const float m = stats[(c_first * heads + h) * 2];
    const float l = stats[(c_first * heads + h) * 2 + 1];
    for (int64_t q = lo + threadIdx.x; q < hi; q += kBlock) {
      const int64_t e = eid ? (int64_t)eid[q] : q;
      y[e * heads + h] = expf(x[e * heads + h] - m) / l;
    }
  }
}

// Head counts up to a wavefront run the chunked scheme with the lanes per slot
// rounded up to a power of two (3 heads: 4 lanes, one idle); more heads the generic
// kernels.
inline bool chunked_heads(int64_t heads) { return heads <= kWave; }
inline int lanes_per_slot_shift(int64_t heads) { return ilog2_ceil((uint64_t)heads); }

}  // namespace
}  // namespace ga

extern "C" {

size_t ga_softmax_workspace_bytes(int64_t n_edges, int64_t heads) {
  if (n_edges <= 0 || heads <= 0) return 0;
  if (ga::chunked_heads(heads)) {
    // two partial (max, sum) pairs per lane of a slot for every chunk of 1024 lanes' elements
    const int shift = ga::lanes_per_slot_shift(heads);
    const int64_t chunk_slots = ga::kChunkElems >> shift;
    const int64_t chunks = (n_edges + chunk_slots - 1) / chunk_slots;
    return (size_t)chunks * 2 * ((size_t)1 << shift) * 2 * sizeof(float);
  }
  if (n_edges <= ga::kLongRow) return 0;
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
  float *stats = (float *)workspace;

  if (chunked_heads(heads)) {
    const int head_shift = lanes_per_slot_shift(heads);
    const bool every_lane_live = heads == ((int64_t)1 << head_shift);
    const int64_t chunk_slots = kChunkElems >> head_shift;
    const int64_t chunks = (n_edges + chunk_slots - 1) / chunk_slots;
    const int64_t blocks = (chunks + kBlock / kWave - 1) / (kBlock / kWave);
    if (blocks > 0x7fffffff) return GA_EUNSUPPORTED;
    if (every_lane_live && !eid && aligned(x, 16) && aligned(y, 16) && aligned(row_of_slot, 16))
      hipLaunchKernelGGL(softmax_chunks_kernel<true>, dim3((unsigned)blocks),
                         dim3(kBlock), 0, s, row_of_slot, eid, x, y, stats,
                         n_edges, head_shift, (int)heads);
    else
      hipLaunchKernelGGL(softmax_chunks_kernel<false>, dim3((unsigned)blocks),
                         dim3(kBlock), 0, s, row_of_slot, eid, x, y, stats,
                         n_edges, head_shift, (int)heads);
    if (chunks > 1) {
      hipLaunchKernelGGL(softmax_row_totals_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, s,
                         pointer, row_of_slot, stats, n_edges, head_shift);
      const int64_t marks = (chunks - 1) >> kWaveMergeShift;   // multiples of the limit below `chunks`
      if (marks > 0)
        hipLaunchKernelGGL(softmax_long_row_totals_kernel, dim3((unsigned)marks),
                           dim3(kTotalsBlock), 0, s, pointer, row_of_slot, stats, head_shift);
      hipLaunchKernelGGL(softmax_boundary_kernel, dim3((unsigned)blocks),
                         dim3(kBlock), 0, s, pointer, row_of_slot, eid, x, y, stats,
                         n_edges, head_shift, (int)heads);
    }
    return launch_status();
  }

  const int64_t lchunks = (n_edges + kLongRow - 1) / kLongRow;
  if (lchunks > 0x7fffffff) return GA_EUNSUPPORTED;
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
    hipLaunchKernelGGL(softmax_long_totals_generic_kernel, dim3((unsigned)lchunks),
                       dim3(kBlock), 0, s, pointer, row_of_slot, stats, (int)heads);
    hipLaunchKernelGGL(softmax_long_write_generic_kernel, dim3((unsigned)lchunks),
                       dim3(kBlock), 0, s, pointer, row_of_slot, eid, x, stats, y,
                       (int)heads);
  }
  return launch_status();
}

}  // extern "C"
