// Edge segment softmax for gfx950 (any number of heads), fp32.
//
// Up to 64 heads run a tiled, load-balanced scheme: the (slot, head) elements are
// cut into chunks of 1024 lane elements, one wavefront per chunk whatever the
// degree distribution, and kTileWaves consecutive chunks form the tile of one
// workgroup.  Lane = (slot group g, head h) with the heads rounded up to a power of
// two (lanes of the padding heads idle); a lane owns 16 consecutive slots of its
// head, so
//   1. segments that lie inside one lane are reduced sequentially in registers;
//   2. segments shared by neighbouring lanes are combined with two segmented
//      shuffle scans over the lanes of a head (rows are sorted, so equal keys at
//      distance d imply equal keys in between);
//   3. segments shared by neighbouring wavefronts of the tile are combined as
//      (max, sum-exp) pairs through LDS, after one workgroup barrier;
//   4. rows that lie inside the tile are normalised and written at once: their
//      logits are read exactly once and stay in registers meanwhile;
//   5. the (at most two) rows a tile shares with its neighbours leave their
//      per-head pair in the workspace; a second launch folds every such row's
//      pairs and writes the row's elements, tile by tile.
// The rows of a chunk's slots come from the row pointer (the row starts inside
// the chunk), not from the slot -> row column, which is read at the two ends of a
// chunk only: 4 bytes per row instead of 4 bytes per slot.
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

// Partial statistics of rows that leave a tile: [tile][A|B][head][max, sum].
// A = the tile's first row when it began in an earlier tile; B = its last row
// when that row started inside the tile and continues in the next one.
__device__ __forceinline__ float *stat_ptr(float *stats, int64_t tile, int which,
                                           int H, int h) {
  return stats + ((tile * 2 + which) * H + h) * 2;
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

// (m, l) <- (m, l) (+) (sm, sl).  The side that holds the maximum keeps its sum
// unscaled (also when both maxima are -inf: the sums are then 0 or NaN and stay
// so); the empty state (-inf, 0) scales by 0.
__device__ __forceinline__ void pair_merge(float &m, float &l, float sm, float sl) {
  const float nm = fmaxf(m, sm);
  const float a = m == nm ? 1.0f : (m == -INFINITY ? 0.0f : exp_fast(m - nm));
  const float b = sm == nm ? 1.0f : (sm == -INFINITY ? 0.0f : exp_fast(sm - nm));
  l = l * a + sl * b;
  m = nm;
}

// ---- pass 1: tiles ----------------------------------------------------------
// A workgroup of W wavefronts owns a tile of W chunks; wavefront w owns chunk
// tile * W + w (1024 lane elements) and keeps it in registers from the load of the
// logits to the store of the results.
constexpr int kTileWaves = 8;                              // wavefronts (chunks) per tile
constexpr int kTilePad = kChunkElems + kChunkElems / kT;   // LDS words per wavefront

// What a wavefront tells the other wavefronts of its tile about its chunk.
constexpr int kActive = 1;      // the chunk holds slots
constexpr int kBegan = 2;       // its first row began before the chunk
constexpr int kContinues = 4;   // its last row continues past the chunk
constexpr int kSingle = 8;      // first row == last row
// a row passes straight through a chunk: began before, fills it, continues
__device__ __forceinline__ bool passes_through(int flags) {
  return (flags & (kBegan | kContinues | kSingle)) == (kBegan | kContinues | kSingle);
}

struct ChunkRows {
  int64_t c0, c1;       // slot range
  int row_first, row_last;
  bool began_before, continues, has_b;
};

// Per-lane state that lives from the reduction (before the workgroup barrier) to
// the store (after it).
template <bool DIRECT>
struct LaneRows {
  int key[kT];          // row of each of the lane's slots, -1 for none
  float p[kT];          // exp(logit - maximum of the segment inside this chunk)
  float l[kT];          // sum of p over the lane's part of the segment
  float raw[DIRECT ? kT : 1];        // DIRECT: the logits (written back for rows that leave the tile)
  int64_t off[DIRECT ? 1 : kT];      // gathered: element offsets
  float mf, ml, lf, ll; // chunk-wide (max, sum) of the lane's first / last segment
};

// Rows of the lane's 16 slots without reading the slot -> row column: the row
// that holds the chunk's first slot and the one that holds its last come from
// that column (two reads per chunk), the row starts in between from the row
// pointer -- each row that starts inside the chunk marks its first slot in a
// wave-private LDS tile, a lane reads its 16 marks, and what lies before a
// lane's first mark is the largest mark of the lanes before it (rows ascend
// with the slot), found with a scan over the lanes.
__device__ __forceinline__ void rows_of_chunk(const int32_t *__restrict__ pointer,
                                              const ChunkRows &cr, int head_shift, int lane,
                                              int *tile, int (&key)[kT]) {
  const int H = 1 << head_shift;
  const int g = lane >> head_shift;
  const int chunk_slots = kChunkElems >> head_shift;
#pragma unroll
  for (int i = 0; i < kT; ++i) {
    const int q = i * kWave + lane;
    if (q < chunk_slots) tile[q + (q >> 4)] = -1;
  }
  __builtin_amdgcn_wave_barrier();
  for (int r = cr.row_first + 1 + lane; r <= cr.row_last; r += kWave) {
    const int s = pointer[r], e = pointer[r + 1];
    if (e > s) {                                  // rows without edges own no slot
      const int q = (int)(s - cr.c0);
      tile[q + (q >> 4)] = r;
    }
  }
  __builtin_amdgcn_wave_barrier();
  int last = -1;
#pragma unroll
  for (int j = 0; j < kT; ++j) {
    key[j] = tile[g * (kT + 1) + j];
    last = max(last, key[j]);
  }
  __builtin_amdgcn_wave_barrier();
  int inc = last;                                 // largest mark of lanes <= me (same head)
  for (int off = H; off < kWave; off <<= 1) {
    const int t = __shfl_up(inc, off);
    if (lane >= off) inc = max(inc, t);
  }
  int before = __shfl_up(inc, H);
  before = lane >= H ? max(before, cr.row_first) : cr.row_first;
#pragma unroll
  for (int j = 0; j < kT; ++j) {
    if (key[j] < 0) key[j] = before;
    before = key[j];
  }
}

// Reduction of one chunk.  DIRECT: edge ids are slot numbers, so the chunk is
// one contiguous piece of x / y; it is moved with fully coalesced 16-byte
// accesses and re-distributed to the owning lanes through the padded,
// wave-private LDS tile.  Otherwise every element is gathered through eid.
// FULL: the chunk holds all 1024 elements and every lane is live, so no element
// needs a validity test.
template <bool DIRECT, bool FULL>
__device__ __forceinline__ void chunk_reduce(
    const int32_t *__restrict__ pointer, const int32_t *__restrict__ eid,
    const float *__restrict__ x, const ChunkRows &cr, int head_shift, int heads,
    float *tile, LaneRows<DIRECT> &S) {
  const int H = 1 << head_shift;              // lanes per slot; heads <= H of them are live
  const int lane = threadIdx.x & (kWave - 1);
  const int g = lane >> head_shift, h = lane & (H - 1);
  const int64_t s0 = cr.c0 + (int64_t)g * kT;   // first slot of this lane
  const int64_t base_elem = cr.c0 << head_shift;
  const int n_elem = (int)((cr.c1 - cr.c0) << head_shift);
  float v[kT];
  float4 xv[kChunkElems / (kWave * 4)];
  if (DIRECT) {                               // the logits first: they depend on nothing
#pragma unroll
    for (int i = 0; i < kChunkElems / (kWave * 4); ++i) {
      const int q = (i * kWave + lane) * 4;
      xv[i] = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
      if (FULL || q + 3 < n_elem) {
        xv[i] = *reinterpret_cast<const float4 *>(x + base_elem + q);
      } else if (q < n_elem) {
        xv[i].x = x[base_elem + q];
        if (q + 1 < n_elem) xv[i].y = x[base_elem + q + 1];
        if (q + 2 < n_elem) xv[i].z = x[base_elem + q + 2];
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < kT; ++j) {
      const int64_t slot = s0 + j;
      const bool valid = FULL || (slot < cr.c1 && h < heads);
      const int64_t e = (valid && eid) ? (int64_t)eid[slot] : slot;
      S.off[j] = e * heads + h;
      v[j] = valid ? x[S.off[j]] : -INFINITY;
    }
  }
  rows_of_chunk(pointer, cr, head_shift, lane, reinterpret_cast<int *>(tile), S.key);
  if (!FULL) {
#pragma unroll
    for (int j = 0; j < kT; ++j)
      if (!(s0 + j < cr.c1 && h < heads)) S.key[j] = -1;
  }
  if (DIRECT) {
#pragma unroll
    for (int i = 0; i < kChunkElems / (kWave * 4); ++i)
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int q = (i * kWave + lane) * 4 + c;
        const int slot = q >> head_shift, hd = q & (H - 1);
        const float xe = c == 0 ? xv[i].x : (c == 1 ? xv[i].y : (c == 2 ? xv[i].z : xv[i].w));
        tile[(((slot >> 4) << head_shift) + hd) * (kT + 1) + (slot & 15)] = xe;
      }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int j = 0; j < kT; ++j) {
      v[j] = (FULL || S.key[j] >= 0) ? tile[lane * (kT + 1) + j] : -INFINITY;
      S.raw[j] = v[j];
    }
    __builtin_amdgcn_wave_barrier();
  }
  // ---- maxima ------------------------------------------------------------
  float m[kT];
  m[0] = v[0];
#pragma unroll
  for (int j = 1; j < kT; ++j)
    m[j] = S.key[j] == S.key[j - 1] ? fmaxf(m[j - 1], v[j]) : v[j];
#pragma unroll
  for (int j = kT - 2; j >= 0; --j)
    if (S.key[j] == S.key[j + 1]) m[j] = m[j + 1];
  const int kf = S.key[0], kl = S.key[kT - 1];
  chunk_totals<true>(m[0], m[kT - 1], kf, kl, lane, H, S.mf, S.ml);
#pragma unroll
  for (int j = 0; j < kT; ++j) m[j] = S.key[j] == kf ? S.mf : (S.key[j] == kl ? S.ml : m[j]);
  // ---- sums of exponentials ------------------------------------------------
#pragma unroll
  for (int j = 0; j < kT; ++j)
    S.p[j] = (FULL || S.key[j] >= 0) ? exp_fast(v[j] - finite_or_zero(m[j])) : 0.0f;
  S.l[0] = S.p[0];
#pragma unroll
  for (int j = 1; j < kT; ++j) S.l[j] = S.key[j] == S.key[j - 1] ? S.l[j - 1] + S.p[j] : S.p[j];
#pragma unroll
  for (int j = kT - 2; j >= 0; --j)
    if (S.key[j] == S.key[j + 1]) S.l[j] = S.l[j + 1];
  chunk_totals<false>(S.l[0], S.l[kT - 1], kf, kl, lane, H, S.lf, S.ll);
}

// After the workgroup barrier: the (max, sum) pairs of the rows a chunk shares
// with other chunks of the tile are in LDS (pair_a / pair_b per wavefront, with
// each wavefront's flags).  Rows that end up complete are normalised and stored;
// rows that leave the tile leave their pair for the tile in `stats` and keep
// their logits (DIRECT: written back unchanged, so that y may be x; gathered:
// not written) for the second pass.
template <bool DIRECT, bool FULL, int W>
__device__ __forceinline__ void chunk_store(
    const ChunkRows &cr, float *__restrict__ y, float *__restrict__ stats, int head_shift,
    int heads, int wave, const int *wflags, const float2 *pair_a, const float2 *pair_b,
    float *tile, const LaneRows<DIRECT> &S) {
  const int H = 1 << head_shift;
  const int lane = threadIdx.x & (kWave - 1);
  const int g = lane >> head_shift, h = lane & (H - 1);
  const int64_t tile_id = blockIdx.x;
  // pairs are stored [wavefront][head] with 64 heads per wavefront
  auto pa = [&](int w) { return pair_a[w * kWave + h]; };
  auto pb = [&](int w) { return pair_b[w * kWave + h]; };
  float scale_a = 0.0f, scale_b = 0.0f;
  bool open_a = false, open_b = false;
  if (cr.began_before) {                    // the chunk's first row
    int j = wave - 1;
    while (j >= 0 && passes_through(wflags[j])) --j;
    const bool open_left = j < 0;           // it began before the tile
    int k = wave;
    if (passes_through(wflags[wave])) {
      k = wave + 1;
      while (k < W && passes_through(wflags[k])) ++k;
    }
    const bool open_right = k >= W;         // it continues past the tile
    const int end = open_right ? W - 1 : k;
    float M = -INFINITY, L = 0.0f;
    if (!open_left) {
      const float2 t = pb(j);
      M = t.x;
      L = t.y;
    }
    for (int q = open_left ? 0 : j + 1; q <= end; ++q) {
      const float2 t = pa(q);
      pair_merge(M, L, t.x, t.y);
    }
    open_a = open_left || open_right;
    if (open_a && g == 0) {
      if (open_left && wave == 0)
        *reinterpret_cast<float2 *>(stat_ptr(stats, tile_id, 0, H, h)) = make_float2(M, L);
      if (!open_left && wave == W - 1)
        *reinterpret_cast<float2 *>(stat_ptr(stats, tile_id, 1, H, h)) = make_float2(M, L);
    }
    scale_a = S.mf == -INFINITY ? 0.0f : exp_fast(S.mf - M) * __builtin_amdgcn_rcpf(L);
  }
  if (cr.has_b) {                           // the chunk's last row, begun in this chunk
    int k = wave + 1;
    while (k < W && passes_through(wflags[k])) ++k;
    open_b = k >= W;
    const int end = open_b ? W - 1 : k;
    const float2 t0 = pb(wave);
    float M = t0.x, L = t0.y;
    for (int q = wave + 1; q <= end; ++q) {
      const float2 t = pa(q);
      pair_merge(M, L, t.x, t.y);
    }
    if (open_b && g == 0 && wave == W - 1)
      *reinterpret_cast<float2 *>(stat_ptr(stats, tile_id, 1, H, h)) = make_float2(M, L);
    scale_b = S.ml == -INFINITY ? 0.0f : exp_fast(S.ml - M) * __builtin_amdgcn_rcpf(L);
  }
  const int kf = S.key[0], kl = S.key[kT - 1];
  const float rf = __builtin_amdgcn_rcpf(S.lf), rl = __builtin_amdgcn_rcpf(S.ll);
  const int key_a = cr.began_before ? cr.row_first : -2;
  const int key_b = cr.has_b ? cr.row_last : -2;
  float o[kT];
  bool keep[kT];
#pragma unroll
  for (int j = 0; j < kT; ++j) {
    const int kj = S.key[j];
    float rt = kj == kf ? rf : (kj == kl ? rl : __builtin_amdgcn_rcpf(S.l[j]));
    bool open = false;
    if (kj == key_a) {
      rt = scale_a;
      open = open_a;
    } else if (kj == key_b) {
      rt = scale_b;
      open = open_b;
    }
    o[j] = S.p[j] * rt;
    keep[j] = open;
    if (DIRECT && open) o[j] = S.raw[j];
  }
  if (DIRECT) {
    const int64_t base_elem = cr.c0 << head_shift;
    const int n_elem = (int)((cr.c1 - cr.c0) << head_shift);
#pragma unroll
    for (int j = 0; j < kT; ++j) tile[lane * (kT + 1) + j] = o[j];
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int i = 0; i < kChunkElems / (kWave * 4); ++i) {
      const int q = (i * kWave + lane) * 4;
      float e[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int qq = q + c;
        const int slot = qq >> head_shift, hd = qq & (H - 1);
        e[c] = tile[(((slot >> 4) << head_shift) + hd) * (kT + 1) + (slot & 15)];
      }
      if (FULL || q + 3 < n_elem) {
        *reinterpret_cast<float4 *>(y + base_elem + q) = make_float4(e[0], e[1], e[2], e[3]);
      } else if (q < n_elem) {
        y[base_elem + q] = e[0];
        if (q + 1 < n_elem) y[base_elem + q + 1] = e[1];
        if (q + 2 < n_elem) y[base_elem + q + 2] = e[2];
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < kT; ++j)
      if ((FULL || S.key[j] >= 0) && !keep[j]) y[S.off[j]] = o[j];
  }
}

template <bool DIRECT, int W>
__global__ __launch_bounds__(W *kWave) void softmax_tiles_kernel(
    const int32_t *__restrict__ pointer, const int32_t *__restrict__ row_of_slot,
    const int32_t *__restrict__ eid, const float *__restrict__ x, float *__restrict__ y,
    float *__restrict__ stats, int64_t n_edges, int head_shift, int heads) {
  // per wavefront: one tile of 1024 words (+ one pad word per 16), used in turn for
  // the row marks, the logits and the results
  __shared__ float lds_tile[W][kTilePad];
  __shared__ float2 pair_a[W * kWave], pair_b[W * kWave];
  __shared__ int wflags[W];
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  const int H = 1 << head_shift;
  const int chunk_slots = kChunkElems >> head_shift;
  const int64_t chunk_id = (int64_t)blockIdx.x * W + wave;
  ChunkRows cr;
  cr.c0 = chunk_id * chunk_slots;
  const bool active = cr.c0 < n_edges;                                // whole wavefront
  cr.c1 = min(cr.c0 + (int64_t)chunk_slots, n_edges);
  // the variant without validity tests needs every lane live: a whole chunk and as
  // many heads as lanes per slot
  const bool full = active && cr.c1 - cr.c0 == chunk_slots && heads == H;
  LaneRows<DIRECT> S;
  int flags = 0;
  if (active) {
    cr.row_first = row_of_slot[cr.c0];
    cr.row_last = row_of_slot[cr.c1 - 1];
    cr.began_before = pointer[cr.row_first] < cr.c0;
    cr.continues = pointer[cr.row_last + 1] > cr.c1;
    cr.has_b = cr.continues && !(cr.began_before && cr.row_first == cr.row_last);
    if (full)
      chunk_reduce<DIRECT, true>(pointer, eid, x, cr, head_shift, heads, lds_tile[wave], S);
    else
      chunk_reduce<DIRECT, false>(pointer, eid, x, cr, head_shift, heads, lds_tile[wave], S);
    flags = kActive | (cr.began_before ? kBegan : 0) | (cr.continues ? kContinues : 0) |
            (cr.row_first == cr.row_last ? kSingle : 0);
    const int g = lane >> head_shift, h = lane & (H - 1);
    if (cr.began_before && g == 0)            // lanes 0..H-1 start with row_first
      pair_a[wave * kWave + h] = make_float2(S.mf, S.lf);
    if (cr.has_b && g == (kWave >> head_shift) - 1)   // a continuing chunk is full
      pair_b[wave * kWave + h] = make_float2(S.ml, S.ll);
  }
  if (lane == 0) wflags[wave] = flags;
  __syncthreads();
  if (!active) return;
  if (full)
    chunk_store<DIRECT, true, W>(cr, y, stats, head_shift, heads, wave, wflags, pair_a, pair_b,
                                 lds_tile[wave], S);
  else
    chunk_store<DIRECT, false, W>(cr, y, stats, head_shift, heads, wave, wflags, pair_a, pair_b,
                                  lds_tile[wave], S);
}

// ---- pass 2: rows that leave a tile -------------------------------------------
// One workgroup per tile.  For the (at most two) rows the tile shares with its
// neighbours -- A: its first row, begun in an earlier tile; B: its last row,
// started here and continuing -- the row's pair is folded from the tiles' partials
// (B of the row's first tile, then A of the following ones, in tile order: every
// tile of a row folds the same chain and gets the same pair), and the row's
// elements inside this tile are normalised with it.  Chains of up to kShortChain
// tiles are folded by every lane of a head for itself; longer ones are cut into a
// piece per lane group, folded in parallel and combined in order.
constexpr int kFixBlock = 256;
constexpr int kShortChain = 16;

__global__ __launch_bounds__(kFixBlock) void softmax_tile_rows_kernel(
    const int32_t *__restrict__ pointer, const int32_t *__restrict__ row_of_slot,
    const int32_t *__restrict__ eid, const float *__restrict__ x, float *__restrict__ y,
    const float *__restrict__ stats, int64_t n_edges, int head_shift, int heads,
    int tile_shift) {
  __shared__ float2 piece[kFixBlock];
  __shared__ float2 total[kWave];
  const int64_t t0 = (int64_t)blockIdx.x << tile_shift;
  const int64_t t1 = min(t0 + ((int64_t)1 << tile_shift), n_edges);
  const int row_first = row_of_slot[t0], row_last = row_of_slot[t1 - 1];
  const bool began_before = pointer[row_first] < t0;
  const bool continues = pointer[row_last + 1] > t1;
  const bool has_b = continues && !(began_before && row_first == row_last);
  if (!began_before && !has_b) return;                      // whole workgroup
  const int H = 1 << head_shift;
  const int G = kFixBlock >> head_shift;
  const int g = threadIdx.x >> head_shift, h = threadIdx.x & (H - 1);
  for (int which = 0; which < 2; ++which) {
    if (which == 0 ? !began_before : !has_b) continue;      // whole workgroup
    const int row = which == 0 ? row_first : row_last;
    const int64_t s = pointer[row], e = pointer[row + 1];
    const int64_t k_lo = s >> tile_shift, k_hi = (e - 1) >> tile_shift;
    const int64_t len = k_hi - k_lo + 1;                    // states: B of k_lo, A of k_lo+1 .. k_hi
    const float *a_of = stats + (size_t)h * 2;              // A pair of tile k: a_of[k * 4H]
    const size_t step = (size_t)4 * H;
    float M, L;
    if (len <= kShortChain) {
      const float2 b0 = *reinterpret_cast<const float2 *>(a_of + k_lo * step + 2 * H);
      M = b0.x;
      L = b0.y;
      for (int64_t k = k_lo + 1; k <= k_hi; ++k) {
        const float2 t = *reinterpret_cast<const float2 *>(a_of + k * step);
        pair_merge(M, L, t.x, t.y);
      }
    } else {
      // piece g: states [len*g/G, len*(g+1)/G) of the chain
      const int64_t w0 = len * g / G, w1 = len * (g + 1) / G;
      M = -INFINITY;
      L = 0.0f;
      int64_t w = w0;
      if (w == 0 && w1 > 0) {
        const float2 b0 = *reinterpret_cast<const float2 *>(a_of + k_lo * step + 2 * H);
        M = b0.x;
        L = b0.y;
        w = 1;
      }
      for (; w + 4 <= w1; w += 4) {
        float2 t[4];
#pragma unroll
        for (int u = 0; u < 4; ++u)
          t[u] = *reinterpret_cast<const float2 *>(a_of + (k_lo + w + u) * step);
#pragma unroll
        for (int u = 0; u < 4; ++u) pair_merge(M, L, t[u].x, t[u].y);
      }
      for (; w < w1; ++w) {
        const float2 t = *reinterpret_cast<const float2 *>(a_of + (k_lo + w) * step);
        pair_merge(M, L, t.x, t.y);
      }
      __syncthreads();                                      // `piece` free again
      piece[threadIdx.x] = make_float2(M, L);
      __syncthreads();
      M = -INFINITY;
      L = 0.0f;
      for (int q = 0; q < G; ++q) {
        const float2 t = piece[(q << head_shift) + h];
        pair_merge(M, L, t.x, t.y);
      }
    }
    __syncthreads();                                        // `total` free again
    if (g == 0) total[h] = make_float2(M, __builtin_amdgcn_rcpf(L));
    __syncthreads();
    // the row's elements inside this tile
    const int64_t lo = max(s, t0), hi = min(e, t1);
    const int64_t n = (hi - lo) * heads;
    for (int64_t base = 0; base < n; base += 4 * kFixBlock) {
      int64_t o[4];
      float xv[4];
      float2 t[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t i = base + u * kFixBlock + threadIdx.x;
        o[u] = -1;
        xv[u] = 0.0f;
        t[u] = make_float2(0.0f, 0.0f);
        if (i < n) {
          const int64_t slot = lo + i / heads;
          const int hd = (int)(i % heads);
          const int64_t ed = eid ? (int64_t)eid[slot] : slot;
          o[u] = ed * heads + hd;
          xv[u] = x[o[u]];
          t[u] = total[hd];
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (o[u] >= 0) y[o[u]] = exp_fast(xv[u] - t[u].x) * t[u].y;
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
    // two partial (max, sum) pairs per lane of a slot for every tile
    const int shift = ga::lanes_per_slot_shift(heads);
    const int64_t tile_slots = (int64_t)ga::kTileWaves * (ga::kChunkElems >> shift);
    const int64_t tiles = (n_edges + tile_slots - 1) / tile_slots;
    return (size_t)tiles * 2 * ((size_t)1 << shift) * 2 * sizeof(float);
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
  if (x != y) {     // y may be x itself; any other overlap would read results as logits
    const uintptr_t xa = reinterpret_cast<uintptr_t>(x), ya = reinterpret_cast<uintptr_t>(y);
    const uintptr_t bytes = (uintptr_t)n_edges * (uintptr_t)heads * sizeof(float);
    if (xa < ya + bytes && ya < xa + bytes) return GA_EINVAL;
  }
  const size_t need = ga_softmax_workspace_bytes(n_edges, heads);
  if (need && (!workspace || workspace_bytes < need || !aligned(workspace, 16)))
    return GA_EWORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  float *stats = (float *)workspace;

  if (chunked_heads(heads)) {
    const int head_shift = lanes_per_slot_shift(heads);
    const bool every_lane_live = heads == ((int64_t)1 << head_shift);
    const int tile_shift = ilog2_floor((uint64_t)kTileWaves) + ilog2_floor((uint64_t)kChunkElems) - head_shift;
    const int64_t tiles = (n_edges + ((int64_t)1 << tile_shift) - 1) >> tile_shift;
    if (tiles > 0x7fffffff) return GA_EUNSUPPORTED;
    if (every_lane_live && !eid && aligned(x, 16) && aligned(y, 16))
      hipLaunchKernelGGL((softmax_tiles_kernel<true, kTileWaves>), dim3((unsigned)tiles),
                         dim3(kTileWaves * kWave), 0, s, pointer, row_of_slot, eid, x, y, stats,
                         n_edges, head_shift, (int)heads);
    else
      hipLaunchKernelGGL((softmax_tiles_kernel<false, kTileWaves>), dim3((unsigned)tiles),
                         dim3(kTileWaves * kWave), 0, s, pointer, row_of_slot, eid, x, y, stats,
                         n_edges, head_shift, (int)heads);
    if (tiles > 1)
      hipLaunchKernelGGL(softmax_tile_rows_kernel, dim3((unsigned)tiles), dim3(kFixBlock), 0, s,
                         pointer, row_of_slot, eid, x, y, stats, n_edges, head_shift, (int)heads,
                         tile_shift);
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
