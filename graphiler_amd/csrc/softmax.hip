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
constexpr int kTilePad = kChunkElems;                      // LDS words per wavefront
constexpr int kQuads = kChunkElems / (kWave * 4);          // 16-byte pieces per lane
// logits of a chunk that span more than this use per-row maxima as the reference
// point of their exponentials; a narrower chunk uses its own maximum for all rows
constexpr float kFlatMinExp = 8.7565108e-27f;   // e^-60

// How a chunk's logits reach the lanes:
//   kDirect  edge ids are slot numbers: the chunk is one contiguous piece of x / y,
//            moved with coalesced 16-byte accesses and re-distributed to the owning
//            lanes through the padded, wave-private LDS tile;
//   kGather4 edge ids differ, at least 4 heads: a 16-byte piece lies inside one
//            edge's row, so the same scheme with one edge-id lookup per piece;
//   kElement every element is gathered through eid by the lane that owns it (fewer
//            than 4 heads with edge ids, or a head count that is not a power of two).
constexpr int kDirect = 0, kGather4 = 1, kElement = 2;

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
  int first_end;        // slots of the chunk before the end of row_first
  int last_start;       // first slot of row_last inside the chunk (0 when it began before)
  bool began_before, continues, has_b;
};

// What pass 2 needs to know about a row that leaves a tile: [tile][A|B] -> (valid,
// first slot, end slot) of the row, 16 bytes each, after the statistics.
__device__ __forceinline__ int4 *desc_ptr(float *stats, int64_t n_tiles, int H) {
  return reinterpret_cast<int4 *>(stats + n_tiles * 4 * H);
}

// Per-lane state that lives from the reduction (before the workgroup barrier) to
// the store (after it).
template <int MODE>
struct LaneRows {
  float c[kT];          // 0: slot j starts a row, 1: it continues the row of slot j-1 (c[0] unused)
  float p[kT];          // exp(logit - reference point of its segment in this chunk)
  int64_t off[MODE == kElement ? kT : 1];   // kElement: element offsets
  int eq[MODE == kGather4 ? kQuads : 1];    // kGather4: edge id of each 16-byte piece
  int kf, kl;           // row of the lane's first / last slot
  float mf, ml;         // reference point of the lane's first / last segment
  float vf;             // sum of p over the lane's part of its first segment
  float tf, tl;         // chunk-wide sum of p over the lane's first / last segment
};

// Largest total a segment is given: a row whose other chunks outweigh this one by
// more than fp32 can express has its elements here rounded to 0.
constexpr float kHugeTotal = 1.0e38f;

// m[j] <- maximum of v over the chunk-wide segment that holds the lane's slot j
// (the chunks whose logits are far apart; c as in LaneRows).
__device__ __forceinline__ void segment_max(float (&m)[kT], const float (&c)[kT], int kf, int kl,
                                            int lane, int H) {
#pragma unroll
  for (int j = 1; j < kT; ++j) m[j] = c[j] == 0.0f ? m[j] : fmaxf(m[j - 1], m[j]);
#pragma unroll
  for (int j = kT - 2; j >= 0; --j) m[j] = c[j + 1] == 0.0f ? m[j] : m[j + 1];
  float tf, tl;
  chunk_totals<true>(m[0], m[kT - 1], kf, kl, lane, H, tf, tl);
  float lead = 1.0f;                // slot j lies in the lane's first segment
#pragma unroll
  for (int j = 0; j < kT; ++j) {
    if (j > 0) lead *= c[j];
    m[j] = lead != 0.0f ? tf : m[j];
  }
  float trail = kf == kl ? 0.0f : 1.0f;   // slot j lies in the lane's last segment (and not its first)
#pragma unroll
  for (int j = kT - 1; j >= 0; --j) {
    m[j] = trail != 0.0f ? tl : m[j];
    trail *= c[j];
  }
}

// exp(x) for x in [-60, 0] (and 0 for -inf): exp2 of the rounded product.  The
// product's rounding (|x| log2 e 2^-24 in the exponent) costs at most 3.6e-6 of the
// result at x = -60 and 3e-7 at x = -5, where exp_fast's correction term would cost
// five more instructions per element.
__device__ __forceinline__ float exp_small(float x) {
  return __builtin_amdgcn_exp2f(x * 1.44269502162933349609375f);
}

// The wave-private tile: lane o owns words [16 o, 16 o + 16), its 16 slots in order,
// as four 16-byte units stored at unit position u ^ ((o >> 1) & 3).  A lane moves its
// 16 values with four 16-byte accesses; with the units permuted this way the eight
// lanes an access serves at a time fall on different banks (lanes two apart share
// their banks, and get different units).
__device__ __forceinline__ int unit_word(int o, int u) {
  return (o << 4) + (((u ^ (o >> 1)) & 3) << 2);
}
__device__ __forceinline__ int own_word(int o, int j) { return unit_word(o, j >> 2) + (j & 3); }

__device__ __forceinline__ void own_read(const float *tile, int lane, float (&v)[kT]) {
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const float4 t = *reinterpret_cast<const float4 *>(tile + unit_word(lane, u));
    v[4 * u] = t.x; v[4 * u + 1] = t.y; v[4 * u + 2] = t.z; v[4 * u + 3] = t.w;
  }
}
__device__ __forceinline__ void own_write(float *tile, int lane, const float (&v)[kT]) {
#pragma unroll
  for (int u = 0; u < 4; ++u)
    *reinterpret_cast<float4 *>(tile + unit_word(lane, u)) =
        make_float4(v[4 * u], v[4 * u + 1], v[4 * u + 2], v[4 * u + 3]);
}

// The 16-byte piece Q of the chunk (elements 4 Q .. 4 Q + 3, element = slot * H + head)
// goes to / comes from the lanes that own its elements (slot / 16, head): one unit of
// one lane for one head, two halves of a unit for two heads, one word each of four
// lanes above.  PieceMap holds the tile words of a lane's piece i = 0 (Q = lane); up
// to 16 heads piece i (Q = 64 i + lane) lies 256 i words further on (16 owner lanes
// per 256 elements, same unit permutation), so the moves below use constant offsets.
template <int HS>
struct PieceMap {
  static constexpr int kWords = HS == 0 ? 1 : (HS == 1 ? 2 : 4);
  int w[kWords];
  int lane;
  __device__ __forceinline__ void locate(int Q, int (&out)[kWords]) const {
    if (HS == 0) {
      out[0] = unit_word(Q >> 2, Q & 3);
    } else if (HS == 1) {
      const int o = (Q >> 3) << 1, j = (Q << 1) & 15;
      out[0] = own_word(o, j);
      out[1] = own_word(o + 1, j);
    } else {
      const int slot = Q >> (HS - 2), j = slot & 15;
      const int o = ((slot >> 4) << HS) + ((Q << 2) & ((1 << HS) - 1));
#pragma unroll
      for (int c = 0; c < 4; ++c) out[c] = own_word(o + c, j);
    }
  }
  __device__ __forceinline__ explicit PieceMap(int lane_) : lane(lane_) { locate(lane_, w); }
  __device__ __forceinline__ void words(int i, int (&out)[kWords]) const {
    if (HS <= 4) {
#pragma unroll
      for (int c = 0; c < kWords; ++c) out[c] = w[c] + 256 * i;
    } else {
      locate(i * kWave + lane, out);
    }
  }
  __device__ __forceinline__ void write(float *tile, int i, const float4 &x) const {
    int a[kWords];
    words(i, a);
    if (HS == 0) {
      *reinterpret_cast<float4 *>(tile + a[0]) = x;
    } else if (HS == 1) {
      *reinterpret_cast<float2 *>(tile + a[0]) = make_float2(x.x, x.z);
      *reinterpret_cast<float2 *>(tile + a[1]) = make_float2(x.y, x.w);
    } else {
      tile[a[0]] = x.x; tile[a[1]] = x.y; tile[a[2]] = x.z; tile[a[3]] = x.w;
    }
  }
  __device__ __forceinline__ float4 read(const float *tile, int i) const {
    int a[kWords];
    words(i, a);
    if (HS == 0) return *reinterpret_cast<const float4 *>(tile + a[0]);
    if (HS == 1) {
      const float2 p = *reinterpret_cast<const float2 *>(tile + a[0]);
      const float2 q = *reinterpret_cast<const float2 *>(tile + a[1]);
      return make_float4(p.x, q.x, p.y, q.y);
    }
    return make_float4(tile[a[0]], tile[a[1]], tile[a[2]], tile[a[3]]);
  }
};

// Maximum / minimum over the wavefront, in every lane: four steps inside the rows of
// 16 lanes with DPP moves, two across the rows.
template <bool IS_MAX>
__device__ __forceinline__ float wave_extreme(float v) {
  auto op = [](float a, float b) { return IS_MAX ? fmaxf(a, b) : fminf(a, b); };
  v = op(v, __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xF, 0xF, true)));   // quad_perm [1,0,3,2]
  v = op(v, __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xF, 0xF, true)));   // quad_perm [2,3,0,1]
  v = op(v, __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x141, 0xF, 0xF, true)));  // row_half_mirror
  v = op(v, __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x140, 0xF, 0xF, true)));  // row_mirror
  v = op(v, __shfl_xor(v, 16));
  v = op(v, __shfl_xor(v, 32));
  return v;
}

// The chunk's logits as the lanes load them (kDirect / kGather4: 16-byte pieces, lane
// after lane).  Issued before anything else the wavefront does: they depend on the
// chunk's position only.
template <int HS, int MODE, bool FULL>
__device__ __forceinline__ void chunk_load(const int32_t *__restrict__ eid,
                                           const float *__restrict__ x, int64_t c0, int64_t c1,
                                           float4 (&xv)[kQuads], LaneRows<MODE> &S) {
  constexpr int H = 1 << HS;
  const int lane = threadIdx.x & (kWave - 1);
  const int n_elem = (int)(c1 - c0) << HS;
  if (MODE == kDirect) {
    const float *xc = x + (c0 << HS);
#pragma unroll
    for (int i = 0; i < kQuads; ++i) {
      const int q = (i * kWave + lane) * 4;
      xv[i] = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
      if (FULL || q + 3 < n_elem) {
        xv[i] = *reinterpret_cast<const float4 *>(xc + q);
      } else if (q < n_elem) {
        xv[i].x = xc[q];
        if (q + 1 < n_elem) xv[i].y = xc[q + 1];
        if (q + 2 < n_elem) xv[i].z = xc[q + 2];
      }
    }
  } else if (MODE == kGather4) {
#pragma unroll
    for (int i = 0; i < kQuads; ++i) {
      const int q = (i * kWave + lane) * 4;
      S.eq[i] = (FULL || q < n_elem) ? eid[c0 + (q >> HS)] : -1;
    }
#pragma unroll
    for (int i = 0; i < kQuads; ++i) {
      const int q = (i * kWave + lane) * 4;
      xv[i] = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
      if (FULL || S.eq[i] >= 0)
        xv[i] = *reinterpret_cast<const float4 *>(x + ((int64_t)S.eq[i] << HS) + (q & (H - 1)));
    }
  }
}

// Reduction of one chunk.  FULL: the chunk holds all 1024 elements and every lane
// is live, so no element needs a validity test.
// Rows of the lane's 16 slots without reading the slot -> row column: the row that
// holds the chunk's first slot and the one that holds its last come from that
// column (two reads per chunk), the row starts in between from the row pointer --
// each row that starts inside the chunk marks its first slot in the wave-private
// LDS tile, a lane reads its 16 marks, and what lies before a lane's first mark is
// the largest mark of the lanes before it (rows ascend with the slot), found with a
// scan over the lanes.
template <int HS, int MODE, bool FULL>
__device__ __forceinline__ void chunk_reduce(
    const int32_t *__restrict__ pointer, const int32_t *__restrict__ eid,
    const float *__restrict__ x, const ChunkRows &cr, int heads, float *tile,
    const float4 (&xv)[kQuads], LaneRows<MODE> &S) {
  constexpr int H = 1 << HS;                  // lanes per slot; heads <= H of them are live
  constexpr int chunk_slots = kChunkElems >> HS;
  const int lane = threadIdx.x & (kWave - 1);
  const int g = lane >> HS, h = lane & (H - 1);
  const int64_t s0 = cr.c0 + (int64_t)g * kT;   // first slot of this lane
  float v[kT];
  if (MODE == kElement) {
#pragma unroll
    for (int j = 0; j < kT; ++j) {
      const int64_t slot = s0 + j;
      const bool valid = FULL || (slot < cr.c1 && h < heads);
      const int64_t e = (valid && eid) ? (int64_t)eid[slot] : slot;
      S.off[j] = e * heads + h;
      v[j] = valid ? x[S.off[j]] : -INFINITY;
    }
  }
  // ---- row starts ------------------------------------------------------------------
  // marks: one word per slot, laid out like the values of a one-head chunk (slot group
  // sg = slot / 16 in place of the lane)
  int *marks = reinterpret_cast<int *>(tile);
#pragma unroll
  for (int i = 0; i < chunk_slots / (kWave * 4); ++i)
    *reinterpret_cast<int4 *>(marks + (i * kWave + lane) * 4) = make_int4(-1, -1, -1, -1);
  if (chunk_slots < kWave * 4 && lane * 4 < chunk_slots)
    *reinterpret_cast<int4 *>(marks + lane * 4) = make_int4(-1, -1, -1, -1);
  __builtin_amdgcn_wave_barrier();
  for (int r = cr.row_first + 1 + lane; r <= cr.row_last; r += kWave) {
    const int s = pointer[r], e = pointer[r + 1];
    if (e > s) {                                  // rows without edges own no slot
      const int q = (int)(s - cr.c0);
      marks[own_word(q >> 4, q & 15)] = r;
    }
  }
  __builtin_amdgcn_wave_barrier();
  int last = -1, mark0;
  {
    float mkf[kT];
    own_read(tile, g, mkf);
#pragma unroll
    for (int j = 0; j < kT; ++j) {
      const int mk = __float_as_int(mkf[j]);
      if (j == 0) mark0 = mk;
      S.c[j] = mk >= 0 ? 0.0f : 1.0f;
      last = max(last, mk);
    }
  }
  __builtin_amdgcn_wave_barrier();
  int inc = last;                                 // largest mark of lanes <= me (same head)
#pragma unroll
  for (int off = H; off < kWave; off <<= 1) {
    const int t = __shfl_up(inc, off);
    if (lane >= off) inc = max(inc, t);
  }
  int before = __shfl_up(inc, H);
  before = lane >= H ? max(before, cr.row_first) : cr.row_first;
  S.kf = mark0 >= 0 ? mark0 : before;
  S.kl = max(last, before);
  // ---- logits to the lanes that own them -----------------------------------------
  if (MODE != kElement) {
    const PieceMap<HS> pm(lane);
#pragma unroll
    for (int i = 0; i < kQuads; ++i) pm.write(tile, i, xv[i]);
    __builtin_amdgcn_wave_barrier();
    own_read(tile, lane, v);
    __builtin_amdgcn_wave_barrier();
  }
  // ---- reference points: the chunk's maximum when its logits are close together,
  //      per-row maxima otherwise ---------------------------------------------------
  float mx = v[0];
#pragma unroll
  for (int j = 1; j < kT; ++j) mx = fmaxf(mx, v[j]);
  mx = wave_extreme<true>(mx);
  // exponentials from the chunk's maximum; the smallest one tells whether that was close
  // enough for every element (elements past the end hold -inf and give 0: left out)
  float pmin = 1.0f;
#pragma unroll
  for (int j = 0; j < kT; ++j) {
    S.p[j] = exp_small(v[j] - mx);
    if (FULL || (s0 + j < cr.c1 && h < heads)) pmin = fminf(pmin, S.p[j]);
  }
  pmin = wave_extreme<false>(pmin);
  // no exponential below e^-60 (none 0, none NaN or inf): every element keeps its precision
  const bool flat = pmin >= kFlatMinExp;
  if (flat) {
    S.mf = S.ml = mx;
  } else {
    // (the logits are still in the tile: read again rather than kept in registers)
    if (MODE != kElement) own_read(tile, lane, v);
    float m[kT];
#pragma unroll
    for (int j = 0; j < kT; ++j) m[j] = v[j];
    segment_max(m, S.c, S.kf, S.kl, lane, H);
    S.mf = m[0];
    S.ml = m[kT - 1];
#pragma unroll
    for (int j = 0; j < kT; ++j) S.p[j] = exp_fast(v[j] - finite_or_zero(m[j]));
  }
  if (!FULL) {
#pragma unroll
    for (int j = 0; j < kT; ++j)
      if (!(s0 + j < cr.c1 && h < heads)) S.p[j] = 0.0f;
  }
  // ---- sums of exponentials: the lane's part of its first and of its last segment,
  //      then what the other lanes of the chunk add to them ------------------------
  float run = S.p[0], vf = S.p[0], lead = 1.0f;
#pragma unroll
  for (int j = 1; j < kT; ++j) {
    run = fmaf(S.c[j], run, S.p[j]);
    lead *= S.c[j];
    vf = fmaf(lead, S.p[j], vf);
  }
  S.vf = vf;
  chunk_totals<false>(vf, run, S.kf, S.kl, lane, H, S.tf, S.tl);
}

// After the workgroup barrier: the (reference point, sum) pairs of the rows a chunk
// shares with other chunks of the tile are in LDS (pair_a / pair_b per wavefront,
// with each wavefront's flags).  Rows that end up complete are normalised and
// stored; rows that leave the tile leave their pair for the tile in `stats`, and
// their elements are not written here (so y may be x): pass 2 writes them.
template <int HS, int MODE, bool FULL, int W>
__device__ __forceinline__ void chunk_store(
    const int32_t *__restrict__ eid, const ChunkRows &cr, float *__restrict__ y,
    float *__restrict__ stats, int heads, int wave, const int *wflags, const float2 *pair_a,
    const float2 *pair_b, float *tile, const LaneRows<MODE> &S) {
  constexpr int H = 1 << HS;
  constexpr int chunk_slots = kChunkElems >> HS;
  const int lane = threadIdx.x & (kWave - 1);
  const int g = lane >> HS, h = lane & (H - 1);
  const int64_t tile_id = blockIdx.x;
  // pairs are stored [wavefront][head] with room for 64 heads per wavefront
  auto pa = [&](int w) { return pair_a[w * kWave + h]; };
  auto pb = [&](int w) { return pair_b[w * kWave + h]; };
  float total_a = 0.0f, total_b = 0.0f;
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
    total_a = L * exp_fast(M - S.mf);      // the row's sum seen from this lane's reference point
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
    total_b = L * exp_fast(M - S.ml);
  }
  // slots [keep_lo, keep_hi) of the chunk are finished here
  const int keep_lo = open_a ? cr.first_end : 0;
  const int keep_hi = open_b ? cr.last_start : chunk_slots;
  const bool lane_a = cr.began_before && S.kf == cr.row_first;
  const bool lane_b = cr.has_b && S.kl == cr.row_last;
  // totals of the lane's first and last segment; a lane inside one segment has one
  float t_lead = lane_a ? total_a : S.tf;
  float t_trail = lane_b ? total_b : S.tl;
  const bool one_segment = S.kf == S.kl;
  if (one_segment && lane_b) t_lead = t_trail;
  // Every slot's segment total: running sums forwards, started so that the first
  // segment ends at its total, then the totals copied backwards from the segment
  // ends (running sums of non-negative terms never exceed their total).
  float seed = t_lead - S.vf;
  seed = seed < kHugeTotal ? seed : kHugeTotal;     // also for NaN
  t_trail = t_trail < kHugeTotal ? t_trail : kHugeTotal;
  float l[kT];
  l[0] = S.p[0] + seed;
#pragma unroll
  for (int j = 1; j < kT; ++j) l[j] = fmaf(S.c[j], l[j - 1], S.p[j]);
  l[kT - 1] = one_segment ? l[kT - 1] : t_trail;
#pragma unroll
  for (int j = kT - 2; j >= 0; --j) l[j] = fmaxf(l[j], S.c[j + 1] * l[j + 1]);
  float o[kT];
#pragma unroll
  for (int j = 0; j < kT; ++j) o[j] = S.p[j] * __builtin_amdgcn_rcpf(l[j]);
  if (MODE != kElement) {
    const int n_elem = (int)((cr.c1 - cr.c0) << HS);
    own_write(tile, lane, o);
    __builtin_amdgcn_wave_barrier();
    const PieceMap<HS> pm(lane);
    float *yc = y + (cr.c0 << HS);
    const bool all_kept = keep_lo == 0 && keep_hi == chunk_slots;    // whole wavefront
#pragma unroll
    for (int i = 0; i < kQuads; ++i) {
      const int q = (i * kWave + lane) * 4;
      const float4 e4 = pm.read(tile, i);
      const float e[4] = {e4.x, e4.y, e4.z, e4.w};
      float *dst = MODE == kDirect ? yc + q : y + ((int64_t)S.eq[i] << HS) + (q & (H - 1));
      if (MODE == kGather4 && !FULL && S.eq[i] < 0) continue;
      const int s_lo = q >> HS, s_hi = (q + 3) >> HS;
      if ((FULL || q + 3 < n_elem) && (all_kept || (s_lo >= keep_lo && s_hi < keep_hi))) {
        *reinterpret_cast<float4 *>(dst) = make_float4(e[0], e[1], e[2], e[3]);
      } else {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const int sl = (q + c) >> HS;
          if (q + c < n_elem && sl >= keep_lo && sl < keep_hi) dst[c] = e[c];
        }
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < kT; ++j) {
      const int sl = g * kT + j;
      if ((FULL || (sl < (int)(cr.c1 - cr.c0) && h < heads)) && sl >= keep_lo && sl < keep_hi)
        y[S.off[j]] = o[j];
    }
  }
}

template <int HS, int MODE, int W>
__global__ __launch_bounds__(W *kWave) void softmax_tiles_kernel(
    const int32_t *__restrict__ pointer, const int32_t *__restrict__ row_of_slot,
    const int32_t *__restrict__ eid, const float *__restrict__ x, float *__restrict__ y,
    float *__restrict__ stats, int64_t n_edges, int heads, int64_t n_tiles) {
  // per wavefront: one tile of 1024 words, used in turn for
  // the row marks, the logits and the results
  extern __shared__ float lds_dyn[];          // tiles_lds_bytes(W)
  float(*lds_tile)[kTilePad] = reinterpret_cast<float(*)[kTilePad]>(lds_dyn);
  float2 *pair_a = reinterpret_cast<float2 *>(lds_dyn + W * kTilePad);
  float2 *pair_b = pair_a + W * kWave;
  int *wflags = reinterpret_cast<int *>(pair_b + W * kWave);
  constexpr int H = 1 << HS;
  constexpr int chunk_slots = kChunkElems >> HS;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);   // uniform: scalar row lookups
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t chunk_id = (int64_t)blockIdx.x * W + wave;
  ChunkRows cr;
  cr.c0 = chunk_id * chunk_slots;
  const bool active = cr.c0 < n_edges;                                // whole wavefront
  cr.c1 = min(cr.c0 + (int64_t)chunk_slots, n_edges);
  // the variant without validity tests needs every lane live: a whole chunk and as
  // many heads as lanes per slot
  const bool full = active && cr.c1 - cr.c0 == chunk_slots && heads == H;
  LaneRows<MODE> S;
  float4 xv[kQuads];
  if (active) {
    if (full)
      chunk_load<HS, MODE, true>(eid, x, cr.c0, cr.c1, xv, S);
    else
      chunk_load<HS, MODE, false>(eid, x, cr.c0, cr.c1, xv, S);
  }
  int flags = 0;
  int4 desc_a = make_int4(0, 0, 0, 0), desc_b = make_int4(0, 0, 0, 0);
  if (active) {
    cr.row_first = row_of_slot[cr.c0];
    cr.row_last = row_of_slot[cr.c1 - 1];
    const int64_t fs = pointer[cr.row_first], fe = pointer[cr.row_first + 1];
    const int64_t ls = pointer[cr.row_last], le = pointer[cr.row_last + 1];
    cr.began_before = fs < cr.c0;
    cr.continues = le > cr.c1;
    cr.has_b = cr.continues && !(cr.began_before && cr.row_first == cr.row_last);
    cr.first_end = (int)(min(fe, cr.c1) - cr.c0);
    cr.last_start = (int)(max(ls, cr.c0) - cr.c0);
    desc_a = make_int4(cr.began_before ? 1 : 0, (int)fs, (int)fe, 0);
    desc_b = make_int4(cr.has_b ? 1 : 0, (int)ls, (int)le, 0);
    if (full)
      chunk_reduce<HS, MODE, true>(pointer, eid, x, cr, heads, lds_tile[wave], xv, S);
    else
      chunk_reduce<HS, MODE, false>(pointer, eid, x, cr, heads, lds_tile[wave], xv, S);
    flags = kActive | (cr.began_before ? kBegan : 0) | (cr.continues ? kContinues : 0) |
            (cr.row_first == cr.row_last ? kSingle : 0);
    const int g = lane >> HS, h = lane & (H - 1);
    if (cr.began_before && g == 0)            // lanes 0..H-1 start with row_first
      pair_a[wave * kWave + h] = make_float2(S.mf, S.tf);
    if (cr.has_b && g == (kWave >> HS) - 1)   // a continuing chunk is full
      pair_b[wave * kWave + h] = make_float2(S.ml, S.tl);
  }
  if (lane == 0) {
    wflags[wave] = flags;
    // a row leaves the tile at its start when the tile's first chunk begins inside
    // it, at its end when the last chunk ends inside a row that began in the tile or
    // at its start (a row over the whole tile counts once, as A)
    int4 *desc = desc_ptr(stats, n_tiles, H);
    if (wave == 0) desc[(int64_t)blockIdx.x * 2] = desc_a;
  }
  __syncthreads();
  if (lane == 0 && wave == W - 1) {
    // B of the tile: the row that is open at the tile's end, unless it is the tile's A row
    int j = W - 1;
    while (j > 0 && passes_through(wflags[j])) --j;
    const bool through = passes_through(wflags[j]) && j == 0;     // one row over the whole tile
    int4 d = make_int4(0, 0, 0, 0);
    if (active && cr.continues && !through) d = make_int4(1, desc_b.y, desc_b.z, 0);
    desc_ptr(stats, n_tiles, H)[(int64_t)blockIdx.x * 2 + 1] = d;
  }
  if (!active) return;
  if (full)
    chunk_store<HS, MODE, true, W>(eid, cr, y, stats, heads, wave, wflags, pair_a, pair_b,
                                   lds_tile[wave], S);
  else
    chunk_store<HS, MODE, false, W>(eid, cr, y, stats, heads, wave, wflags, pair_a, pair_b,
                                    lds_tile[wave], S);
}

// ---- pass 2: rows that leave a tile -------------------------------------------
// Wavefront 2 t + w handles row A (w = 0: the tile's first row, begun in an earlier
// tile) or B (w = 1: its last row, started here and continuing) of tile t, when the
// tile has one (its descriptor says so).  The row's pair is folded from the tiles'
// partials (B of the row's first tile, then A of the following ones, in tile order:
// every tile of a row folds the same chain and gets the same pair), and the row's
// elements inside this tile are normalised with it.  Chains of up to kShortChain
// tiles are folded by every lane of a head for itself; longer ones are cut into a
// piece per lane group, folded in parallel and combined in order.  The kFixWaves
// wavefronts of a workgroup fold the pair each for itself (no workgroup barrier) and
// share the row's elements: a row over a whole tile is two batches per lane.
constexpr int kShortChain = 8;
constexpr int kFixSplit = 1;      // workgroups that share a row's elements inside one tile (1: the waves of one workgroup do)
constexpr int kFixQuads = 4;      // 16-byte pieces in flight per lane
constexpr int kFixWaves = 4;
constexpr int kFixBlock = kFixWaves * kWave;

template <int MODE>
__global__ __launch_bounds__(kFixBlock) void softmax_tile_rows_kernel(
    const int32_t *__restrict__ eid, const float *__restrict__ x, float *__restrict__ y,
    float *__restrict__ stats, int64_t n_edges, int head_shift, int heads, int tile_shift,
    int64_t n_tiles) {
  __shared__ float2 piece_w[kFixWaves][kWave];
  __shared__ float2 total_w[kFixWaves][kWave];
  const int H = 1 << head_shift;
  const int4 d = desc_ptr(stats, n_tiles, H)[blockIdx.x];
  if (!d.x) return;                                         // whole workgroup
  const int lane = threadIdx.x & (kWave - 1);
  float2 *piece = piece_w[threadIdx.x / kWave], *total = total_w[threadIdx.x / kWave];
  const int64_t tile_id = blockIdx.x >> 1;
  const int64_t t0 = tile_id << tile_shift;
  const int64_t t1 = min(t0 + ((int64_t)1 << tile_shift), n_edges);
  const int64_t s = d.y, e = d.z;
  const int64_t lo = max(s, t0), hi = min(e, t1);
  // ---- the first batch of logits does not wait for the row's pair -------------------
  // kDirect: the row's elements [lo * H, hi * H) are contiguous; 16-byte pieces from the
  //   aligned address below the first one, lane after lane.
  // kGather4: H / 4 pieces per slot, each slot's row found through eid.
  // kElement: single elements, row through eid when given.
  const int64_t first = MODE == kDirect ? ((lo << head_shift) & ~(int64_t)3) : 0;
  const int64_t n = MODE == kDirect ? (hi << head_shift) - first
                                    : (MODE == kGather4 ? (hi - lo) << head_shift : (hi - lo) * heads);
  const int64_t skip = MODE == kDirect ? (lo << head_shift) - first : 0;   // elements before the row
  float4 xq[kFixQuads];
  int64_t oq[kFixQuads];
  auto fetch = [&](int64_t base) {      // base: element index of the batch's first piece
#pragma unroll
    for (int u = 0; u < kFixQuads; ++u) {
      const int64_t i = base + ((int64_t)u * kFixBlock + threadIdx.x) * (MODE == kElement ? 1 : 4);
      oq[u] = -1;
      xq[u] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      if (i >= n) continue;
      if (MODE == kDirect) {
        oq[u] = first + i;
        if (i >= skip && i + 3 < n) {
          xq[u] = *reinterpret_cast<const float4 *>(x + oq[u]);
        } else {
          if (i >= skip) xq[u].x = x[oq[u]];
          if (i + 1 >= skip && i + 1 < n) xq[u].y = x[oq[u] + 1];
          if (i + 2 >= skip && i + 2 < n) xq[u].z = x[oq[u] + 2];
          if (i + 3 >= skip && i + 3 < n) xq[u].w = x[oq[u] + 3];
        }
      } else if (MODE == kGather4) {
        const int64_t ed = eid[lo + (i >> head_shift)];
        oq[u] = (ed << head_shift) + (i & (H - 1));
        xq[u] = *reinterpret_cast<const float4 *>(x + oq[u]);
      } else {
        const int64_t slot = lo + i / heads;
        const int64_t ed = eid ? (int64_t)eid[slot] : slot;
        oq[u] = ed * heads + i % heads;
        xq[u].x = x[oq[u]];
        xq[u].y = __int_as_float((int)(i % heads));
      }
    }
  };
  const int64_t batch = (int64_t)kFixQuads * kFixBlock * (MODE == kElement ? 1 : 4);   // elements per step
  if ((int64_t)blockIdx.y * batch >= n) return;             // whole workgroup: nothing of the row left for it
  fetch((int64_t)blockIdx.y * batch);
  // ---- the row's pair ------------------------------------------------------------------
  const int G = kWave >> head_shift;
  const int g = lane >> head_shift, h = lane & (H - 1);
  const int64_t k_lo = s >> tile_shift, k_hi = (e - 1) >> tile_shift;
  const int64_t len = k_hi - k_lo + 1;                      // states: B of k_lo, A of k_lo+1 .. k_hi
  const float *a_of = stats + (size_t)h * 2;                // A pair of tile k: a_of[k * 4H]
  const size_t step = (size_t)4 * H;
  float M, L;
  if (len <= kShortChain) {
    float2 t[kShortChain];
#pragma unroll
    for (int u = 0; u < kShortChain; ++u)
      if (u < len)
        t[u] = *reinterpret_cast<const float2 *>(a_of + (k_lo + u) * step + (u == 0 ? 2 * H : 0));
    M = t[0].x;
    L = t[0].y;
#pragma unroll
    for (int u = 1; u < kShortChain; ++u)
      if (u < len) pair_merge(M, L, t[u].x, t[u].y);
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
    piece[lane] = make_float2(M, L);
    __builtin_amdgcn_wave_barrier();
    M = -INFINITY;
    L = 0.0f;
    for (int q = 0; q < G; ++q) {
      const float2 t = piece[(q << head_shift) + h];
      pair_merge(M, L, t.x, t.y);
    }
  }
  if (g == 0) total[h] = make_float2(M, __builtin_amdgcn_rcpf(L));
  __builtin_amdgcn_wave_barrier();
  // a lane's pieces always hold the same heads: 512 elements per step, a multiple of H
  float2 th[4];
  if (MODE != kElement) {
    const int h0 = MODE == kDirect ? (int)((first + 4 * threadIdx.x) & (H - 1)) : (4 * threadIdx.x) & (H - 1);
#pragma unroll
    for (int c = 0; c < 4; ++c) th[c] = total[(h0 + c) & (H - 1)];
  }
  for (int64_t base = (int64_t)blockIdx.y * batch; base < n; base += kFixSplit * batch) {
    if (base >= kFixSplit * batch) fetch(base);
#pragma unroll
    for (int u = 0; u < kFixQuads; ++u) {
      if (oq[u] < 0) continue;
      if (MODE == kElement) {
        const float2 t = total[__float_as_int(xq[u].y)];
        y[oq[u]] = exp_fast(xq[u].x - t.x) * t.y;
        continue;
      }
      const float4 o = make_float4(exp_fast(xq[u].x - th[0].x) * th[0].y,
                                   exp_fast(xq[u].y - th[1].x) * th[1].y,
                                   exp_fast(xq[u].z - th[2].x) * th[2].y,
                                   exp_fast(xq[u].w - th[3].x) * th[3].y);
      const int64_t i = oq[u] - first;       // kDirect: position in the aligned range
      if (MODE == kGather4 || (i >= skip && i + 3 < n)) {
        *reinterpret_cast<float4 *>(y + oq[u]) = o;
      } else {
        if (i >= skip) y[oq[u]] = o.x;
        if (i + 1 >= skip && i + 1 < n) y[oq[u] + 1] = o.y;
        if (i + 2 >= skip && i + 2 < n) y[oq[u] + 2] = o.z;
        if (i + 3 >= skip && i + 3 < n) y[oq[u] + 3] = o.w;
      }
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
constexpr size_t tiles_lds_bytes(int W) {
  return (size_t)W * kTilePad * sizeof(float) + 2 * (size_t)W * kWave * sizeof(float2) + W * sizeof(int);
}

// Workgroups of more than 8 wavefronts need more LDS than a kernel gets by default.
template <class K>
void tiles_launch(K kernel, unsigned tiles, hipStream_t s, const int32_t *pointer,
                  const int32_t *row_of_slot, const int32_t *eid, const float *x, float *y,
                  float *stats, int64_t n_edges, int heads, int64_t n_tiles) {
  constexpr size_t lds = tiles_lds_bytes(kTileWaves);
  if (lds > 65536) {
    static bool raised = false;     // per kernel instantiation
    if (!raised) {
      (void)hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      raised = true;
    }
  }
  hipLaunchKernelGGL(kernel, dim3(tiles), dim3(kTileWaves * kWave), lds, s, pointer, row_of_slot, eid,
                     x, y, stats, n_edges, heads, n_tiles);
}

template <int HS>
void launch_tiles_hs(int mode, unsigned tiles, hipStream_t s, const int32_t *pointer,
                     const int32_t *row_of_slot, const int32_t *eid, const float *x, float *y,
                     float *stats, int64_t n_edges, int heads, int64_t n_tiles) {
  constexpr int W = kTileWaves;
  if (mode == kDirect)
    tiles_launch(softmax_tiles_kernel<HS, kDirect, W>, tiles, s, pointer, row_of_slot, eid, x, y, stats,
                 n_edges, heads, n_tiles);
  else if (mode == kGather4 && HS >= 2)
    tiles_launch(softmax_tiles_kernel<(HS >= 2 ? HS : 2), kGather4, W>, tiles, s, pointer, row_of_slot,
                 eid, x, y, stats, n_edges, heads, n_tiles);
  else
    tiles_launch(softmax_tiles_kernel<HS, kElement, W>, tiles, s, pointer, row_of_slot, eid, x, y, stats,
                 n_edges, heads, n_tiles);
}

void launch_tiles(int head_shift, int mode, unsigned tiles, hipStream_t s, const int32_t *pointer,
                  const int32_t *row_of_slot, const int32_t *eid, const float *x, float *y,
                  float *stats, int64_t n_edges, int heads, int64_t n_tiles) {
  switch (head_shift) {
#define GA_TILES_CASE(HS)                                                                       \
  case HS:                                                                                      \
    launch_tiles_hs<HS>(mode, tiles, s, pointer, row_of_slot, eid, x, y, stats, n_edges, heads, \
                        n_tiles);                                                               \
    break;
    GA_TILES_CASE(0) GA_TILES_CASE(1) GA_TILES_CASE(2) GA_TILES_CASE(3) GA_TILES_CASE(4)
    GA_TILES_CASE(5) GA_TILES_CASE(6)
#undef GA_TILES_CASE
  }
}

inline bool chunked_heads(int64_t heads) { return heads <= kWave; }
inline int lanes_per_slot_shift(int64_t heads) { return ilog2_ceil((uint64_t)heads); }

}  // namespace
}  // namespace ga

extern "C" {

size_t ga_softmax_workspace_bytes(int64_t n_edges, int64_t heads) {
  if (n_edges <= 0 || heads <= 0) return 0;
  if (ga::chunked_heads(heads)) {
    // per tile: two (reference point, sum) pairs per lane of a slot and two row descriptors
    const int shift = ga::lanes_per_slot_shift(heads);
    const int64_t tile_slots = (int64_t)ga::kTileWaves * (ga::kChunkElems >> shift);
    const int64_t tiles = (n_edges + tile_slots - 1) / tile_slots;
    return (size_t)tiles * (2 * ((size_t)1 << shift) * 2 * sizeof(float) + 2 * sizeof(int4));
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
    if (tiles > 0x3fffffff) return GA_EUNSUPPORTED;
    int mode = kElement;
    if (every_lane_live && aligned(x, 16) && aligned(y, 16)) {
      if (!eid) mode = kDirect;
      else if (head_shift >= 2) mode = kGather4;
    }
    launch_tiles(head_shift, mode, (unsigned)tiles, s, pointer, row_of_slot, eid, x, y, stats, n_edges,
                 (int)heads, tiles);
    if (tiles > 1) {
      const dim3 grid((unsigned)(2 * tiles), kFixSplit), block(kFixBlock);
      if (mode == kDirect)
        hipLaunchKernelGGL(softmax_tile_rows_kernel<kDirect>, grid, block, 0, s, eid, x, y, stats,
                           n_edges, head_shift, (int)heads, tile_shift, tiles);
      else if (mode == kGather4)
        hipLaunchKernelGGL(softmax_tile_rows_kernel<kGather4>, grid, block, 0, s, eid, x, y, stats,
                           n_edges, head_shift, (int)heads, tile_shift, tiles);
      else
        hipLaunchKernelGGL(softmax_tile_rows_kernel<kElement>, grid, block, 0, s, eid, x, y, stats,
                           n_edges, head_shift, (int)heads, tile_shift, tiles);
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
