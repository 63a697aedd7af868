// Typed neighbour sum for gfx950: the message and reduce steps of an RGCN layer
// (examples/RGCN/RGCN.py:25-33) in one pass,
//   out[v, :] = sum over the in-edges e of v of  scale[e] * (x[src(e), :] @ W[type(e)]),
// without the (E, M) message tensor that BroadcastSrcNode -> SegmentMMEdge -> mul ->
// SpMMEdge (broadcast.cu:58-63, segment_mm.cu:29-33, spmm.cu:359-373) write and read
// back: 2 M b bytes per edge against the K b bytes of the source row.
//
// The matrix cores want edges of one relation side by side, the sum wants edges of
// one destination side by side.  Both hold inside a tile of 128 (or 144) destination
// nodes whose edges are ordered by relation:
//
//   preparation (once per graph)   slots of the in-adjacency are sorted, stably, by
//     (destination / tile height, relation); every (tile, relation) group is padded to whole
//     chunks of 16 slots, and per padded slot the source node, the destination inside
//     the tile and the edge id are written out, per chunk its relation, per tile its
//     first chunk.  A pad slot has source and edge id -1.
//   kernel   one workgroup of four wavefronts per tile.  With 64 output columns a
//     wavefront owns 32 of them and walks every second chunk of the tile (two
//     wavefronts share a chunk, one per column half); with 32, 16 or 8 columns it owns
//     them all and walks every fourth chunk.  Its 128 x 32 (or narrower) fp32 partial
//     sums stay in matrix-core accumulators (64 registers), and the partial tiles meet
//     in LDS at the end.  Per chunk it gathers the 16 source rows (one 16- or 8-byte
//     read per lane and 16 input features), multiplies them with its columns of the
//     relation's weights (K / 4 v_mfma_f32_16x16x4_f32, or K / 16
//     v_mfma_f32_16x16x16_bf16) and scales the 16 x 16 result rows: the messages.  The
//     sum over destinations is a second matrix product: tile block b += S_b @ messages
//     with the 0 / 1 selection matrix S_b[i][r] = (destination of chunk row r is row
//     16 b + i), built in registers from the destination bytes, for the blocks the chunk
//     touches.  The messages enter as bf16: rounded to nearest for bf16 tensors (the
//     values the two-operator chain stores), as three truncated terms of 8 bits each for
//     fp32 (their sum is the fp32 message to 2^-24; products with 0 / 1 are exact and the
//     accumulation is fp32).  No LDS, no atomics: a run gives the same bits every time.
//     Messages that are not finite would turn the zeros of S_b into NaN for their
//     neighbours: they are replaced by zero and remembered as one bit per element and
//     kind (+inf, -inf, NaN), which the final write adds back in.
//
// Chunk ids and source rows are requested two and one of the wavefront's own chunks
// ahead of the arithmetic.
// HBM traffic per edge: 9 index bytes (+ padding), the 4-byte scale, the K b-byte
// source row (from L2 when x fits) and M b / degree output bytes.
#include "common.h"

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_scan.hpp>

namespace ga {
namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef short shortx4 __attribute__((ext_vector_type(4)));

// destination nodes per tile: 128 or 144 (8 or 9 blocks of 16), chosen per graph so that
// the workgroups fill whole rounds of the chip (ga_typed_tile_rows)
constexpr int kMaxTileRows = 144;
inline bool tile_rows_ok(int64_t r) { return r == 128 || r == 144; }
constexpr int kChunk = 16;                      // slots per chunk: rows of one MFMA
constexpr int kTypedWaves = 4;
constexpr int kTypedBlock = kTypedWaves * kWave;
inline bool typed_cols_ok(int64_t m) { return m == 8 || m == 16 || m == 32 || m == 64; }

// ------------------------------------------------------------------ preparation ----
// key of a slot: tile * n_types + relation
__global__ __launch_bounds__(kBlock) void typed_keys_kernel(
    const int32_t *__restrict__ row_of_slot, const int32_t *__restrict__ eid,
    const int32_t *__restrict__ type_pointer, int n_types, int64_t n_edges, int tile_rows,
    int32_t *__restrict__ key, int32_t *__restrict__ ids) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= n_edges) return;
  const int e = eid ? eid[i] : (int)i;
  int lo = 0, hi = n_types;                 // largest t with type_pointer[t] <= e
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (type_pointer[mid] <= e) lo = mid; else hi = mid;
  }
  key[i] = (row_of_slot[i] / tile_rows) * n_types + lo;
  ids[i] = (int32_t)i;
}

// chunks[k] = chunks group k needs, for k < n_groups; chunks[n_groups] = 0
__global__ __launch_bounds__(kBlock) void typed_group_chunks_kernel(
    const int32_t *__restrict__ key_sorted, int64_t n_groups, int64_t n_edges,
    int32_t *__restrict__ first, int32_t *__restrict__ chunks) {
  const int64_t k = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (k > n_groups) return;
  int64_t b[2];
  for (int s = 0; s < 2; ++s) {             // first sorted index with key >= k + s
    int64_t lo = 0, hi = n_edges;
    while (lo < hi) {
      const int64_t mid = (lo + hi) >> 1;
      if ((int64_t)key_sorted[mid] < k + s) lo = mid + 1; else hi = mid;
    }
    b[s] = lo;
  }
  first[k] = (int32_t)b[0];
  chunks[k] = k < n_groups ? (int32_t)((b[1] - b[0] + kChunk - 1) / kChunk) : 0;
}

__global__ __launch_bounds__(kBlock) void typed_tile_pointer_kernel(
    const int32_t *__restrict__ chunk_base, int64_t n_tiles, int n_types,
    int32_t *__restrict__ tile_chunk_pointer) {
  const int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (t <= n_tiles) tile_chunk_pointer[t] = chunk_base[t * n_types];
}

// one thread per padded slot of the capacity
__global__ __launch_bounds__(kBlock) void typed_fill_kernel(
    const int32_t *__restrict__ chunk_base, const int32_t *__restrict__ first,
    const int32_t *__restrict__ ids_sorted, const int32_t *__restrict__ row_of_slot,
    const int32_t *__restrict__ nbr, const int32_t *__restrict__ eid, int64_t n_groups,
    int n_types, int tile_rows, int64_t chunk_capacity, int32_t *__restrict__ chunk_type,
    int32_t *__restrict__ slot_src, unsigned char *__restrict__ slot_dst,
    int32_t *__restrict__ slot_edge) {
  const int64_t p = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (p >= chunk_capacity * kChunk) return;      // whole chunks: 16 neighbouring threads leave together
  const int64_t c = p / kChunk;
  int src = -1, edge = -1, dst = 0xff, type = 0;     // pad: no row of a tile
  if (c < chunk_base[n_groups]) {
    int64_t lo = 0, hi = n_groups;          // the group k with base[k] <= c < base[k + 1]
    while (hi - lo > 1) {
      const int64_t mid = (lo + hi) >> 1;
      if (chunk_base[mid] <= c) lo = mid; else hi = mid;
    }
    // groups without chunks share their base with the next one: take the last of them
    const int64_t k = lo;
    type = (int)(k % n_types);
    const int64_t off = p - (int64_t)chunk_base[k] * kChunk;
    if (off < first[k + 1] - first[k]) {
      const int i = ids_sorted[first[k] + off];
      src = nbr[i];
      edge = eid ? eid[i] : i;
      dst = row_of_slot[i] % tile_rows;
    }
  }
  slot_src[p] = src;
  slot_edge[p] = edge;
  slot_dst[p] = (unsigned char)dst;
  // the 16-row blocks of the tile that the chunk has rows in, beside its relation: the 16
  // threads of a chunk are neighbours in a wavefront
  unsigned blocks = src >= 0 ? 1u << (dst >> 4) : 0u;
#pragma unroll
  for (int off = 1; off < kChunk; off <<= 1) blocks |= __shfl_xor(blocks, off);
  if ((p & (kChunk - 1)) == 0) chunk_type[c] = type | (int)(blocks << 16);
}

inline size_t round_up(size_t v) { return (v + 255) & ~(size_t)255; }

struct TilesLayout {
  size_t key, key_sorted, ids, ids_sorted, first, chunks, base, temp, total;
  size_t sort_bytes, scan_bytes;
};

int end_bit_for(int64_t n_keys) {
  int bits = 1;
  while (bits < 31 && ((int64_t)1 << bits) < n_keys) ++bits;
  return bits;
}

int tiles_layout(int64_t n_groups, int64_t n_edges, TilesLayout &L) {
  int32_t *k = nullptr;
  L.sort_bytes = L.scan_bytes = 0;
  if (n_edges > 0) {
    hipError_t e = rocprim::radix_sort_pairs(nullptr, L.sort_bytes, k, k, k, k, (size_t)n_edges,
                                             0, end_bit_for(n_groups));
    if (e != hipSuccess) return (int)e;
  }
  hipError_t e = rocprim::exclusive_scan(nullptr, L.scan_bytes, k, k, (int32_t)0,
                                         (size_t)(n_groups + 1), rocprim::plus<int32_t>());
  if (e != hipSuccess) return (int)e;
  size_t off = 0;
  L.key = off;         off += round_up((size_t)n_edges * 4);
  L.key_sorted = off;  off += round_up((size_t)n_edges * 4);
  L.ids = off;         off += round_up((size_t)n_edges * 4);
  L.ids_sorted = off;  off += round_up((size_t)n_edges * 4);
  L.first = off;       off += round_up((size_t)(n_groups + 1) * 4);
  L.chunks = off;      off += round_up((size_t)(n_groups + 1) * 4);
  L.base = off;        off += round_up((size_t)(n_groups + 1) * 4);
  L.temp = off;        off += round_up(L.sort_bytes > L.scan_bytes ? L.sort_bytes : L.scan_bytes);
  L.total = off;
  return GA_OK;
}

inline int64_t tiles_of(int64_t n_rows, int64_t tile_rows) {
  return (n_rows + tile_rows - 1) / tile_rows;
}

// ------------------------------------------------------------------------ kernel ----
// Byte offsets into x, W and row_scale are 32-bit (checked on the host): a load is then
// "uniform base + lane offset", one or two address instructions instead of a 64-bit sum.
template <typename V>
__device__ __forceinline__ V load_at(const void *base, uint32_t byte_offset) {
  return *reinterpret_cast<const V *>(reinterpret_cast<const char *>(base) + byte_offset);
}

// How the MC output columns are shared out.  A wavefront owns kCB 16-column blocks of
// the tile (at most two: a 128 x 32 tile per wavefront is 64 accumulator registers,
// three wavefronts fit a SIMD and the whole grid is resident at once); the blocks of a
// tile make kColGroups groups of kCB, one wavefront per group works on a chunk, and the
// kTurns wavefronts of a group take turns on the chunks of the tile.  Eight columns run
// as a block of 16 whose upper half repeats the lower one and is never stored.
template <int MC>
struct Cols {
  static constexpr int kBlocks = MC >= 16 ? MC / 16 : 1;
  static constexpr int kCB = kBlocks >= 2 ? 2 : 1;
  static constexpr int kColGroups = kBlocks / kCB;
  static constexpr int kTurns = kTypedWaves / kColGroups;
  static constexpr int kMergeStride = MC + 4;   // row stride of the LDS tile the waves meet in
  // column of the weights behind lane n of block 0
  static __device__ __forceinline__ uint32_t lane_col(int n) { return MC >= 16 ? n : n % MC; }
};
template <typename T, int KS, int MC>
struct TypedFrag;

template <int KS, int MC>
struct TypedFrag<float, KS, MC> {
  static constexpr int kCB = Cols<MC>::kCB;
  float4 x[KS];           // row n of the chunk: k = 16 j + 4 q .. + 3
  float w[kCB][KS][4];    // my column block c: W[16 j + 4 q + s][16 (cb0 + c) + n]
  static __device__ __forceinline__ void load_x(TypedFrag &f, const float *x, uint32_t row, int q) {
#pragma unroll
    for (int j = 0; j < KS; ++j)
      f.x[j] = load_at<float4>(x, (row * (16u * KS) + 16u * j + 4u * q) * 4u);
  }
  // wt: the relation's weights (uniform); lane_off: element (4 q, n) of them.  One
  // element per load: reading them four at a time from a copy of the weights stored
  // column by column measured slower (16 cache lines per load instead of 4).
  static __device__ __forceinline__ void load_w(TypedFrag &f, const float *wt, uint32_t lane_off) {
#pragma unroll
    for (int cb = 0; cb < kCB; ++cb)
#pragma unroll
      for (int j = 0; j < KS; ++j)
#pragma unroll
        for (int s = 0; s < 4; ++s)
          f.w[cb][j][s] = load_at<float>(wt, (lane_off + (16u * j + s) * MC + 16u * cb) * 4u);
  }
  static __device__ __forceinline__ floatx4 mma(const TypedFrag &f, int cb) {
    floatx4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < KS; ++j) {
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(f.x[j].x, f.w[cb][j][0], acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(f.x[j].y, f.w[cb][j][1], acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(f.x[j].z, f.w[cb][j][2], acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x4f32(f.x[j].w, f.w[cb][j][3], acc, 0, 0, 0);
    }
    return acc;
  }
};

template <int KS, int MC>
struct TypedFrag<bf16_t, KS, MC> {
  static constexpr int kCB = Cols<MC>::kCB;
  uint2 x[KS];            // four bf16: k = 16 j + 4 q .. + 3
  uint2 w[kCB][KS];       // my column block c: W[16 j + 4 q .. + 3][16 (cb0 + c) + n]
  static __device__ __forceinline__ void load_x(TypedFrag &f, const bf16_t *x, uint32_t row, int q) {
#pragma unroll
    for (int j = 0; j < KS; ++j)
      f.x[j] = load_at<uint2>(x, (row * (16u * KS) + 16u * j + 4u * q) * 2u);
  }
  static __device__ __forceinline__ void load_w(TypedFrag &f, const bf16_t *wt, uint32_t lane_off) {
#pragma unroll
    for (int cb = 0; cb < kCB; ++cb)
#pragma unroll
      for (int j = 0; j < KS; ++j) {
        uint32_t h[4];
#pragma unroll
        for (int s = 0; s < 4; ++s)
          h[s] = load_at<bf16_t>(wt, (lane_off + (16u * j + s) * MC + 16u * cb) * 2u);
        f.w[cb][j] = make_uint2(h[0] | (h[1] << 16), h[2] | (h[3] << 16));
      }
  }
  static __device__ __forceinline__ floatx4 mma(const TypedFrag &f, int cb) {
    floatx4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < KS; ++j)
      acc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(shortx4, f.x[j]),
                                                      __builtin_bit_cast(shortx4, f.w[cb][j]), acc,
                                                      0, 0, 0);
    return acc;
  }
};

struct ChunkIds {
  int src;                // source node of row n (-1: pad)
  uint32_t dst4;          // destinations inside the tile of rows 4 q .. 4 q + 3, one byte each
  int edge;               // edge id of row 4 q + (n & 3) (-1: pad)
  int type;               // relation of the chunk | its block mask << 16
};

template <typename T, int KS, int MC>
struct ChunkData {
  TypedFrag<T, KS, MC> f;
  float sc;               // scale of row 4 q + (n & 3)
  uint32_t dst4;
  unsigned hit;           // blocks of the tile the chunk has rows in (the same in every lane)
};

// lane L of my row of 16 lanes
template <int L>
__device__ __forceinline__ float row_share(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x150 + L, 0xF, 0xF, true));
}

// The messages of a chunk as bf16 terms whose sum is the message: one term for bf16
// (the message rounded to nearest even, what the two-operator chain stores), three
// truncated terms for fp32 (8 + 8 + 8 significant bits).  A term is the B operand of
// v_mfma_f32_16x16x16_bf16: lane (n, q) holds rows 4 q .. 4 q + 3 of column n.
template <typename T>
struct Terms;
template <>
struct Terms<bf16_t> {
  static constexpr int kTerms = 1;
  static __device__ __forceinline__ void split(const float (&m)[4], uint2 (&t)[1]) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    // v_cvt_pk_bf16_f32: round to nearest even, like f32_to_bf16_bits
    const bf16x2 lo = __builtin_convertvector(f32x2{m[0], m[1]}, bf16x2);
    const bf16x2 hi = __builtin_convertvector(f32x2{m[2], m[3]}, bf16x2);
    t[0] = make_uint2(__builtin_bit_cast(uint32_t, lo), __builtin_bit_cast(uint32_t, hi));
  }
};
template <>
struct Terms<float> {
  static constexpr int kTerms = 3;
  static __device__ __forceinline__ void split(const float (&m)[4], uint2 (&t)[3]) {
    uint32_t h[3][4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float r = m[i];
#pragma unroll
      for (int k = 0; k < 3; ++k) {
        h[k][i] = __float_as_uint(r);                        // its upper half is the term
        if (k < 2) r -= __uint_as_float(h[k][i] & 0xffff0000u);   // exact
      }
    }
#pragma unroll
    for (int k = 0; k < 3; ++k)     // upper halves of two values in one word
      t[k] = make_uint2(__builtin_amdgcn_perm(h[k][1], h[k][0], 0x07060302u),
                        __builtin_amdgcn_perm(h[k][3], h[k][2], 0x07060302u));
  }
};

// The value of a message as it enters the sum.
__device__ __forceinline__ float as_summed(float m, float) { return m; }
__device__ __forceinline__ float as_summed(float m, bf16_t) {
  return __uint_as_float(f32_to_bf16_bits(m) << 16);
}
__device__ __forceinline__ bool is_finite(float v) {
  return (__float_as_uint(v) & 0x7f800000u) != 0x7f800000u;
}

__device__ __forceinline__ float activated(float o, int act) {
  return act == GA_ACT_ELU ? elu(o) : relu_keep_nan(o);
}

__device__ __forceinline__ void store_row4(float *p, const float4 &v) {
  *reinterpret_cast<float4 *>(p) = v;
}
__device__ __forceinline__ void store_row4(bf16_t *p, const float4 &v) {
  *reinterpret_cast<uint2 *>(p) = make_uint2(pack_bf16(v.x, v.y), pack_bf16(v.z, v.w));
}

// Elements of a tile that received a message that is not finite, by kind: bit
// 4 b + i of word cb is element (b, cb, i) of the lane (up to 9 blocks: 36 bits).
template <int kCB>
struct Poison {
  uint64_t pinf[kCB], ninf[kCB], nan[kCB];
};

struct TypedArgs {
  const int32_t *chunk_type, *slot_src, *slot_edge;
  const uint32_t *slot_dst4;
  const void *x, *W;
  const float *row_scale;
};

// The chunks first, first + kTurns, ... < c1 of a tile into the lane's share of the
// wavefront's 128 x (16 kCB) tile: tile[b][c][i] = row 16 b + 4 q + i, column 16 c + n of
// the wavefront's columns (w_lane already points at them).  CHECKED: messages that
// are not finite are replaced by zero and recorded in `poison`.
template <typename T, int KS, int MC, bool SCALED, bool CHECKED, int NB>
__device__ __forceinline__ void walk_chunks(const TypedArgs &A, int first, int c1, int n, int q,
                                            floatx4 (&tile)[NB][Cols<MC>::kCB],
                                            Poison<Cols<MC>::kCB> &poison) {
  constexpr int kTerms = Terms<T>::kTerms;
  constexpr int kCB = Cols<MC>::kCB, kTurns = Cols<MC>::kTurns;
  using Frag = TypedFrag<T, KS, MC>;
  using Data = ChunkData<T, KS, MC>;
  const uint32_t w_lane = (4u * q) * MC + Cols<MC>::lane_col(n);
  // Loads are issued without branches around them (a chunk index past the end reads the
  // last chunk again, a pad slot reads row 0 of x and edge 0 of the scale; no row of a
  // tile selects what they produce): the waits for the loads of the chunk before then
  // leave the newer ones in flight.
  auto load_ids = [&](int c, ChunkIds &I) __attribute__((always_inline)) {
    c = c < c1 ? c : c1 - 1;
    I.src = A.slot_src[c * kChunk + n];
    I.dst4 = A.slot_dst4[c * 4 + q];
    I.edge = A.slot_edge[c * kChunk + 4 * q + (n & 3)];
    // A vector load on purpose: scalar loads return out of order, so waiting for the
    // type of the chunk at hand would also wait for the one requested just now.
    I.type = __hip_atomic_load(A.chunk_type + c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  };
  auto load_data = [&](const ChunkIds &I, Data &D) __attribute__((always_inline)) {
    Frag::load_x(D.f, (const T *)A.x, (uint32_t)(I.src < 0 ? 0 : I.src), q);
    const int word = __builtin_amdgcn_readfirstlane(I.type);     // relation | blocks << 16
    Frag::load_w(D.f, (const T *)A.W + (int64_t)(word & 0xffff) * (16 * KS * MC), w_lane);
    D.hit = (unsigned)word >> 16;
    D.sc = SCALED ? load_at<float>(A.row_scale, (uint32_t)(I.edge < 0 ? 0 : I.edge) * 4u) : 1.0f;
    D.dst4 = I.dst4;
  };
  auto compute = [&](const Data &d) __attribute__((always_inline)) {
    // ---- messages of the chunk: rows 4 q + i, columns 16 cb + n ------------------------
    float sc[4] = {1.0f, 1.0f, 1.0f, 1.0f};
    if (SCALED) {
      sc[0] = row_share<0>(d.sc); sc[1] = row_share<1>(d.sc);
      sc[2] = row_share<2>(d.sc); sc[3] = row_share<3>(d.sc);
    }
    uint2 t[kCB][kTerms];
#pragma unroll
    for (int cb = 0; cb < kCB; ++cb) {
      const floatx4 acc = Frag::mma(d.f, cb);
      float m[4] = {acc[0] * sc[0], acc[1] * sc[1], acc[2] * sc[2], acc[3] * sc[3]};
      if (CHECKED) {
        bool fin = true;
#pragma unroll
        for (int i = 0; i < 4; ++i) fin = fin && is_finite(as_summed(m[i], T()));
        if (__builtin_amdgcn_ballot_w64(!fin) != 0) {
          // row r of the chunk is held by the lanes (., r / 4) in m[r % 4]; its element
          // of the tile by register dst % 4 of the lanes (., dst % 16 / 4) of block dst / 16
#pragma unroll
          for (int r = 0; r < kChunk; ++r) {
            const int dst =
                (__builtin_amdgcn_readlane(d.dst4, 16 * (r >> 2)) >> (8 * (r & 3))) & 0xff;
            const float v = as_summed(__shfl(m[r & 3], 16 * (r >> 2) + n), T());
            if (dst < 16 * NB && q == ((dst & 15) >> 2) && !is_finite(v)) {
              const uint64_t bit = 1ull << ((dst >> 4) * 4 + (dst & 3));
              poison.nan[cb] |= v != v ? bit : 0ull;
              poison.pinf[cb] |= v == INFINITY ? bit : 0ull;
              poison.ninf[cb] |= v == -INFINITY ? bit : 0ull;
            }
          }
#pragma unroll
          for (int i = 0; i < 4; ++i) m[i] = is_finite(as_summed(m[i], T())) ? m[i] : 0.0f;
        }
      }
      Terms<T>::split(m, t[cb]);
    }
    // destination of row 4 q + j inside the tile, minus my lane's row of a block
    int u[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) u[j] = (int)((d.dst4 >> (8 * j)) & 0xffu) - n;
    const unsigned hit = d.hit;
    // tile[b] += S_b @ messages: S_b[i][r] = 1 where row r of the chunk goes to row
    // 16 b + i of the tile; lane (n, q) holds S_b[n][4 q .. 4 q + 3]
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      if (hit >> b & 1u) {
        const uint32_t s0 = u[0] == 16 * b ? 0x3f80u : 0u, s1 = u[1] == 16 * b ? 0x3f800000u : 0u;
        const uint32_t s2 = u[2] == 16 * b ? 0x3f80u : 0u, s3 = u[3] == 16 * b ? 0x3f800000u : 0u;
        const shortx4 sel = __builtin_bit_cast(shortx4, make_uint2(s0 | s1, s2 | s3));
#pragma unroll
        for (int k = 0; k < kTerms; ++k)
#pragma unroll
          for (int cb = 0; cb < kCB; ++cb)    // independent accumulators back to back
            tile[b][cb] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(
                sel, __builtin_bit_cast(shortx4, t[cb][k]), tile[b][cb], 0, 0, 0);
      }
    }
  };

  if (first >= c1) return;
  // kDepth sets of registers take turns (the loop is unrolled kDepth times, so no
  // copies): the ids of one of my chunks are requested kDepth, its rows and weights
  // kDepth - 1 of my chunks ahead of the arithmetic.  Ids are requested before the rows
  // of the same step: the wait for them at the next step then leaves that step's rows
  // and weights in flight (loads return in order).  Three and four sets measured slower
  // at every shape (fewer wavefronts fit, and the kernel is not waiting for memory).
  constexpr int kDepth = 2;
  ChunkIds ids[kDepth];
  Data data[kDepth];
#pragma unroll
  for (int s = 0; s < kDepth; ++s) load_ids(first + s * kTurns, ids[s]);
#pragma unroll
  for (int s = 0; s + 1 < kDepth; ++s) load_data(ids[s], data[s]);
  for (int c = first; c < c1; c += kDepth * kTurns) {
#pragma unroll
    for (int s = 0; s < kDepth; ++s) {
      constexpr int kLast = kDepth - 1;
      load_ids(c + (s + kDepth) * kTurns, ids[s]);
      load_data(ids[(s + kLast) % kDepth], data[(s + kLast) % kDepth]);
      if (s == 0 || c + s * kTurns < c1) compute(data[s]);
    }
  }
}

// Wavefronts per SIMD the kernel is compiled for: three where the registers allow it
// without spilling (one k step of 16), no promise otherwise.
constexpr int typed_waves_per_simd(int KS, int MC) { return KS == 1 ? 3 : 1; }

template <typename T, int KS, int MC, bool SCALED, int NB>
__global__ __launch_bounds__(kTypedBlock, typed_waves_per_simd(KS, MC)) void typed_tiles_kernel(
    const int32_t *__restrict__ tile_chunk_pointer, TypedArgs A, T *__restrict__ out,
    int64_t n_rows, int act) {
  constexpr int kTileRows = 16 * NB;
  constexpr int kCB = Cols<MC>::kCB, kColGroups = Cols<MC>::kColGroups, kTurns = Cols<MC>::kTurns;
  constexpr int kMergeStride = Cols<MC>::kMergeStride;
  static_assert(4 * NB <= 64 && kTileRows <= kMaxTileRows, "one bit per tile element of a lane");
  __shared__ __attribute__((aligned(16))) float merged[kTileRows * kMergeStride];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int lane = threadIdx.x & (kWave - 1);
  const int n = lane & 15, q = lane >> 4;
  const int c0 = tile_chunk_pointer[blockIdx.x], c1 = tile_chunk_pointer[blockIdx.x + 1];
  // my column group and my turn on the chunks
  const int colgroup = wave % kColGroups, turn = wave / kColGroups;
  A.W = static_cast<const T *>(A.W) + 16 * kCB * colgroup;
  floatx4 tile[NB][kCB];
  Poison<kCB> poison;
#pragma unroll
  for (int cb = 0; cb < kCB; ++cb) poison.pinf[cb] = poison.ninf[cb] = poison.nan[cb] = 0ull;
  auto clear = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
      for (int cb = 0; cb < kCB; ++cb) tile[b][cb] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
  };
  clear();
  walk_chunks<T, KS, MC, SCALED, false, NB>(A, c0 + turn, c1, n, q, tile, poison);
  // A message that is not finite turns the zeros of the selection matrix into NaN for
  // the rows around it.  Such a message leaves something that is not finite in the tile:
  // then the wavefront walks its chunks again, keeping those messages out of the matrix
  // cores and adding them here instead.
  bool fin = true;
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int cb = 0; cb < kCB; ++cb)
#pragma unroll
      for (int i = 0; i < 4; ++i) fin = fin && is_finite(tile[b][cb][i]);
  if (__builtin_amdgcn_ballot_w64(!fin) != 0) {
    clear();
    walk_chunks<T, KS, MC, SCALED, true, NB>(A, c0 + turn, c1, n, q, tile, poison);
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
      for (int cb = 0; cb < kCB; ++cb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int bit = 4 * b + i;
          if (poison.pinf[cb] >> bit & 1ull) tile[b][cb][i] += INFINITY;
          if (poison.ninf[cb] >> bit & 1ull) tile[b][cb][i] -= INFINITY;
          if (poison.nan[cb] >> bit & 1ull) tile[b][cb][i] = NAN;
        }
  }
  // ---- the partial tiles meet in LDS: the column groups side by side, the wavefronts of
  // a group one after the other in a fixed order ------------------------------------------
  for (int w = 0; w < kTurns; ++w) {
    if (turn == w && (MC >= 16 || n < MC)) {
#pragma unroll
      for (int b = 0; b < NB; ++b) {
#pragma unroll
        for (int cb = 0; cb < kCB; ++cb)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float *p = merged + (16 * b + 4 * q + i) * kMergeStride + 16 * (kCB * colgroup + cb) + n;
            *p = w == 0 ? tile[b][cb][i] : *p + tile[b][cb][i];
          }
        // one block at a time: few values in flight, not the whole tile
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __syncthreads();
  }
  // ---- and go to memory: a thread moves four columns of a row at a time -----------------
  const int64_t row0 = (int64_t)blockIdx.x * kTileRows;
  for (int i = threadIdx.x; i < kTileRows * (MC / 4); i += kTypedBlock) {
    const int r = i / (MC / 4), c4 = i % (MC / 4);
    if (row0 + r < n_rows) {
      float4 v = *reinterpret_cast<const float4 *>(merged + r * kMergeStride + 4 * c4);
      if (act != GA_ACT_NONE) {
        // the activation between layers (examples/RGCN/RGCN.py:69) on the fp32 sums, before
        // they are rounded and stored; NaN stays NaN
        v.x = activated(v.x, act); v.y = activated(v.y, act);
        v.z = activated(v.z, act); v.w = activated(v.w, act);
      }
      store_row4(out + (row0 + r) * MC + 4 * c4, v);
    }
  }
}

template <typename T, int KS, int MC, int NB>
int launch_typed_nb(const int32_t *tcp, const TypedArgs &A, void *out, int64_t n_rows, int act,
                    hipStream_t s) {
  const dim3 grid((unsigned)tiles_of(n_rows, 16 * NB));
  if (A.row_scale)
    hipLaunchKernelGGL((typed_tiles_kernel<T, KS, MC, true, NB>), grid, dim3(kTypedBlock), 0, s,
                       tcp, A, (T *)out, n_rows, act);
  else
    hipLaunchKernelGGL((typed_tiles_kernel<T, KS, MC, false, NB>), grid, dim3(kTypedBlock), 0, s,
                       tcp, A, (T *)out, n_rows, act);
  return launch_status();
}

template <typename T, int KS, int MC>
int launch_typed_mc(const int32_t *tcp, const TypedArgs &A, void *out, int64_t n_rows,
                    int64_t tile_rows, int act, hipStream_t s) {
  if (tile_rows == 144) return launch_typed_nb<T, KS, MC, 9>(tcp, A, out, n_rows, act, s);
  return launch_typed_nb<T, KS, MC, 8>(tcp, A, out, n_rows, act, s);
}

template <typename T, int KS>
int launch_typed(const int32_t *tcp, const TypedArgs &A, void *out, int64_t n_rows,
                 int64_t tile_rows, int64_t M, int act, hipStream_t s) {
  switch (M) {
    case 8: return launch_typed_mc<T, KS, 8>(tcp, A, out, n_rows, tile_rows, act, s);
    case 16: return launch_typed_mc<T, KS, 16>(tcp, A, out, n_rows, tile_rows, act, s);
    case 32: return launch_typed_mc<T, KS, 32>(tcp, A, out, n_rows, tile_rows, act, s);
    default: return launch_typed_mc<T, KS, 64>(tcp, A, out, n_rows, tile_rows, act, s);
  }
}

// Workgroups of the kernel that a CU holds at once (three wavefronts per SIMD by its
// registers, four wavefronts per workgroup).
constexpr int kTypedGroupsPerCu = 3;

int typed_cu_count() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
      cus = v;
    else
      cus = 256;
  }
  return cus;
}

}  // namespace
}  // namespace ga

extern "C" {

int64_t ga_typed_tile_rows(int64_t n_rows) {
  // The kernel holds kTypedGroupsPerCu workgroups per CU at once, one workgroup per tile:
  // of the two tile heights take the one whose tiles fill whole rounds of the chip best
  // (a last round with a few workgroups costs as much as a full one); 128 on a tie.
  const int64_t slots = (int64_t)ga::typed_cu_count() * ga::kTypedGroupsPerCu;
  int64_t best = 128;
  double best_fill = 0.0;
  for (int64_t rows : {(int64_t)128, (int64_t)144}) {
    const int64_t tiles = ga::tiles_of(n_rows < 1 ? 1 : n_rows, rows);
    const int64_t rounds = (tiles + slots - 1) / slots;
    const double fill = (double)tiles / (double)(rounds * slots);
    if (fill > best_fill + 1e-9) {
      best_fill = fill;
      best = rows;
    }
  }
  return best;
}

int64_t ga_typed_tiles_chunk_capacity(int64_t n_rows, int64_t n_edges, int64_t n_types,
                                      int64_t tile_rows) {
  if (n_rows < 0 || n_edges < 0 || n_types <= 0 || !ga::tile_rows_ok(tile_rows)) return 0;
  // every (tile, relation) group that has edges wastes less than one chunk
  const int64_t groups = ga::tiles_of(n_rows, tile_rows) * n_types;
  return (n_edges + ga::kChunk - 1) / ga::kChunk + (groups < n_edges ? groups : n_edges);
}

size_t ga_typed_tiles_workspace_bytes(int64_t n_rows, int64_t n_edges, int64_t n_types,
                                      int64_t tile_rows) {
  if (n_rows < 0 || n_edges < 0 || n_types <= 0 || n_edges > 0x7fffffff) return 0;
  if (!ga::tile_rows_ok(tile_rows)) return 0;
  const int64_t groups = ga::tiles_of(n_rows, tile_rows) * n_types;
  if (groups > 0x7ffffffe) return 0;
  ga::TilesLayout L;
  if (ga::tiles_layout(groups, n_edges, L) != GA_OK) return 0;
  return L.total;
}

int ga_typed_tiles_build(const int32_t *row_of_slot, const int32_t *nbr, const int32_t *eid,
                         const int32_t *type_pointer, int64_t n_rows, int64_t n_edges,
                         int64_t n_types, int64_t tile_rows, int32_t *tile_chunk_pointer,
                         int32_t *chunk_type,
                         int32_t *slot_src, unsigned char *slot_dst, int32_t *slot_edge,
                         void *workspace, size_t workspace_bytes, ga_stream_t stream) {
  using namespace ga;
  if (n_rows < 0 || n_edges < 0 || n_types <= 0) return GA_EINVAL;
  if (n_rows > 0x7fffffff || n_edges > 0x7fffffff || n_types > 0x7fffffff) return GA_EINVAL;
  if (!tile_rows_ok(tile_rows)) return GA_EINVAL;
  if (n_types > 0xffff) return GA_EUNSUPPORTED;      // the relation shares a word with the block mask
  const int64_t n_tiles = tiles_of(n_rows, tile_rows), n_groups = n_tiles * n_types;
  if (n_groups > 0x7ffffffe) return GA_EUNSUPPORTED;
  const int64_t cap = ga_typed_tiles_chunk_capacity(n_rows, n_edges, n_types, tile_rows);
  if (cap * kChunk > 0x7fffffff) return GA_EUNSUPPORTED;
  if (!tile_chunk_pointer || !type_pointer) return GA_EINVAL;
  if (n_edges > 0 && (!row_of_slot || !nbr || !chunk_type || !slot_src || !slot_dst || !slot_edge))
    return GA_EINVAL;
  if (!aligned(slot_dst, 4) || !aligned(slot_edge, 16) || !aligned(slot_src, 4)) return GA_EALIGN;
  TilesLayout L;
  const int rc = tiles_layout(n_groups, n_edges, L);
  if (rc != GA_OK) return rc;
  if (!workspace || workspace_bytes < L.total || !aligned(workspace, 256)) return GA_EWORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  char *ws = (char *)workspace;
  int32_t *key = (int32_t *)(ws + L.key), *key_sorted = (int32_t *)(ws + L.key_sorted);
  int32_t *ids = (int32_t *)(ws + L.ids), *ids_sorted = (int32_t *)(ws + L.ids_sorted);
  int32_t *first = (int32_t *)(ws + L.first), *chunks = (int32_t *)(ws + L.chunks);
  int32_t *base = (int32_t *)(ws + L.base);
  if (n_edges > 0) {
    const int64_t blocks = (n_edges + kBlock - 1) / kBlock;
    hipLaunchKernelGGL(typed_keys_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, s, row_of_slot,
                       eid, type_pointer, (int)n_types, n_edges, (int)tile_rows, key, ids);
    size_t tb = L.sort_bytes;
    hipError_t e = rocprim::radix_sort_pairs(ws + L.temp, tb, key, key_sorted, ids, ids_sorted,
                                             (size_t)n_edges, 0, end_bit_for(n_groups), s);
    if (e != hipSuccess) return (int)e;
  }
  {
    const int64_t blocks = (n_groups + 1 + kBlock - 1) / kBlock;
    hipLaunchKernelGGL(typed_group_chunks_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, s,
                       key_sorted, n_groups, n_edges, first, chunks);
    size_t tb = L.scan_bytes;
    hipError_t e = rocprim::exclusive_scan(ws + L.temp, tb, chunks, base, (int32_t)0,
                                           (size_t)(n_groups + 1), rocprim::plus<int32_t>(), s);
    if (e != hipSuccess) return (int)e;
    const int64_t tblocks = (n_tiles + 1 + kBlock - 1) / kBlock;
    hipLaunchKernelGGL(typed_tile_pointer_kernel, dim3((unsigned)tblocks), dim3(kBlock), 0, s, base,
                       n_tiles, (int)n_types, tile_chunk_pointer);
  }
  if (cap > 0) {
    const int64_t blocks = (cap * kChunk + kBlock - 1) / kBlock;
    hipLaunchKernelGGL(typed_fill_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, s, base, first,
                       ids_sorted, row_of_slot, nbr, eid, n_groups, (int)n_types, (int)tile_rows, cap,
                       chunk_type,
                       slot_src, slot_dst, slot_edge);
  }
  return launch_status();
}

int ga_typed_spmm(const int32_t *tile_chunk_pointer, const int32_t *chunk_type,
                  const int32_t *slot_src, const unsigned char *slot_dst,
                  const int32_t *slot_edge, const void *x, const void *W,
                  const float *row_scale, void *out, int64_t n_rows, int64_t n_src,
                  int64_t n_edges, int64_t n_types, int64_t tile_rows, int64_t K, int64_t M,
                  int dtype, ga_stream_t stream) {
  return ga_typed_spmm_act(tile_chunk_pointer, chunk_type, slot_src, slot_dst, slot_edge, x, W,
                           row_scale, out, n_rows, n_src, n_edges, n_types, tile_rows, K, M,
                           GA_ACT_NONE, dtype, stream);
}

int ga_typed_spmm_act(const int32_t *tile_chunk_pointer, const int32_t *chunk_type,
                      const int32_t *slot_src, const unsigned char *slot_dst,
                      const int32_t *slot_edge, const void *x, const void *W,
                      const float *row_scale, void *out, int64_t n_rows, int64_t n_src,
                      int64_t n_edges, int64_t n_types, int64_t tile_rows, int64_t K, int64_t M,
                      int activation, int dtype, ga_stream_t stream) {
  using namespace ga;
  if (activation < GA_ACT_NONE || activation > GA_ACT_ELU) return GA_EINVAL;
  if (n_rows < 0 || n_src < 0 || n_edges < 0 || n_types <= 0 || K <= 0 || M <= 0) return GA_EINVAL;
  if (!tile_rows_ok(tile_rows)) return GA_EINVAL;
  if (n_rows > 0x7fffffff || n_edges > 0x7fffffff) return GA_EINVAL;
  if (dtype != GA_F32 && dtype != GA_BF16) return GA_EINVAL;
  if (!typed_cols_ok(M) || K % 16 != 0 || K > 64 || n_types > 0xffff) return GA_EUNSUPPORTED;
  const size_t esz = dtype == GA_F32 ? 4 : 2;
  // the kernel addresses x, one relation of W and row_scale with 32-bit byte offsets,
  // the slot arrays with 32-bit indices
  if ((uint64_t)n_src * K * esz > 0xffffffffull || (uint64_t)n_edges * 4 > 0xffffffffull ||
      ga_typed_tiles_chunk_capacity(n_rows, n_edges, n_types, tile_rows) * kChunk > 0x7fffffff)
    return GA_EUNSUPPORTED;
  if (n_rows == 0) return GA_OK;
  if (!tile_chunk_pointer || !out) return GA_EINVAL;
  if (n_edges > 0 && (!chunk_type || !slot_src || !slot_dst || !slot_edge || !x || !W))
    return GA_EINVAL;
  // four-element reads of the rows of x and writes of the rows of out
  if (!aligned(slot_edge, 4) || !aligned(slot_dst, 4) || !aligned(x, 4 * esz) ||
      !aligned(out, 4 * esz) || !aligned(W, esz) || (row_scale && !aligned(row_scale, 4)))
    return GA_EALIGN;
  hipStream_t s = (hipStream_t)stream;
  const TypedArgs A{chunk_type, slot_src, slot_edge, (const uint32_t *)slot_dst, x, W, row_scale};
  const int ks = (int)(K / 16);
#define GA_TYPED(T, KS) \
  return launch_typed<T, KS>(tile_chunk_pointer, A, out, n_rows, tile_rows, M, activation, s)
  if (dtype == GA_F32) {
    switch (ks) {
      case 1: GA_TYPED(float, 1);
      case 2: GA_TYPED(float, 2);
      case 3: GA_TYPED(float, 3);
      default: GA_TYPED(float, 4);
    }
  }
  switch (ks) {
    case 1: GA_TYPED(bf16_t, 1);
    case 2: GA_TYPED(bf16_t, 2);
    case 3: GA_TYPED(bf16_t, 3);
    default: GA_TYPED(bf16_t, 4);
  }
#undef GA_TYPED
}

}  // extern "C"
