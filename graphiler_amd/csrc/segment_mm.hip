// segment_mm (typed linear) for gfx950 on the matrix cores.
//
//   Y[r, h, :] = X[r, h, :] @ W[type(r), h, :, :]      rows sorted by type
//
// Every configured shape (K, M <= 128) is bound by streaming X in and Y out, so
// the kernel is organised around the row stream: a workgroup (4 waves) takes a
// chunk of consecutive rows of ONE type, keeps that type's weights in LDS, and
// each wave pushes 16-row tiles through MFMA with fp32 accumulation:
//   fp32          v_mfma_f32_16x16x4_f32; one 16-byte X load per lane covers
//                 K = 16 (its four components feed four MFMAs; the k order
//                 inside a block is permuted identically for X and W, which a
//                 dot product allows);
//   bf16, K%32==0 v_mfma_f32_16x16x32_bf16, one 16-byte X load covers K = 32;
//   bf16, other   v_mfma_f32_16x16x16_bf16, one 8-byte X load covers K = 16.
// Heads are folded into one product with a block-diagonal weight tile
// (Kt = heads*K, Mt = heads*M, zeros off the diagonal): whole rows are loaded
// with wide accesses; the MFMAs spent on zero blocks are far below the time the
// row stream takes.  All X fragments of a
// tile are loaded before its MFMAs.  Accumulators come out as D[row][column]
// with 16 adjacent lanes holding 16 adjacent columns, so stores coalesce; for
// bf16 two column blocks interleave their columns (even / odd) so a lane packs
// two neighbouring outputs into one 4-byte store.  The type of a chunk is found
// on the device from type_pointer (block-wide prefix sum of chunks per type):
// no host copy, no synchronisation.
//
// Two fused forms of the exact-shape kernel serve per-edge products whose
// operand lives on the nodes (Y[e] = X[endpoint(e)] @ W[type(e)], the
// Broadcast -> bmm pairs of examples/RGCN/RGCN.py:26-28 and
// examples/HGT/HGT.py:35-44): rows of X are read through an index instead of
// being materialised per edge first, and the product can be reduced on the spot
// against a second gathered row, out[e, h] = <Y[e, h, :], Q[q_index[e], h, :]>
// (HGT's sum(k * q)), in which case Y never reaches memory.
#include "common.h"
#include "wide_mm.h"

#include <type_traits>

namespace ga {
namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short shortx4 __attribute__((ext_vector_type(4)));

constexpr int kTileRows = 16;                   // rows per wave tile
constexpr int kWaves = kBlock / kWave;          // 4
constexpr int kTileBlock = kTileRows * kWaves;  // 64 rows per workgroup step
constexpr int kMaxLds = 64 * 1024;          // default per-workgroup LDS limit
constexpr int kMaxLdsOptIn = 158 * 1024;    // gfx950 has 160 KB per CU

// Raises a kernel's dynamic LDS limit when a tile needs more than 64 KB.
inline bool allow_lds(const void *kernel, size_t bytes) {
  if (bytes <= (size_t)kMaxLds) return true;
  if (bytes > (size_t)kMaxLdsOptIn) return false;
  return hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                             (int)bytes) == hipSuccess;
}
constexpr int kMaxFrags = 8;                    // X fragments preloaded per tile

// Problem seen by one launch: rows of type t use the (Kt x Mt) block-diagonal
// tile built from `hb` consecutive (K x M) head blocks of W[t].
struct MmGeom {
  int n_types;
  int chunk_rows;
  int K, M, hb;        // per-head sizes, heads folded into the tile
  int Kt, Mt;          // hb*K, hb*M
  int KB, MB;          // k blocks / 16-column blocks of the tile
  int64_t ldx, ldy;    // row strides of X and Y (elements)
  int64_t w_type_stride;  // elements between W[t] and W[t+1]
  int64_t ldw;            // elements between rows k and k+1 of one (K x M) block
  int64_t rows;           // used when there is no type pointer: one type, rows [0, rows)
  // dense projection wider than one tile: column passes of pass_cols columns
  // (whole heads of dph columns) inside one launch; n_pass <= 1: a single tile
  int n_pass, pass_cols, m_total, dph;
  // dot form: tile column c sits in column block c % 2^perm_shift at lane column
  // c >> perm_shift, so a lane's columns are adjacent in memory; -1: natural order
  int perm_shift;
};

// Optional gather / dot-product operands of the exact-shape kernel.
struct MmExt {
  const int64_t *x_index;   // row r reads X[x_index[r]]; null: X[r]
  const void *Q;            // dot operand rows (ldq elements apart); null: store Y
  const int64_t *q_index;   // row r is reduced against Q[q_index[r]]; null: Q[r]
  float *dot;               // (rows, ldd) fp32, column = head
  const float *scale;       // (n_types, ldd) factor per type and head; null: 1
  const float *row_scale;   // kEpiStore: Y[r, :] *= row_scale[r]; null: 1
  int64_t ldq, ldd;
  const float *a_l, *a_r;   // attention vectors over the tile's columns (kEpiAttn)
  float *el, *er;           // (rows, ldd) fp32
  int n_heads;              // heads inside the tile (kEpiAttn)
  unsigned head_end;        // kEpiAttn: bit cb: a head's columns end with column block cb
  int half_heads;           // kEpiAttn, bf16, head width 16: a block pair holds two heads
};

// Column of the tile held by lane column j of column block cb.
template <bool PAIRED>
__device__ __forceinline__ int tile_col(int cb, int j) {
  return PAIRED ? ((cb >> 1) * 32 + 2 * j + (cb & 1)) : (cb * 16 + j);
}

template <typename T, int KBLK>
struct Mma;

template <>
struct Mma<float, 16> {          // LDS: [k][col], row stride ws floats
  typedef float4 frag_t;
  static constexpr bool kPaired = false;
  static __host__ __device__ int mb_pad(int MB) { return MB; }
  static __host__ __device__ int ws(int KB, int MB) { return MB * 16 + 4; }
  static __host__ __device__ int tile_elems(int KB, int MB) { return KB * 16 * ws(KB, MB); }
  static __device__ __forceinline__ frag_t zero() { return make_float4(0, 0, 0, 0); }
  static __device__ __forceinline__ frag_t load(const float *p) {
    return *reinterpret_cast<const float4 *>(p);
  }
  static __device__ __forceinline__ int k_of_lane(int lk) { return lk * 4; }
  static __device__ __forceinline__ floatx4 mma(floatx4 acc, const float *tile, int wsv,
                                                int kb, int cb, int lr, int lk,
                                                const frag_t &x) {
    const float *w = tile + (kb * 16 + lk * 4) * wsv + cb * 16 + lr;
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(x.x, w[0], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(x.y, w[wsv], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(x.z, w[2 * wsv], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(x.w, w[3 * wsv], acc, 0, 0, 0);
    return acc;
  }
  // zero the padded tile, then copy the hb diagonal (K x M) blocks; no integer
  // divisions: lanes run along the columns, waves along the rows
  static __device__ void stage(const float *__restrict__ w, float *tile,
                               const MmGeom &g) {
    const int wsv = ws(g.KB, g.MB);
    const int total4 = (g.KB * 16 * wsv) >> 2;          // wsv is a multiple of 4
    for (int i = threadIdx.x; i < total4; i += kBlock)
      reinterpret_cast<float4 *>(tile)[i] = make_float4(0, 0, 0, 0);
    __syncthreads();
    const int tx = threadIdx.x & (kWave - 1), ty = threadIdx.x / kWave;
    const bool vec = (g.M & 3) == 0 && (g.ldw & 3) == 0 && g.perm_shift < 0 &&
                     (reinterpret_cast<uintptr_t>(w) & 15) == 0;
    for (int h = 0; h < g.hb; ++h) {
      const float *wh = w + (int64_t)h * g.K * g.ldw;
      float *th = tile + (h * g.K) * wsv + h * g.M;
      if (vec) {
        for (int k = ty; k < g.K; k += kBlock / kWave)
          for (int m = tx * 4; m < g.M; m += kWave * 4) {
            const float4 v = *reinterpret_cast<const float4 *>(wh + (int64_t)k * g.ldw + m);
            float *d = th + k * wsv + m;       // 16-byte aligned only when h*M is
            d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
          }
      } else {
        for (int k = ty; k < g.K; k += kBlock / kWave)
          for (int m = tx; m < g.M; m += kWave) {
            int c = h * g.M + m;                           // tile column
            if (g.perm_shift >= 0)
              c = (c & ((1 << g.perm_shift) - 1)) * 16 + (c >> g.perm_shift);
            tile[(h * g.K + k) * wsv + c] = wh[(int64_t)k * g.ldw + m];
          }
      }
    }
  }
};

// bf16 weights live transposed in LDS: [lane column][k], row stride ws elements,
// so a lane's k-contiguous fragment is one vector read.  LDS row cb*16 + j holds
// tile column tile_col<true>(cb, j).
template <int KBLK>
struct MmaBf16Base {
  static constexpr bool kPaired = true;
  static __host__ __device__ int mb_pad(int MB) { return (MB + 1) & ~1; }
  static __host__ __device__ int ws(int KB, int MB) { return KB * KBLK + 8; }
  static __host__ __device__ int tile_elems(int KB, int MB) {
    return mb_pad(MB) * 16 * ws(KB, MB);
  }
  // zero the padded tile, then transpose the hb diagonal (K x M) blocks: a
  // thread gathers 8 consecutive k of one column (loads coalesce across threads
  // along the columns) and writes them as one 16-byte LDS vector.  No divisions.
  static __device__ void stage(const bf16_t *__restrict__ w, bf16_t *tile,
                               const MmGeom &g) {
    const int wsv = ws(g.KB, g.MB);
    const int total8 = (mb_pad(g.MB) * 16 * wsv) >> 3;   // wsv is a multiple of 8
    for (int i = threadIdx.x; i < total8; i += kBlock)
      reinterpret_cast<uint4 *>(tile)[i] = make_uint4(0, 0, 0, 0);
    __syncthreads();
    const int tx = threadIdx.x & (kWave - 1), ty = threadIdx.x / kWave;
    for (int h = 0; h < g.hb; ++h) {
      const bf16_t *wh = w + (int64_t)h * g.K * g.ldw;
      for (int kc = ty * 8; kc < g.K; kc += (kBlock / kWave) * 8)
        for (int m = tx; m < g.M; m += kWave) {
          uint32_t v[8];
#pragma unroll
          for (int q = 0; q < 8; ++q)
            v[q] = kc + q < g.K ? (uint32_t)wh[(int64_t)(kc + q) * g.ldw + m] : 0u;
          const int c = h * g.M + m;                       // tile column
          const int lrow = g.perm_shift >= 0
                               ? (c & ((1 << g.perm_shift) - 1)) * 16 + (c >> g.perm_shift)
                               : ((c >> 5) * 2 + (c & 1)) * 16 + ((c & 31) >> 1);
          bf16_t *d = tile + lrow * wsv + h * g.K + kc;
          if (((h * g.K + kc) & 7) == 0) {
            uint4 o;
            o.x = v[0] | (v[1] << 16);
            o.y = v[2] | (v[3] << 16);
            o.z = v[4] | (v[5] << 16);
            o.w = v[6] | (v[7] << 16);
            *reinterpret_cast<uint4 *>(d) = o;
          } else {
#pragma unroll
            for (int q = 0; q < 8; ++q)
              if (kc + q < g.K) d[q] = (bf16_t)v[q];
          }
        }
    }
  }
};

template <>
struct Mma<bf16_t, 32> : MmaBf16Base<32> {
  typedef uint4 frag_t;
  static __device__ __forceinline__ frag_t zero() { return make_uint4(0, 0, 0, 0); }
  static __device__ __forceinline__ frag_t load(const bf16_t *p) {
    return *reinterpret_cast<const uint4 *>(p);
  }
  static __device__ __forceinline__ int k_of_lane(int lk) { return lk * 8; }
  static __device__ __forceinline__ floatx4 mma(floatx4 acc, const bf16_t *tile, int wsv,
                                                int kb, int cb, int lr, int lk,
                                                const frag_t &x) {
    const uint4 w = *reinterpret_cast<const uint4 *>(tile + (cb * 16 + lr) * wsv +
                                                     kb * 32 + lk * 8);
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, x),
                                                   __builtin_bit_cast(bf16x8, w),
                                                   acc, 0, 0, 0);
  }
};

template <>
struct Mma<bf16_t, 16> : MmaBf16Base<16> {
  typedef uint2 frag_t;
  static __device__ __forceinline__ frag_t zero() { return make_uint2(0, 0); }
  static __device__ __forceinline__ frag_t load(const bf16_t *p) {
    return *reinterpret_cast<const uint2 *>(p);
  }
  static __device__ __forceinline__ int k_of_lane(int lk) { return lk * 4; }
  static __device__ __forceinline__ floatx4 mma(floatx4 acc, const bf16_t *tile, int wsv,
                                                int kb, int cb, int lr, int lk,
                                                const frag_t &x) {
    const uint2 w = *reinterpret_cast<const uint2 *>(tile + (cb * 16 + lr) * wsv +
                                                     kb * 16 + lk * 4);
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(shortx4, x),
                                                     __builtin_bit_cast(shortx4, w),
                                                     acc, 0, 0, 0);
  }
};

// Which chunk of which type does this workgroup own?  chunks(t) =
// ceil(rows_t / chunk_rows); workgroup id -> (t, first row, end row).
__device__ __forceinline__ bool locate_chunk(const int32_t *__restrict__ tp,
                                             int n_types, int chunk_rows, int target,
                                             int &type, int &row0, int &row1) {
  __shared__ int scan[kBlock];
  __shared__ int found[3];
  if (!tp) {               // one type; the caller passes the row count as n_types
    type = 0;
    if ((int64_t)target * chunk_rows >= n_types) return false;
    row0 = target * chunk_rows;
    row1 = min(n_types, row0 + chunk_rows);
    return true;
  }
  if (threadIdx.x == 0) found[0] = -1;
  int base = 0;
  for (int t0 = 0; t0 < n_types; t0 += kBlock) {
    const int t = t0 + threadIdx.x;
    int p0 = 0, p1 = 0, cnt = 0;
    if (t < n_types) {
      p0 = tp[t];
      p1 = tp[t + 1];
      cnt = (p1 - p0 + chunk_rows - 1) / chunk_rows;
    }
    __syncthreads();
    scan[threadIdx.x] = cnt;
    __syncthreads();
    for (int off = 1; off < kBlock; off <<= 1) {
      const int add = threadIdx.x >= off ? scan[threadIdx.x - off] : 0;
      __syncthreads();
      scan[threadIdx.x] += add;
      __syncthreads();
    }
    const int incl = base + scan[threadIdx.x];
    const int excl = incl - cnt;
    if (cnt > 0 && target >= excl && target < incl) {
      found[0] = t;
      found[1] = p0 + (target - excl) * chunk_rows;
      found[2] = p1;
    }
    base += scan[kBlock - 1];
    if (base > target) break;   // uniform: every thread sees the same totals
  }
  __syncthreads();
  type = found[0];
  if (type < 0) return false;
  row0 = found[1];
  row1 = min(found[2], row0 + chunk_rows);
  return true;
}

// CG = 16-column blocks accumulated per pass (compile time, so accumulators
// stay in registers); passes repeat when the tile is wider.
template <typename T, int KBLK, int CG>
__global__ __launch_bounds__(kBlock) void segment_mm_kernel(
    const int32_t *__restrict__ tp, const T *__restrict__ X,
    const T *__restrict__ W, T *__restrict__ Y, MmGeom g) {
  typedef Mma<T, KBLK> MM;
  typedef typename MM::frag_t frag_t;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  T *tile = reinterpret_cast<T *>(lds_raw);
  int type, row0, row1;
  if (!locate_chunk(tp, g.n_types, g.chunk_rows, blockIdx.x, type, row0, row1)) return;
  MM::stage(W + (int64_t)type * g.w_type_stride, tile, g);
  __syncthreads();

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int lr = lane & 15;   // X row inside the tile (loads) / column (results)
  const int lk = lane >> 4;   // k slot (loads) / row quad (results)
  const int wsv = MM::ws(g.KB, g.MB);
  const int klane = MM::k_of_lane(lk);
  const int mb_pad = MM::mb_pad(g.MB);

  for (int tile0 = row0 + wave * kTileRows; tile0 < row1; tile0 += kTileBlock) {
    const T *xrow = X + (int64_t)(tile0 + lr) * g.ldx;
    const bool xlive = tile0 + lr < row1;
    for (int cg = 0; cg < mb_pad; cg += CG) {
      floatx4 acc[CG];
#pragma unroll
      for (int cb = 0; cb < CG; ++cb) acc[cb] = floatx4{0, 0, 0, 0};
      // k blocks that meet a non-zero part of these columns (heads on the
      // diagonal); everything when there is one head
      int kb_lo = 0, kb_hi = g.KB - 1;
      if (g.hb > 1) {
        const int c_lo = cg * 16, c_hi = min((cg + CG) * 16, g.Mt) - 1;
        kb_lo = ((c_lo / g.M) * g.K) / KBLK;
        kb_hi = min(((c_hi / g.M + 1) * g.K - 1) / KBLK, g.KB - 1);
      }
      for (int kc = kb_lo; kc <= kb_hi; kc += kMaxFrags) {
        frag_t xa[kMaxFrags];
#pragma unroll
        for (int f = 0; f < kMaxFrags; ++f) {
          const int k0 = (kc + f) * KBLK + klane;
          xa[f] = MM::zero();
          if (xlive && kc + f <= kb_hi && k0 < g.Kt) xa[f] = MM::load(xrow + k0);
        }
#pragma unroll
        for (int f = 0; f < kMaxFrags; ++f) {
          if (kc + f <= kb_hi) {
#pragma unroll
            for (int cb = 0; cb < CG; ++cb)
              if (cg + cb < mb_pad)
                acc[cb] = MM::mma(acc[cb], tile, wsv, kc + f, cg + cb, lr, lk, xa[f]);
          }
        }
      }
      // lane holds rows tile0 + 4*lk + r, column lr of every block
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = tile0 + lk * 4 + r;
        if (row < row1) {
          T *yrow = Y + (int64_t)row * g.ldy;
          if (MM::kPaired) {
#pragma unroll
            for (int cb = 0; cb < CG; cb += 2) {
              const int m = tile_col<true>(cg + cb, lr);   // even column
              if (m + 1 < g.Mt && (g.Mt & 1) == 0) {
                *reinterpret_cast<uint32_t *>(yrow + m) =
                    pack_bf16(acc[cb][r], acc[cb + 1 < CG ? cb + 1 : cb][r]);
              } else {
                if (m < g.Mt) yrow[m] = (T)f32_to_bf16_bits(acc[cb][r]);
                if (m + 1 < g.Mt && cb + 1 < CG)
                  yrow[m + 1] = (T)f32_to_bf16_bits(acc[cb + 1][r]);
              }
            }
          } else {
#pragma unroll
            for (int cb = 0; cb < CG; ++cb) {
              const int m = (cg + cb) * 16 + lr;
              if (m < g.Mt) yrow[m] = acc[cb][r];
            }
          }
        }
      }
    }
  }
}

// element loads / stores widened to fp32
template <typename T>
__device__ __forceinline__ float ldf(const T *p);
template <>
__device__ __forceinline__ float ldf<float>(const float *p) { return *p; }
template <>
__device__ __forceinline__ float ldf<bf16_t>(const bf16_t *p) { return bf16_lo(*p); }
__device__ __forceinline__ void stf(float *p, float v) { *p = v; }
__device__ __forceinline__ void stf(bf16_t *p, float v) { *p = (bf16_t)f32_to_bf16_bits(v); }

// ---- exact-shape kernel ------------------------------------------------------
// NF = k blocks and CG = 16-column blocks of the tile, both compile-time (the
// tile is zero padded up to them), so the LDS layout, every LDS / global offset
// and the accumulator set are static and the loop body is straight-line code:
// NF wide loads, NF*CG MFMAs, 4*CG coalesced stores.
template <typename T, int KBLK, int NF, int CG>
struct Tight;

template <int NF, int CG>
struct Tight<float, 16, NF, CG> {
  static constexpr int kWs = CG * 16 + 4;
  static constexpr int kTileElems = NF * 16 * kWs;
  static __device__ __forceinline__ floatx4 mma(floatx4 acc, const float *wl, int f,
                                                int cb, const float4 &x) {
    const float *w = wl + f * 16 * kWs + cb * 16;   // wl = tile + lk*4*kWs + lr
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(x.x, w[0], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(x.y, w[kWs], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(x.z, w[2 * kWs], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(x.w, w[3 * kWs], acc, 0, 0, 0);
    return acc;
  }
  static __device__ __forceinline__ const float *lane_base(const float *tile, int lr, int lk) {
    return tile + lk * 4 * kWs + lr;
  }
};

template <int NF, int CG>
struct Tight<bf16_t, 32, NF, CG> {
  static constexpr int kWs = NF * 32 + 8;
  static constexpr int kTileElems = CG * 16 * kWs;
  static __device__ __forceinline__ floatx4 mma(floatx4 acc, const bf16_t *wl, int f,
                                                int cb, const uint4 &x) {
    const uint4 w = *reinterpret_cast<const uint4 *>(wl + cb * 16 * kWs + f * 32);
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, x),
                                                   __builtin_bit_cast(bf16x8, w),
                                                   acc, 0, 0, 0);
  }
  static __device__ __forceinline__ const bf16_t *lane_base(const bf16_t *tile, int lr, int lk) {
    return tile + lr * kWs + lk * 8;   // wl = tile + lr*kWs + lk*8
  }
};

template <int NF, int CG>
struct Tight<bf16_t, 16, NF, CG> {
  static constexpr int kWs = NF * 16 + 8;
  static constexpr int kTileElems = CG * 16 * kWs;
  static __device__ __forceinline__ floatx4 mma(floatx4 acc, const bf16_t *wl, int f,
                                                int cb, const uint2 &x) {
    const uint2 w = *reinterpret_cast<const uint2 *>(wl + cb * 16 * kWs + f * 16);
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(shortx4, x),
                                                     __builtin_bit_cast(shortx4, w),
                                                     acc, 0, 0, 0);
  }
  static __device__ __forceinline__ const bf16_t *lane_base(const bf16_t *tile, int lr, int lk) {
    return tile + lr * kWs + lk * 4;
  }
};

// What happens to a finished tile.
constexpr int kEpiStore = 0;   // Y
constexpr int kEpiDot = 1;     // dot[r, h] = <Y[r, h, :], Q[q_index[r], h, :]> only
constexpr int kEpiAttn = 2;    // Y and el / er[r, h] = <Y[r, h, :], a_l / a_r[h, :]>

template <typename T, int KBLK, int NF, int CG, int EPI>
__global__ __launch_bounds__(kBlock) void segment_mm_tight_kernel(
    const int32_t *__restrict__ tp, const T *__restrict__ X,
    const T *__restrict__ W, T *__restrict__ Y, MmGeom g, MmExt e) {
  typedef Mma<T, KBLK> MM;
  typedef Tight<T, KBLK, NF, CG> TT;
  typedef typename MM::frag_t frag_t;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  T *tile = reinterpret_cast<T *>(lds_raw);
  int type, row0, row1;
  int chunk = blockIdx.x;
  if (g.n_pass > 1) {
    // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2:
    // the passes of one row chunk get ids 8 apart, so they run on the same XCD
    // at about the same time and the later ones find the chunk's rows in its L2.
    const int group = blockIdx.x / (8 * g.n_pass), within = blockIdx.x % (8 * g.n_pass);
    const int pass = within >> 3;
    chunk = group * 8 + (within & 7);
    const int col0 = pass * g.pass_cols;
    W += col0;
    Y += col0;
    e.a_l += col0;
    e.a_r += col0;
    e.el += col0 / g.dph;
    e.er += col0 / g.dph;
    g.M = g.Mt = min(g.pass_cols, g.m_total - col0);
    e.n_heads = g.Mt / g.dph;
  }
  if (!locate_chunk(tp, tp ? g.n_types : (int)g.rows, g.chunk_rows, chunk, type, row0, row1))
    return;
  MM::stage(W + (int64_t)type * g.w_type_stride, tile, g);   // g.KB == NF, g.MB == CG
  __syncthreads();

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int lr = lane & 15;
  const int lk = lane >> 4;
  const int klane = MM::k_of_lane(lk);
  const T *wl = TT::lane_base(tile, lr, lk);

  // k fragments of this lane that lie inside the row
  unsigned kmask = 0;
#pragma unroll
  for (int f = 0; f < NF; ++f)
    if (f * KBLK + klane < g.Kt) kmask |= 1u << f;
  const bool full_cols = g.Mt == CG * 16;
  const bool pack_ok = (g.Mt & 1) == 0 && (g.ldy & 1) == 0;

  // source row of X for tile row `row` (rows at or beyond row1 are never read)
  const int64_t *__restrict__ xi = e.x_index;
  auto src_row = [&](int row) -> int64_t {
    if (row >= row1) return 0;
    return xi ? xi[row] : (int64_t)row;
  };
  const int first = row0 + wave * kTileRows + lr;
  T *yp = Y + (int64_t)(row0 + wave * kTileRows + lk * 4) * g.ldy +
          (MM::kPaired ? 2 * lr : lr);
  const int64_t ystep = (int64_t)kTileBlock * g.ldy;

  // fragments of the next tile are requested before the current tile's MFMAs,
  // and the source row of the tile after that before those loads are needed
  frag_t xn[NF];
  {
    const T *xp = X + src_row(first) * g.ldx + klane;
    const bool xlive = first < row1;
#pragma unroll
    for (int f = 0; f < NF; ++f) {
      xn[f] = MM::zero();
      if (xlive && (kmask >> f & 1)) xn[f] = MM::load(xp + f * KBLK);
    }
  }
  int64_t inext = src_row(first + kTileBlock);
  // per-row factors of the stored rows (one per edge, in row order), also
  // requested one tile ahead
  const float *__restrict__ rsp = EPI == kEpiStore ? e.row_scale : nullptr;
  float rsn[4] = {1.0f, 1.0f, 1.0f, 1.0f};
  if (rsp) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = row0 + wave * kTileRows + lk * 4 + r;
      if (row < row1) rsn[r] = rsp[row];
    }
  }

  // dot operand: the values this lane needs from Q (4 rows x its column of every
  // block; a packed bf16 pair per block pair) are requested one tile ahead as
  // well, their row indices two tiles ahead
  constexpr bool DOT = EPI == kEpiDot;
  constexpr int NQ = DOT ? (MM::kPaired ? CG / 2 : CG) : 1;
  typedef typename std::conditional<MM::kPaired, uint32_t, float>::type qv_t;
  const T *__restrict__ Qb = static_cast<const T *>(e.Q);
  const int64_t *__restrict__ qix = e.q_index;
  auto q_row = [&](int row) -> int64_t {
    if (row >= row1) return 0;
    return qix ? qix[row] : (int64_t)row;
  };
  // The dot form stages W with its columns permuted (MmGeom::perm_shift): lane
  // column lr of block cb is tile column lr * CG + cb, so the CG values of Q that
  // meet this lane's accumulators are adjacent: one or two wide loads per row.
  auto load_q = [&](int64_t qr, bool live, qv_t (&dst)[NQ]) {
    const T *p = Qb + qr * e.ldq + lr * CG;
    const bool on = live && lr * CG < g.Mt;      // Mt is a multiple of CG
#pragma unroll
    for (int i = 0; i < NQ; ++i) dst[i] = 0;
    if (!on) return;
    if constexpr (DOT) {
      if constexpr (MM::kPaired) {
        if constexpr (CG == 8) {
          const uint4 v = *reinterpret_cast<const uint4 *>(p);
          dst[0] = v.x; dst[1] = v.y; dst[2] = v.z; dst[3] = v.w;
        } else if constexpr (CG == 4) {
          const uint2 v = *reinterpret_cast<const uint2 *>(p);
          dst[0] = v.x; dst[1] = v.y;
        } else {
          dst[0] = *reinterpret_cast<const uint32_t *>(p);
        }
      } else {
        if constexpr (CG >= 4) {
#pragma unroll
          for (int i = 0; i < CG; i += 4) {
            const float4 v = *reinterpret_cast<const float4 *>(p + i);
            dst[i] = v.x; dst[i + 1] = v.y; dst[i + 2] = v.z; dst[i + 3] = v.w;
          }
        } else if constexpr (CG == 2) {
          const float2 v = *reinterpret_cast<const float2 *>(p);
          dst[0] = v.x; dst[1] = v.y;
        } else {
          dst[0] = *p;
        }
      }
    }
  };
  // lanes per head, the head of this lane and its factor for this chunk's type
  // (read once: a load inside the tile loop would make every tile wait for the
  // prefetches issued before it)
  const int lph = DOT ? g.M / CG : 1;
  const int my_head = lr / lph;
  float my_scale = 1.0f;
  if (DOT && e.scale && my_head < g.hb) my_scale = e.scale[(int64_t)type * e.ldd + my_head];
  // attention vectors at this lane's column of every block (0 beyond the tile)
  float alv[CG], arv[CG];
#pragma unroll
  for (int cb = 0; cb < CG; ++cb) {
    alv[cb] = arv[cb] = 0.0f;
    if (EPI == kEpiAttn) {
      const int m = tile_col<MM::kPaired>(cb, lr);
      if (m < g.Mt) {
        alv[cb] = e.a_l[m];
        arv[cb] = e.a_r[m];
      }
    }
  }
  qv_t qn[4][NQ];
  int64_t qinext[4];
  if (DOT) {
    const int t0 = row0 + wave * kTileRows + lk * 4;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      load_q(q_row(t0 + r), t0 + r < row1, qn[r]);
      qinext[r] = q_row(t0 + kTileBlock + r);
    }
  }
  for (int tile0 = row0 + wave * kTileRows; tile0 < row1;
       tile0 += kTileBlock, yp += ystep) {
    // With many weight fragments the compiler would otherwise keep them all in
    // registers across tiles (one wave per SIMD); re-reading them from LDS per
    // tile is cheap, so forbid hoisting past this point.
    if (NF * CG * (int)(sizeof(frag_t) / 4) > 32) asm volatile("" ::: "memory");
    frag_t xa[NF];
#pragma unroll
    for (int f = 0; f < NF; ++f) xa[f] = xn[f];
    {
      const T *xp = X + inext * g.ldx + klane;
      const bool xlive = tile0 + kTileBlock + lr < row1;
#pragma unroll
      for (int f = 0; f < NF; ++f) {
        xn[f] = MM::zero();
        if (xlive && (kmask >> f & 1)) xn[f] = MM::load(xp + f * KBLK);
      }
    }
    inext = src_row(tile0 + 2 * kTileBlock + lr);
    float rsa[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) rsa[r] = rsn[r];
    if (rsp) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = tile0 + kTileBlock + lk * 4 + r;
        if (row < row1) rsn[r] = rsp[row];
      }
    }
    qv_t qa[4][NQ];
    if (DOT) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
#pragma unroll
        for (int i = 0; i < NQ; ++i) qa[r][i] = qn[r][i];
        const int nrow = tile0 + kTileBlock + lk * 4 + r;
        load_q(qinext[r], nrow < row1, qn[r]);
        qinext[r] = q_row(nrow + kTileBlock);
      }
    }
    floatx4 acc[CG];
#pragma unroll
    for (int cb = 0; cb < CG; ++cb) acc[cb] = floatx4{0, 0, 0, 0};
#pragma unroll
    for (int f = 0; f < NF; ++f) {
#pragma unroll
      for (int cb = 0; cb < CG; ++cb)
        acc[cb] = TT::mma(acc[cb], wl, f, cb, xa[f]);
    }
    // lane holds rows tile0 + 4*lk + r, lane column lr of every column block
    if (DOT) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = tile0 + lk * 4 + r;
        float v = 0.0f;
#pragma unroll
        for (int cb = 0; cb < CG; ++cb) {
          float qf;
          if constexpr (MM::kPaired)
            qf = (cb & 1) ? bf16_hi(qa[r][cb >> 1]) : bf16_lo(qa[r][cb >> 1]);
          else
            qf = qa[r][cb];
          v = fmaf(acc[cb][r], qf, v);
        }
        // sum over the lanes of the head (a power of two, at most the 16 of a row)
        if (lph >= 2) v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xF, 0xF, true));
        if (lph >= 4) v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xF, 0xF, true));
        if (lph >= 8) v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x141, 0xF, 0xF, true));
        if (lph >= 16) v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x140, 0xF, 0xF, true));
        if (row < row1 && (lr & (lph - 1)) == 0 && my_head < g.hb)
          e.dot[(int64_t)row * e.ldd + my_head] = v * my_scale;
      }
      continue;
    }
    if (EPI == kEpiAttn) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = tile0 + lk * 4 + r;
        const bool live = row < row1;
        float sl = 0.0f, sr = 0.0f;
        int head = 0;
        constexpr int step = MM::kPaired ? 2 : 1;
#pragma unroll
        for (int cb = 0; cb < CG; cb += step) {
#pragma unroll
          for (int i = 0; i < step; ++i) {
            sl = fmaf(acc[cb + i < CG ? cb + i : cb][r], alv[cb + i < CG ? cb + i : cb], sl);
            sr = fmaf(acc[cb + i < CG ? cb + i : cb][r], arv[cb + i < CG ? cb + i : cb], sr);
          }
          if (MM::kPaired && e.half_heads) {     // lanes 0-7: one head, 8-15: the next
            const float tl = row8_sum(sl), tr = row8_sum(sr);
            const int h = (cb >> 1) * 2 + (lr >> 3);
            if (live && (lr & 7) == 0 && h < (int)e.n_heads) {
              e.el[(int64_t)row * e.ldd + h] = tl;
              e.er[(int64_t)row * e.ldd + h] = tr;
            }
            sl = sr = 0.0f;
          } else if (e.head_end >> (cb + step - 1) & 1) {
            const float tl = row16_sum(sl), tr = row16_sum(sr);
            if (live && lr == 0 && head < e.n_heads) {   // blocks past the tile are padding
              e.el[(int64_t)row * e.ldd + head] = tl;
              e.er[(int64_t)row * e.ldd + head] = tr;
            }
            ++head;
            sl = sr = 0.0f;
          }
        }
      }
    }
    if (EPI == kEpiStore && rsp) {
#pragma unroll
      for (int cb = 0; cb < CG; ++cb)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[cb][r] *= rsa[r];
    }
    if (EPI == kEpiStore && g.perm_shift >= 0) {
      // permuted tile: this lane holds columns [lr * CG, (lr + 1) * CG) of its four
      // rows, so a row leaves as one vector store per lane (a whole 256-byte row
      // per 16 lanes at CG = 8 bf16 / CG = 4 fp32)
      if (lr * CG < g.Mt) {                        // Mt is a multiple of CG
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if (tile0 + lk * 4 + r >= row1) continue;
          T *yw = yp + (int64_t)r * g.ldy - (MM::kPaired ? 2 * lr : lr) + lr * CG;
          if constexpr (MM::kPaired) {
            uint32_t pk[CG / 2];
#pragma unroll
            for (int i = 0; i < CG / 2; ++i) pk[i] = pack_bf16(acc[2 * i][r], acc[2 * i + 1][r]);
            if constexpr (CG == 8)
              *reinterpret_cast<uint4 *>(yw) = make_uint4(pk[0], pk[1], pk[2], pk[3]);
            else if constexpr (CG == 4)
              *reinterpret_cast<uint2 *>(yw) = make_uint2(pk[0], pk[1]);
            else
              *reinterpret_cast<uint32_t *>(yw) = pk[0];
          } else {
            if constexpr (CG >= 4) {
#pragma unroll
              for (int i = 0; i < CG; i += 4)
                *reinterpret_cast<float4 *>(yw + i) =
                    make_float4(acc[i][r], acc[i + 1][r], acc[i + 2][r], acc[i + 3][r]);
            } else if constexpr (CG == 2) {
              *reinterpret_cast<float2 *>(yw) = make_float2(acc[0][r], acc[1][r]);
            } else {
              *yw = acc[0][r];
            }
          }
        }
      }
      continue;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      if (tile0 + lk * 4 + r < row1) {
        T *yrow = yp + (int64_t)r * g.ldy;
        if (MM::kPaired) {
#pragma unroll
          for (int cb = 0; cb < CG; cb += 2) {
            const int m = (cb >> 1) * 32 + 2 * lr;
            if (pack_ok && (full_cols || m + 1 < g.Mt)) {
              *reinterpret_cast<uint32_t *>(yrow + (cb >> 1) * 32) =
                  pack_bf16(acc[cb][r], acc[cb + 1][r]);
            } else {
              if (m < g.Mt) yrow[(cb >> 1) * 32] = (T)f32_to_bf16_bits(acc[cb][r]);
              if (m + 1 < g.Mt) yrow[(cb >> 1) * 32 + 1] = (T)f32_to_bf16_bits(acc[cb + 1][r]);
            }
          }
        } else {
#pragma unroll
          for (int cb = 0; cb < CG; ++cb)
            if (full_cols || cb * 16 + lr < g.Mt) yrow[cb * 16] = acc[cb][r];
        }
      }
    }
  }
}

// ---- any shape: one thread per output element ------------------------------
template <typename T>
__global__ __launch_bounds__(kBlock) void segment_mm_scalar_kernel(
    const int32_t *__restrict__ tp, int n_types, const T *__restrict__ X,
    const T *__restrict__ W, T *__restrict__ Y, int64_t rows, int heads, int K,
    int M) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= rows * heads * M) return;
  const int m = (int)(i % M);
  const int h = (int)((i / M) % heads);
  const int64_t r = i / ((int64_t)M * heads);
  if (r < tp[0] || r >= tp[n_types]) return;   // row outside every type
  int lo = 0, hi = n_types;                    // tp[lo] <= r < tp[hi]
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (tp[mid] <= r) lo = mid; else hi = mid;
  }
  const T *x = X + (r * heads + h) * K;
  const T *w = W + (((int64_t)lo * heads + h) * K) * M + m;
  float s = 0.0f;
  for (int k = 0; k < K; ++k) s = fmaf(ldf(x + k), ldf(w + (int64_t)k * M), s);
  stf(Y + i, s);
}

template <typename T, int KBLK, int CG>
int launch_cg(const int32_t *tp, const T *X, const T *W, T *Y, const MmGeom &g,
              int64_t grid, size_t lds, hipStream_t s) {
  // weight tiles above the default 64 KB (fp32 K = 256 x M = 64 and up) opt in to
  // the CU's full LDS
  if (!allow_lds((const void *)segment_mm_kernel<T, KBLK, CG>, lds)) return GA_EUNSUPPORTED;
  hipLaunchKernelGGL((segment_mm_kernel<T, KBLK, CG>), dim3((unsigned)grid),
                     dim3(kBlock), lds, s, tp, X, W, Y, g);
  return launch_status();
}

template <typename T, int KBLK, int NF, int CG, int EPI>
int launch_tight_as(const int32_t *tp, const T *X, const T *W, T *Y, MmGeom g,
                    const MmExt &e, int64_t grid, hipStream_t s) {
  typedef Tight<T, KBLK, NF, CG> TT;
  const size_t lds = (size_t)TT::kTileElems * sizeof(T);
  if (!allow_lds((const void *)segment_mm_tight_kernel<T, KBLK, NF, CG, EPI>, lds))
    return GA_EUNSUPPORTED;
  g.KB = NF;   // the tile is padded to the compile-time shape
  g.MB = CG;
  hipLaunchKernelGGL((segment_mm_tight_kernel<T, KBLK, NF, CG, EPI>),
                     dim3((unsigned)grid), dim3(kBlock), lds, s, tp, X, W, Y, g, e);
  return launch_status();
}

template <typename T, int KBLK, int NF, int CG>
int launch_tight(const int32_t *tp, const T *X, const T *W, T *Y, const MmGeom &g,
                 const MmExt &e, int64_t grid, hipStream_t s) {
  if (e.Q) return launch_tight_as<T, KBLK, NF, CG, kEpiDot>(tp, X, W, Y, g, e, grid, s);
  if (e.a_l) return launch_tight_as<T, KBLK, NF, CG, kEpiAttn>(tp, X, W, Y, g, e, grid, s);
  return launch_tight_as<T, KBLK, NF, CG, kEpiStore>(tp, X, W, Y, g, e, grid, s);
}

template <typename T, int KBLK, int NF>
int pick_tight_cg(int cg, const int32_t *tp, const T *X, const T *W, T *Y,
                  const MmGeom &g, const MmExt &e, int64_t grid, hipStream_t s) {
  switch (cg) {
    case 1: return launch_tight<T, KBLK, NF, Mma<T, KBLK>::kPaired ? 2 : 1>(tp, X, W, Y, g, e, grid, s);
    case 2: return launch_tight<T, KBLK, NF, 2>(tp, X, W, Y, g, e, grid, s);
    case 4: return launch_tight<T, KBLK, NF, 4>(tp, X, W, Y, g, e, grid, s);
    default: return launch_tight<T, KBLK, NF, 8>(tp, X, W, Y, g, e, grid, s);
  }
}

template <typename T, int KBLK>
int pick_tight(int nf, int cg, const int32_t *tp, const T *X, const T *W, T *Y,
               const MmGeom &g, const MmExt &e, int64_t grid, hipStream_t s) {
  switch (nf) {
    case 1: return pick_tight_cg<T, KBLK, 1>(cg, tp, X, W, Y, g, e, grid, s);
    case 2: return pick_tight_cg<T, KBLK, 2>(cg, tp, X, W, Y, g, e, grid, s);
    case 4: return pick_tight_cg<T, KBLK, 4>(cg, tp, X, W, Y, g, e, grid, s);
    default: return pick_tight_cg<T, KBLK, 8>(cg, tp, X, W, Y, g, e, grid, s);
  }
}

inline int pow2_ceil_int(int v) {
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}

int mm_cu_count() {
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

// One launch for `hb` folded heads starting at head h0.
template <typename T, int KBLK>
int launch_fold(const int32_t *tp, int n_types, const T *X, const T *W, T *Y,
                int64_t rows, int heads, int K, int M, int h0, int hb,
                const MmExt &ext, hipStream_t s) {
  typedef Mma<T, KBLK> MM;
  MmGeom g = {};
  g.n_types = n_types;
  g.K = K; g.M = M; g.hb = hb;
  g.Kt = hb * K; g.Mt = hb * M;
  g.KB = (g.Kt + KBLK - 1) / KBLK;
  g.MB = (g.Mt + 15) / 16;
  g.ldx = (int64_t)heads * K;
  g.ldy = (int64_t)heads * M;
  g.w_type_stride = (int64_t)heads * K * M;
  g.ldw = M;
  g.rows = rows;
  g.perm_shift = -1;
  // rows per workgroup: a multiple of the 64-row step, large enough to
  // amortise the weight staging, small enough to keep every CU busy
  // (the device holds three of these workgroups per CU at once: up to 16 steps, the
  // fewest with which the grid still fits one such round -- at 269 k rows 6 steps take
  // 30 us, 4 steps 38 and 12 steps 40)
  const int64_t slots = 3 * (int64_t)mm_cu_count() - n_types;
  int64_t steps = (rows + kTileBlock * (slots > 1 ? slots : 1) - 1) / (kTileBlock * (slots > 1 ? slots : 1));
  if (steps < 1) steps = 1;
  if (steps > 16) steps = 16;
  g.chunk_rows = (int)steps * kTileBlock;
  const int64_t grid = (rows + g.chunk_rows - 1) / g.chunk_rows + n_types;
  if (grid > 0x7fffffff) return GA_EUNSUPPORTED;
  const T *Xh = X + (int64_t)h0 * K;
  const T *Wh = W + (int64_t)h0 * K * M;
  T *Yh = Y ? Y + (int64_t)h0 * M : nullptr;
  const bool fused = ext.x_index || ext.Q;
  {
    if (g.KB <= 8 && g.MB <= 8) {
      MmExt e = ext;
      int cg = pow2_ceil_int(g.MB);        // column blocks of the tile as compiled
      if (Mma<T, KBLK>::kPaired && cg < 2) cg = 2;
      // stores: with the permuted tile (lane column j holds columns
      // [j * cg, (j + 1) * cg)) a lane writes its part of a row as one vector
      if (!e.Q && !e.a_l && g.Mt % cg == 0 && (g.ldy % cg) == 0 &&
          aligned(Yh, (size_t)cg * sizeof(T)))
        g.perm_shift = ilog2_floor((uint64_t)cg);
      if (e.Q) {
        // a head must cover a power-of-two number of lane columns
        const int lph = M / cg;
        if (M % cg != 0 || lph > 16 || (lph & (lph - 1)) != 0) return GA_EUNSUPPORTED;
        g.perm_shift = ilog2_floor((uint64_t)cg);
        e.Q = static_cast<const T *>(ext.Q) + (int64_t)h0 * M;
        e.dot = ext.dot + h0;
        if (e.scale) e.scale = ext.scale + h0;
      }
      const int rc = pick_tight<T, KBLK>(pow2_ceil_int(g.KB), pow2_ceil_int(g.MB), tp, Xh,
                                         Wh, Yh, g, e, grid, s);
      if (rc != GA_EUNSUPPORTED || fused) return rc;
    }
  }
  // only the exact-shape kernel gathers, and only it takes a row factor: a call that
  // carries one must not come back "done" from a kernel that ignores it
  if (fused || ext.row_scale) return GA_EUNSUPPORTED;
  const size_t lds = (size_t)MM::tile_elems(g.KB, g.MB) * sizeof(T);
  if (lds > (size_t)kMaxLdsOptIn) return GA_EUNSUPPORTED;
  const int mbp = MM::mb_pad(g.MB);
  if (MM::kPaired) {
    if (mbp <= 2) return launch_cg<T, KBLK, 2>(tp, Xh, Wh, Yh, g, grid, lds, s);
    if (mbp <= 4) return launch_cg<T, KBLK, 4>(tp, Xh, Wh, Yh, g, grid, lds, s);
    return launch_cg<T, KBLK, 8>(tp, Xh, Wh, Yh, g, grid, lds, s);
  }
  if (mbp <= 1) return launch_cg<T, KBLK, 1>(tp, Xh, Wh, Yh, g, grid, lds, s);
  if (mbp <= 2) return launch_cg<T, KBLK, 2>(tp, Xh, Wh, Yh, g, grid, lds, s);
  return launch_cg<T, KBLK, 4>(tp, Xh, Wh, Yh, g, grid, lds, s);
}

template <typename T, int KBLK>
int launch_mfma(const int32_t *tp, int n_types, const void *X, const void *W,
                void *Y, int64_t rows, int heads, int K, int M, const MmExt &ext,
                hipStream_t s) {
  // all heads folded into one block-diagonal tile when that fits the LDS and
  // the fragment budget; otherwise one launch per head
  if (heads > 1) {
    int rc = GA_EUNSUPPORTED;
    if ((int64_t)heads * K <= kMaxFrags * KBLK)
      rc = launch_fold<T, KBLK>(tp, n_types, (const T *)X, (const T *)W, (T *)Y,
                                rows, heads, K, M, 0, heads, ext, s);
    if (rc != GA_EUNSUPPORTED) return rc;
  }
  for (int h = 0; h < heads; ++h) {
    const int rc = launch_fold<T, KBLK>(tp, n_types, (const T *)X, (const T *)W,
                                        (T *)Y, rows, heads, K, M, h, 1, ext, s);
    // a fused form that does not fit fails on its first launch, before
    // anything was written
    if (rc != GA_OK) return rc;
  }
  return GA_OK;
}

}  // namespace
}  // namespace ga

namespace ga {
namespace {

// Wide bf16 outputs (whole groups of 128 columns, one head, few types): the kernel of
// wide_mm.hip reads X once for all of `n_w` weight tensors.  GA_EUNSUPPORTED: not its shape.
int wide_typed(const int32_t *type_pointer, int64_t n_types, const void *X,
               const void *const *W, void *const *Y, int n_w, int64_t rows, int64_t K,
               int64_t M, const float *row_scale, hipStream_t s, const float *type_gate = nullptr,
               bool gate_sigmoid = false) {
  if (M % kWideGroupCols != 0 || n_types > 64) return GA_EUNSUPPORTED;
  const int per_w = (int)(M / kWideGroupCols);
  if (!wide_mm_fits((int)K, n_w * per_w)) return GA_EUNSUPPORTED;
  WideMm p = {};
  p.tp = type_pointer;
  p.n_types = (int)n_types;
  p.rows = rows;
  p.X = (const bf16_t *)X;
  p.K = (int)K;
  p.n_groups = n_w * per_w;
  p.row_scale = row_scale;
  p.type_gate = type_gate;
  p.gate_sigmoid = gate_sigmoid;
  for (int w = 0; w < n_w; ++w)
    for (int c = 0; c < per_w; ++c) {
      const int g = w * per_w + c;
      p.W[g] = (const bf16_t *)W[w] + c * kWideGroupCols;
      p.w_type_stride[g] = K * M;
      p.ldw[g] = M;
      p.Y[g] = (bf16_t *)Y[w] + c * kWideGroupCols;
      p.ldy[g] = M;
    }
  return wide_mm_launch(p, s);
}

int segment_mm_any(const int32_t *type_pointer, int64_t n_types, const void *X,
                   const void *W, void *Y, int64_t rows, int64_t heads, int64_t K,
                   int64_t M, int dtype, const MmExt &ext, hipStream_t s) {
  const bool fused = ext.x_index || ext.Q;
  int rc = GA_EUNSUPPORTED;
  if (dtype == GA_BF16 && heads == 1 && !fused && Y) {
    rc = wide_typed(type_pointer, n_types, X, &W, &Y, 1, rows, K, M, ext.row_scale, s);
    if (rc != GA_EUNSUPPORTED) return rc;
  }
  if (aligned(X, 16) && (!Y || aligned(Y, 16)) && (!ext.Q || aligned(ext.Q, 16))) {
    if (dtype == GA_F32 && K % 4 == 0)
      rc = launch_mfma<float, 16>(type_pointer, (int)n_types, X, W, Y, rows,
                                  (int)heads, (int)K, (int)M, ext, s);
    else if (dtype == GA_BF16 && K % 8 == 0)
      rc = launch_mfma<bf16_t, 32>(type_pointer, (int)n_types, X, W, Y, rows,
                                   (int)heads, (int)K, (int)M, ext, s);
    else if (dtype == GA_BF16 && K % 4 == 0 && !fused)
      rc = launch_mfma<bf16_t, 16>(type_pointer, (int)n_types, X, W, Y, rows,
                                   (int)heads, (int)K, (int)M, ext, s);
  }
  // (the scalar kernel below takes no index column, dot operand or row factor)
  if (rc != GA_EUNSUPPORTED || fused || ext.row_scale) return rc;

  // shapes the MFMA path does not take (odd K, weights beyond the LDS budget)
  const int64_t total = rows * heads * M;
  const int64_t blocks = (total + kBlock - 1) / kBlock;
  if (blocks > 0x7fffffff) return GA_EUNSUPPORTED;
  if (dtype == GA_F32)
    hipLaunchKernelGGL((segment_mm_scalar_kernel<float>), dim3((unsigned)blocks),
                       dim3(kBlock), 0, s, type_pointer, (int)n_types,
                       (const float *)X, (const float *)W, (float *)Y, rows,
                       (int)heads, (int)K, (int)M);
  else
    hipLaunchKernelGGL((segment_mm_scalar_kernel<bf16_t>), dim3((unsigned)blocks),
                       dim3(kBlock), 0, s, type_pointer, (int)n_types,
                       (const bf16_t *)X, (const bf16_t *)W, (bf16_t *)Y, rows,
                       (int)heads, (int)K, (int)M);
  return launch_status();
}

int check_mm_args(int64_t n_types, int64_t rows, int64_t heads, int64_t K, int64_t M,
                  int dtype) {
  if (n_types < 0 || rows < 0 || heads <= 0 || K <= 0 || M <= 0) return GA_EINVAL;
  if (dtype != GA_F32 && dtype != GA_BF16) return GA_EINVAL;
  if (rows > 0x7fffffff || n_types > 0x7fffffff || heads * K > 0x7fffffff ||
      heads * M > 0x7fffffff)
    return GA_EINVAL;
  return GA_OK;
}

}  // namespace
}  // namespace ga

namespace ga {
namespace {

// Z = X @ W for one weight matrix plus el / er = <Z_h, a_l[h]>, <Z_h, a_r[h]>:
// the exact-shape kernel with a single type; output columns beyond 128 are
// covered by further column passes of the same launch (whole heads each).
template <typename T, int KBLK>
int launch_dense_attn(const T *X, const T *W, T *Z, const float *a_l, const float *a_r,
                      float *el, float *er, int64_t rows, int K, int M, int heads,
                      hipStream_t s) {
  typedef Mma<T, KBLK> MM;
  constexpr bool paired = MM::kPaired;
  const int dph = M / heads;
  if (dph > 128 || (K + KBLK - 1) / KBLK > 8) return GA_EUNSUPPORTED;
  const bool half = paired && dph == 16;
  if (!half && dph % (paired ? 32 : 16) != 0) return GA_EUNSUPPORTED;
  const int pass = (128 / dph) * dph;              // columns per pass: whole heads
  const int pw = M < pass ? M : pass;              // widest pass fixes the tile shape
  MmGeom g = {};
  g.n_types = 1;
  g.K = K; g.M = pw; g.hb = 1;
  g.Kt = K; g.Mt = pw;
  g.KB = (K + KBLK - 1) / KBLK;
  g.MB = (pw + 15) / 16;
  g.ldx = K;
  g.ldy = M;
  g.w_type_stride = 0;
  g.ldw = M;
  g.rows = rows;
  g.n_pass = (M + pass - 1) / pass;
  g.pass_cols = pass;
  g.m_total = M;
  g.dph = dph;
  g.perm_shift = -1;
  int64_t steps = rows / (kTileBlock * 2048);
  if (steps < 1) steps = 1;
  if (steps > 16) steps = 16;
  g.chunk_rows = (int)steps * kTileBlock;
  const int64_t chunks = (rows + g.chunk_rows - 1) / g.chunk_rows;
  // with several passes the chunk count is padded to a multiple of 8 (surplus
  // workgroups return at once)
  const int64_t grid = g.n_pass > 1 ? (chunks + 7) / 8 * 8 * g.n_pass : chunks;
  if (grid > 0x7fffffff) return GA_EUNSUPPORTED;
  MmExt e = {};
  e.a_l = a_l;
  e.a_r = a_r;
  e.el = el;
  e.er = er;
  e.ldd = heads;
  e.n_heads = pw / dph;
  e.half_heads = half;
  for (int b = 0; b < 32; ++b) {
    const int end_col = paired ? ((b >> 1) + 1) * 32 : (b + 1) * 16;
    if ((!paired || (b & 1)) && end_col % dph == 0) e.head_end |= 1u << b;
  }
  return pick_tight<T, KBLK>(pow2_ceil_int(g.KB), pow2_ceil_int(g.MB), nullptr, X, W, Z, g, e,
                             grid, s);
}

}  // namespace
}  // namespace ga

extern "C" int ga_project_attn(const void *X, const void *W, const float *a_l,
                               const float *a_r, void *Z, float *el, float *er,
                               int64_t rows, int64_t K, int64_t M, int64_t heads,
                               int dtype, ga_stream_t stream) {
  using namespace ga;
  if (rows < 0 || K <= 0 || M <= 0 || heads <= 0 || M % heads) return GA_EINVAL;
  if (dtype != GA_F32 && dtype != GA_BF16) return GA_EINVAL;
  if (rows > 0x7fffffff || K > 0x7fffffff || M > 0x7fffffff) return GA_EINVAL;
  if (rows == 0) return GA_OK;
  if (!X || !W || !a_l || !a_r || !Z || !el || !er) return GA_EINVAL;
  const size_t esz = dtype == GA_F32 ? 4 : 2;
  if (!aligned(X, esz) || !aligned(W, esz) || !aligned(Z, esz) || !aligned(a_l, 4) ||
      !aligned(a_r, 4) || !aligned(el, 4) || !aligned(er, 4))
    return GA_EALIGN;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == GA_F32) {
    const int rc = ga_linear_attn((const float *)X, (const float *)W, a_l, a_r, (float *)Z,
                                  el, er, rows, K, M, heads, stream);
    if (rc != GA_EUNSUPPORTED) return rc;
    if (aligned(X, 16) && aligned(Z, 16) && K % 4 == 0)
      return launch_dense_attn<float, 16>((const float *)X, (const float *)W, (float *)Z, a_l,
                                          a_r, el, er, rows, (int)K, (int)M, (int)heads, s);
    return GA_EUNSUPPORTED;
  }
  if ((M & 1) || !aligned(Z, 4)) return GA_EUNSUPPORTED;      // packed bf16 pair stores
  {
    // whole groups of 128 columns holding whole heads: one pass over X for all of them
    const int64_t dph = M / heads;
    if (M % kWideGroupCols == 0 && (dph == 32 || dph == 64 || dph == 128) &&
        wide_mm_fits((int)K, (int)(M / kWideGroupCols))) {
      WideMm p = {};
      p.n_types = 1;
      p.rows = rows;
      p.X = (const bf16_t *)X;
      p.K = (int)K;
      p.n_groups = (int)(M / kWideGroupCols);
      p.ldd = heads;
      p.dph = (int)dph;
      for (int g = 0; g < p.n_groups; ++g) {
        p.W[g] = (const bf16_t *)W + g * kWideGroupCols;
        p.ldw[g] = M;
        p.Y[g] = (bf16_t *)Z + g * kWideGroupCols;
        p.ldy[g] = M;
        p.a_l[g] = a_l + g * kWideGroupCols;
        p.a_r[g] = a_r + g * kWideGroupCols;
        p.el[g] = el + g * (kWideGroupCols / dph);
        p.er[g] = er + g * (kWideGroupCols / dph);
      }
      const int rc = wide_mm_launch(p, s);
      if (rc != GA_EUNSUPPORTED) return rc;
    }
  }
  if (aligned(X, 16) && K % 8 == 0)
    return launch_dense_attn<bf16_t, 32>((const bf16_t *)X, (const bf16_t *)W, (bf16_t *)Z,
                                         a_l, a_r, el, er, rows, (int)K, (int)M, (int)heads, s);
  if (aligned(X, 8) && K % 4 == 0)
    return launch_dense_attn<bf16_t, 16>((const bf16_t *)X, (const bf16_t *)W, (bf16_t *)Z,
                                         a_l, a_r, el, er, rows, (int)K, (int)M, (int)heads, s);
  return GA_EUNSUPPORTED;
}

namespace ga {
namespace {
// out[b][j][i] = W[b][i][j] * scale[b] * factor over square blocks of D x D values
template <typename T, typename S>
__global__ __launch_bounds__(kBlock) void transpose_scale_blocks_kernel(
    const T *__restrict__ W, const S *__restrict__ scale, float factor, T *__restrict__ out,
    int D, int64_t total) {
  const int64_t o = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (o >= total) return;
  const int i = (int)(o % D), j = (int)(o / D % D);
  const int64_t b = o / ((int64_t)D * D);
  const float v = elem_to_f32(W[(b * D + i) * D + j]) * (scale ? elem_to_f32(scale[b]) : 1.0f) * factor;
  f32_to_elem(v, out[o]);
}
}  // namespace
}  // namespace ga

extern "C" int ga_transpose_scale_blocks_as(const void *W, const void *scale, int scale_dtype,
                                            float factor, void *out, int64_t n_blocks, int64_t D,
                                            int dtype, ga_stream_t stream) {
  using namespace ga;
  if (n_blocks < 0 || D <= 0 || D > 0x7fff) return GA_EINVAL;
  if (dtype != GA_F32 && dtype != GA_BF16) return GA_EINVAL;
  if (scale_dtype != GA_F32 && scale_dtype != GA_BF16) return GA_EINVAL;
  const int64_t total = n_blocks * D * D;
  if (total == 0) return GA_OK;
  if (!W || !out || W == out) return GA_EINVAL;
  const size_t esz = dtype == GA_F32 ? 4 : 2;
  if (!aligned(W, esz) || !aligned(out, esz) || (scale && !aligned(scale, scale_dtype == GA_F32 ? 4 : 2)))
    return GA_EALIGN;
  const int64_t blocks = (total + kBlock - 1) / kBlock;
  if (blocks > 0x7fffffff) return GA_EUNSUPPORTED;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)blocks), block(kBlock);
  if (dtype == GA_F32 && scale_dtype == GA_F32)
    hipLaunchKernelGGL((transpose_scale_blocks_kernel<float, float>), grid, block, 0, s, (const float *)W,
                       (const float *)scale, factor, (float *)out, (int)D, total);
  else if (dtype == GA_F32)
    hipLaunchKernelGGL((transpose_scale_blocks_kernel<float, bf16_t>), grid, block, 0, s, (const float *)W,
                       (const bf16_t *)scale, factor, (float *)out, (int)D, total);
  else if (scale_dtype == GA_F32)
    hipLaunchKernelGGL((transpose_scale_blocks_kernel<bf16_t, float>), grid, block, 0, s, (const bf16_t *)W,
                       (const float *)scale, factor, (bf16_t *)out, (int)D, total);
  else
    hipLaunchKernelGGL((transpose_scale_blocks_kernel<bf16_t, bf16_t>), grid, block, 0, s, (const bf16_t *)W,
                       (const bf16_t *)scale, factor, (bf16_t *)out, (int)D, total);
  return launch_status();
}

extern "C" int ga_transpose_scale_blocks(const void *W, const float *scale, float factor,
                                         void *out, int64_t n_blocks, int64_t D, int dtype,
                                         ga_stream_t stream) {
  return ga_transpose_scale_blocks_as(W, scale, GA_F32, factor, out, n_blocks, D, dtype, stream);
}

extern "C" int ga_segment_mm(const int32_t *type_pointer, int64_t n_types,
                             const void *X, const void *W, void *Y, int64_t rows,
                             int64_t heads, int64_t K, int64_t M, int dtype,
                             ga_stream_t stream) {
  using namespace ga;
  const int bad = check_mm_args(n_types, rows, heads, K, M, dtype);
  if (bad != GA_OK) return bad;
  if (rows == 0 || n_types == 0) return GA_OK;
  if (!type_pointer || !X || !W || !Y) return GA_EINVAL;
  const size_t esz = dtype == GA_F32 ? 4 : 2;
  if (!aligned(X, esz) || !aligned(W, esz) || !aligned(Y, esz)) return GA_EALIGN;
  MmExt ext = {};
  return segment_mm_any(type_pointer, n_types, X, W, Y, rows, heads, K, M, dtype, ext,
                        (hipStream_t)stream);
}

extern "C" int ga_segment_mm_stacked(const int32_t *type_pointer, int64_t n_types,
                                     const void *X, const void *const *W, void *const *Y,
                                     int64_t n_weights, int64_t rows, int64_t K, int64_t M,
                                     int dtype, ga_stream_t stream) {
  using namespace ga;
  if (n_weights < 1 || n_weights > 4 || !W || !Y) return GA_EINVAL;
  const int bad = check_mm_args(n_types, rows, 1, K, M, dtype);
  if (bad != GA_OK) return bad;
  if (rows == 0 || n_types == 0) return GA_OK;
  if (!type_pointer || !X) return GA_EINVAL;
  const size_t esz = dtype == GA_F32 ? 4 : 2;
  if (!aligned(X, esz)) return GA_EALIGN;
  for (int64_t i = 0; i < n_weights; ++i) {
    if (!W[i] || !Y[i]) return GA_EINVAL;
    if (!aligned(W[i], esz) || !aligned(Y[i], esz)) return GA_EALIGN;
  }
  hipStream_t s = (hipStream_t)stream;
  if (dtype == GA_BF16) {
    const int rc = wide_typed(type_pointer, n_types, X, W, Y, (int)n_weights, rows, K, M, nullptr, s);
    if (rc != GA_EUNSUPPORTED) return rc;
  }
  // any other shape: one product per weight tensor
  MmExt ext = {};
  for (int64_t i = 0; i < n_weights; ++i) {
    const int rc = segment_mm_any(type_pointer, n_types, X, W[i], Y[i], rows, 1, K, M, dtype, ext, s);
    if (rc != GA_OK) return rc;
  }
  return GA_OK;
}

extern "C" int ga_segment_mm_gated(const int32_t *type_pointer, int64_t n_types, const void *X,
                                   const void *W, void *Y, const float *gate, int gate_sigmoid,
                                   int64_t rows, int64_t K, int64_t M, int dtype,
                                   ga_stream_t stream) {
  using namespace ga;
  const int bad = check_mm_args(n_types, rows, 1, K, M, dtype);
  if (bad != GA_OK) return bad;
  if (rows == 0 || n_types == 0) return GA_OK;
  if (!type_pointer || !X || !W || !Y || !gate) return GA_EINVAL;
  const size_t esz = dtype == GA_F32 ? 4 : 2;
  if (!aligned(X, esz) || !aligned(W, esz) || !aligned(Y, esz) || !aligned(gate, 4)) return GA_EALIGN;
  if (dtype != GA_BF16) return GA_EUNSUPPORTED;
  return wide_typed(type_pointer, n_types, X, &W, &Y, 1, rows, K, M, nullptr, (hipStream_t)stream,
                    gate, gate_sigmoid != 0);
}

extern "C" int ga_segment_mm_gather(const int32_t *type_pointer, int64_t n_types,
                                    const void *X, const int64_t *x_index,
                                    const void *W, void *Y, const void *Q,
                                    const int64_t *q_index, const float *scale,
                                    float *dot, const float *row_scale, int64_t rows,
                                    int64_t heads, int64_t K, int64_t M, int dtype,
                                    ga_stream_t stream) {
  using namespace ga;
  const int bad = check_mm_args(n_types, rows, heads, K, M, dtype);
  if (bad != GA_OK) return bad;
  if (rows == 0 || n_types == 0) return GA_OK;   // empty results may have no address
  if ((Y != nullptr) == (dot != nullptr)) return GA_EINVAL;   // exactly one result
  if ((Q != nullptr) != (dot != nullptr)) return GA_EINVAL;
  if ((q_index || scale) && !Q) return GA_EINVAL;
  if (row_scale && !Y) return GA_EINVAL;
  if (!type_pointer || !X || !W) return GA_EINVAL;
  const size_t esz = dtype == GA_F32 ? 4 : 2;
  if (!aligned(X, esz) || !aligned(W, esz) || (Y && !aligned(Y, esz)) ||
      (Q && !aligned(Q, esz)) || (dot && !aligned(dot, 4)) ||
      (scale && !aligned(scale, 4)) || (row_scale && !aligned(row_scale, 4)) ||
      (x_index && !aligned(x_index, 8)) || (q_index && !aligned(q_index, 8)))
    return GA_EALIGN;
  MmExt ext = {};
  ext.x_index = x_index;
  ext.Q = Q;
  ext.q_index = q_index;
  ext.dot = dot;
  ext.scale = scale;
  ext.row_scale = row_scale;
  ext.ldq = heads * M;
  ext.ldd = heads;
  return segment_mm_any(type_pointer, n_types, X, W, Y, rows, heads, K, M, dtype, ext,
                        (hipStream_t)stream);
}
