// Typed GEMM for wide bf16 outputs on gfx950: Y_g[r, :] = X[r, :] @ W_g[type(r)] for up
// to four groups of 128 output columns, rows sorted by type, fp32 accumulation.
//
// The shapes it serves -- the K | Q | V projections of an HGT layer (three (T, 128, 128)
// weights applied to the same rows, examples/HGT/HGT.py:35-44 through
// segment_mm.cu:4-33) and the 256-wide projections of a GAT layer -- stream far more
// bytes of X and Y than the matrix cores need time for, so the kernel is built around
// reading X once and writing Y in whole cache lines:
//
//   * a workgroup (8 wavefronts) owns a long chunk of consecutive rows of one type
//     (about rows / #CUs of them) and keeps the weights of ALL groups for that type in
//     LDS, transposed to [column][k] (up to 136 KB: one workgroup per CU);
//   * a wavefront takes 32 rows per step (two 16-row tiles; one tile at K = 256, where
//     two would not fit the registers): the rows' k fragments are read once (16-byte
//     loads straight into the A-operand layout), one step ahead of their use, and
//     multiplied against every group in turn; every weight fragment read from LDS feeds
//     one v_mfma_f32_16x16x32_bf16 per tile;
//   * inside a group the 8 column blocks interleave their columns (block j, lane n =
//     column 8 n + j), so a lane ends up with 8 adjacent outputs of a row and a row of a
//     group leaves as 16 lanes x 16 bytes = one 256-byte line;
//   * optionally the GAT attention terms el / er[r, head] = <Y[r, head, :], a[head, :]>
//     are taken from the fp32 accumulators (8 products per lane, then a DPP sum over
//     the lanes of the head), so Y is not read again for them.
#include "wide_mm.h"

namespace ga {
namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kWideBlock = 512;         // 8 wavefronts: two per SIMD when one workgroup fills a CU
constexpr int kWideMaxLds = 158 * 1024;

// two fp32 -> packed bf16 in one instruction (v_cvt_pk_bf16_f32: round to nearest even,
// the same values as f32_to_bf16_bits)
__device__ __forceinline__ uint32_t cvt_pk_bf16(float lo, float hi) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, bf16x2));
}

__host__ __device__ constexpr int wide_ws(int nf) { return nf * 32 + 8; }   // LDS row stride
__host__ __device__ constexpr int wide_group_elems(int nf) { return kWideGroupCols * wide_ws(nf); }

// Which chunk of which type does this workgroup own?  chunks(t) = ceil(rows_t /
// chunk_rows); workgroup id -> (type, first row, end row); false: none.
__device__ __forceinline__ bool wide_locate(const int32_t *__restrict__ tp, int n_types,
                                            int64_t rows, int chunk_rows, int target, int &type,
                                            int &row0, int &row1) {
  if (!tp) {
    type = 0;
    if ((int64_t)target * chunk_rows >= rows) return false;
    row0 = target * chunk_rows;
    row1 = (int)min(rows, (int64_t)row0 + chunk_rows);
    return true;
  }
  // few types, every lane walks them (uniform scalar loads)
  int base = 0;
  for (int t = 0; t < n_types; ++t) {
    const int p0 = tp[t], p1 = tp[t + 1];
    const int cnt = (p1 - p0 + chunk_rows - 1) / chunk_rows;
    if (target < base + cnt) {
      type = t;
      row0 = p0 + (target - base) * chunk_rows;
      row1 = min(p1, row0 + chunk_rows);
      return true;
    }
    base += cnt;
  }
  return false;
}

// One group's (K x 128) weights into LDS as [column][k].  A thread takes 8 rows of k x 8
// adjacent columns: eight 16-byte loads (16 threads cover a 256-byte row of the group),
// an 8 x 8 transpose in registers, eight 16-byte LDS writes (one per column).  All loads
// of a thread are in flight together: staging costs about one memory latency.
// LDS row (c & 7) * 16 + (c >> 3) holds column c.
template <int NF>
__device__ __forceinline__ void wide_stage(const bf16_t *__restrict__ w, int64_t ldw, int K,
                                           bf16_t *tile, bool wide_ok) {
  constexpr int kTasks = NF * 4 * 16;              // k octets x column octets
  for (int task = threadIdx.x; task < kTasks; task += kWideBlock) {
    const int m8 = task & 15, kc = (task >> 4) * 8;
    uint4 r[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const bf16_t *src = w + (int64_t)(kc + j) * ldw + 8 * m8;
      if (kc + j >= K) {
        r[j] = make_uint4(0, 0, 0, 0);
      } else if (wide_ok) {
        r[j] = *reinterpret_cast<const uint4 *>(src);
      } else {                                     // rows that are not 16-byte aligned
        r[j] = make_uint4(src[0] | ((uint32_t)src[1] << 16), src[2] | ((uint32_t)src[3] << 16),
                          src[4] | ((uint32_t)src[5] << 16), src[6] | ((uint32_t)src[7] << 16));
      }
    }
    // word i of r[j] holds columns 2 i (low half) and 2 i + 1 (high half) of row kc + j
    constexpr uint32_t kLow = 0x05040100u, kHigh = 0x07060302u;   // halves of (S1, S0)
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      const uint32_t sel = (c & 1) ? kHigh : kLow;
      auto word = [&](const uint4 &v) { return c < 2 ? v.x : c < 4 ? v.y : c < 6 ? v.z : v.w; };
      const uint4 o = make_uint4(__builtin_amdgcn_perm(word(r[1]), word(r[0]), sel),
                                 __builtin_amdgcn_perm(word(r[3]), word(r[2]), sel),
                                 __builtin_amdgcn_perm(word(r[5]), word(r[4]), sel),
                                 __builtin_amdgcn_perm(word(r[7]), word(r[6]), sel));
      // column 8 m8 + c lives in LDS row c * 16 + m8
      *reinterpret_cast<uint4 *>(tile + (c * 16 + m8) * wide_ws(NF) + kc) = o;
    }
  }
}

template <int NF, int NG, bool ATTN, int TW, bool X8>
__global__ __launch_bounds__(kWideBlock) void wide_mm_kernel(WideMm p, int chunk_rows) {
  constexpr int kWaveRows = 16 * TW;                       // rows of a wavefront per step
  constexpr int kStepRows = (kWideBlock / kWave) * kWaveRows;
  extern __shared__ __attribute__((aligned(16))) unsigned char wide_lds[];
  bf16_t *tile = reinterpret_cast<bf16_t *>(wide_lds);
  constexpr int kWs = wide_ws(NF);
  int type, row0, row1;
  if (!wide_locate(p.tp, p.n_types, p.rows, chunk_rows, blockIdx.x, type, row0, row1)) return;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int n = lane & 15, q = lane >> 4;
  // factor of every row of this workgroup's type (HGT's sigmoid(skip[type]) gate)
  float gate = 1.0f;
  if (!ATTN && p.type_gate) {
    const float v = p.type_gate[type];
    gate = p.gate_sigmoid ? 1.0f / (1.0f + __expf(-v)) : v;
  }

  // halves (4 elements) of this lane's k fragments that lie inside a row: bits 2 f, 2 f + 1
  unsigned kmask = 0;
#pragma unroll
  for (int f = 0; f < NF; ++f) {
    if (f * 32 + q * 8 < p.K) kmask |= 1u << (2 * f);
    if (f * 32 + q * 8 + 4 < p.K) kmask |= 2u << (2 * f);
  }
  // Addresses inside the chunk are "uniform base + 32-bit lane offset" (the host keeps a
  // chunk below 4 GiB of X and of every Y): no 64-bit arithmetic per access.
  const char *xbase = reinterpret_cast<const char *>(p.X + (int64_t)row0 * p.K);
  const uint32_t xrow = (uint32_t)p.K * 2u;
  const int nrows = row1 - row0;
  auto load_rows = [&](int rel, uint4 (&x)[TW][NF]) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < TW; ++t) {
      const int r = rel + 16 * t + n;
      const uint32_t off = (uint32_t)(r < nrows ? r : nrows - 1) * xrow + (uint32_t)q * 16u;
#pragma unroll
      for (int f = 0; f < NF; ++f) {
        if (X8) {       // rows 8-byte aligned only (K % 8 == 4): two loads per fragment
          const uint2 lo = (kmask >> (2 * f) & 1) ? *reinterpret_cast<const uint2 *>(xbase + off + f * 64)
                                                  : make_uint2(0, 0);
          const uint2 hi = (kmask >> (2 * f) & 2) ? *reinterpret_cast<const uint2 *>(xbase + off + f * 64 + 8)
                                                  : make_uint2(0, 0);
          x[t][f] = make_uint4(lo.x, lo.y, hi.x, hi.y);
        } else {
          x[t][f] = (kmask >> (2 * f) & 1) ? *reinterpret_cast<const uint4 *>(xbase + off + f * 64)
                                           : make_uint4(0, 0, 0, 0);
        }
      }
    }
  };
  // the rows of the first step are on their way while the weights are staged
  uint4 xn[TW][NF];
  load_rows(wave * kWaveRows, xn);
#pragma unroll
  for (int g = 0; g < NG; ++g)
    wide_stage<NF>(p.W[g] + (int64_t)type * p.w_type_stride[g], p.ldw[g], p.K,
                   tile + g * wide_group_elems(NF), p.w_wide);
  __syncthreads();

  const bf16_t *wl = tile + n * kWs + q * 8;      // my fragment of LDS row 0
  for (int rel = wave * kWaveRows; rel < nrows; rel += kStepRows) {
    uint4 xa[TW][NF];
#pragma unroll
    for (int t = 0; t < TW; ++t)
#pragma unroll
      for (int f = 0; f < NF; ++f) xa[t][f] = xn[t][f];
    if (rel + kStepRows < nrows) load_rows(rel + kStepRows, xn);
    const bool full = rel + kWaveRows <= nrows;
    // factors of my rows rel + 16 t + 4 q + i (requested now, used after the products)
    float rs[TW][4];
#pragma unroll
    for (int t = 0; t < TW; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int r = rel + 16 * t + 4 * q + i;
        rs[t][i] = !ATTN && p.row_scale ? gate * p.row_scale[row0 + (r < nrows ? r : nrows - 1)] : gate;
      }
#pragma unroll 1
    for (int g = 0; g < NG; ++g) {
      // The weight fragments do not change from step to step, and the compiler would
      // keep them all in registers (there are up to 1024 of them): they are cheap to read
      // again from LDS, so nothing may be carried over this point.
      asm volatile("" ::: "memory");
      floatx4 acc[TW][8];
#pragma unroll
      for (int t = 0; t < TW; ++t)
#pragma unroll
        for (int cb = 0; cb < 8; ++cb) acc[t][cb] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int f = 0; f < NF; ++f) {
#pragma unroll
        for (int cb = 0; cb < 8; ++cb) {
          const bf16x8 w = __builtin_bit_cast(
              bf16x8, *reinterpret_cast<const uint4 *>(wl + g * wide_group_elems(NF) +
                                                       cb * 16 * kWs + f * 32));
#pragma unroll
          for (int t = 0; t < TW; ++t)
            acc[t][cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                __builtin_bit_cast(bf16x8, xa[t][f]), w, acc[t][cb], 0, 0, 0);
        }
      }
      // lane (n, q) holds rows rel + 16 t + 4 q + i, columns 8 n .. 8 n + 7 of the group
      if (!ATTN && (p.row_scale || p.type_gate)) {
#pragma unroll
        for (int t = 0; t < TW; ++t)
#pragma unroll
          for (int cb = 0; cb < 8; ++cb)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[t][cb][i] *= rs[t][i];
      }
      char *ybase = reinterpret_cast<char *>(p.Y[g] + (int64_t)row0 * p.ldy[g]);
      const uint32_t yrow = (uint32_t)p.ldy[g] * 2u;
      const uint32_t yoff = (uint32_t)(rel + 4 * q) * yrow + (uint32_t)n * 16u;
#pragma unroll
      for (int t = 0; t < TW; ++t) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (full || rel + 16 * t + 4 * q + i < nrows)
            *reinterpret_cast<uint4 *>(ybase + yoff + (uint32_t)(16 * t + i) * yrow) =
                make_uint4(cvt_pk_bf16(acc[t][0][i], acc[t][1][i]), cvt_pk_bf16(acc[t][2][i], acc[t][3][i]),
                           cvt_pk_bf16(acc[t][4][i], acc[t][5][i]), cvt_pk_bf16(acc[t][6][i], acc[t][7][i]));
        }
      }
      if (ATTN) {
        float al[8], ar[8];
        {
          const float4 a0 = *reinterpret_cast<const float4 *>(p.a_l[g] + 8 * n);
          const float4 a1 = *reinterpret_cast<const float4 *>(p.a_l[g] + 8 * n + 4);
          const float4 b0 = *reinterpret_cast<const float4 *>(p.a_r[g] + 8 * n);
          const float4 b1 = *reinterpret_cast<const float4 *>(p.a_r[g] + 8 * n + 4);
          al[0] = a0.x; al[1] = a0.y; al[2] = a0.z; al[3] = a0.w;
          al[4] = a1.x; al[5] = a1.y; al[6] = a1.z; al[7] = a1.w;
          ar[0] = b0.x; ar[1] = b0.y; ar[2] = b0.z; ar[3] = b0.w;
          ar[4] = b1.x; ar[5] = b1.y; ar[6] = b1.z; ar[7] = b1.w;
        }
        const int lph = p.dph >> 3;               // lanes of a head: 4, 8 or 16
#pragma unroll
        for (int t = 0; t < TW; ++t) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float sl = 0.0f, sr = 0.0f;
#pragma unroll
            for (int cb = 0; cb < 8; ++cb) {
              sl = fmaf(acc[t][cb][i], al[cb], sl);
              sr = fmaf(acc[t][cb][i], ar[cb], sr);
            }
            // quads first, then the half row and the row when a head has that many lanes
            sl += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(sl), 0xB1, 0xF, 0xF, true));
            sr += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(sr), 0xB1, 0xF, 0xF, true));
            sl += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(sl), 0x4E, 0xF, 0xF, true));
            sr += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(sr), 0x4E, 0xF, 0xF, true));
            if (lph >= 8) {
              sl += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(sl), 0x141, 0xF, 0xF, true));
              sr += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(sr), 0x141, 0xF, 0xF, true));
            }
            if (lph >= 16) {
              sl += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(sl), 0x140, 0xF, 0xF, true));
              sr += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(sr), 0x140, 0xF, 0xF, true));
            }
            const int r = rel + 16 * t + 4 * q + i;
            if ((n & (lph - 1)) == 0 && r < nrows) {
              p.el[g][(int64_t)(row0 + r) * p.ldd + n / lph] = sl;
              p.er[g][(int64_t)(row0 + r) * p.ldd + n / lph] = sr;
            }
          }
        }
      }
    }
  }
}

int wide_cu_count() {
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

template <int NF, int NG, bool ATTN, bool X8>
int wide_launch_x(const WideMm &p, hipStream_t s) {
  const size_t lds = (size_t)NG * wide_group_elems(NF) * sizeof(bf16_t);
  if (lds > (size_t)kWideMaxLds) return GA_EUNSUPPORTED;
  // two row tiles per wavefront where the registers allow it: every weight fragment read
  // from LDS then feeds two matrix instructions
  constexpr int TW = NF <= 4 ? 2 : 1;
  constexpr int kStepRows = (kWideBlock / kWave) * 16 * TW;
  const void *kernel = (const void *)wide_mm_kernel<NF, NG, ATTN, TW, X8>;
  if (lds > 64 * 1024) {
    static bool granted = false;       // per instantiation
    if (!granted) {
      if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) !=
          hipSuccess)
        return GA_EUNSUPPORTED;
      granted = true;
    }
  }
  // One round of workgroups: as many as fit the chip at once (LDS decides how many per
  // CU), each with a chunk of whole steps.  ceil(rows / chunk) + n_types bounds the
  // chunks of all types; workgroups beyond the real count return at once.
  int per_cu = (int)((size_t)(160 * 1024) / lds);
  if (per_cu < 1) per_cu = 1;
  if (per_cu > 2) per_cu = 2;          // longer chunks rather than more weight staging
  int64_t target = (int64_t)wide_cu_count() * per_cu - (p.tp ? p.n_types : 0);
  if (target < 1) target = 1;
  int64_t chunk = (p.rows + target - 1) / target;
  chunk = (chunk + kStepRows - 1) / kStepRows * kStepRows;
  int64_t widest = p.K;
  for (int g = 0; g < p.n_groups; ++g) widest = p.ldy[g] > widest ? p.ldy[g] : widest;
  if (chunk * widest * 2 > 0xffffffffll) return GA_EUNSUPPORTED;    // 32-bit offsets in a chunk
  const int64_t grid = (p.rows + chunk - 1) / chunk + (p.tp ? p.n_types : 0);
  hipLaunchKernelGGL((wide_mm_kernel<NF, NG, ATTN, TW, X8>), dim3((unsigned)grid), dim3(kWideBlock), lds, s, p,
                     (int)chunk);
  return launch_status();
}

template <int NF, int NG, bool ATTN>
int wide_launch_as(const WideMm &p, hipStream_t s) {
  // the 8-byte form only where its shapes occur: K <= 128, at most two groups
  if constexpr (NF <= 4 && NG <= 2) {
    if (p.K % 8 != 0) return wide_launch_x<NF, NG, ATTN, true>(p, s);
  }
  if (p.K % 8 != 0) return GA_EUNSUPPORTED;
  return wide_launch_x<NF, NG, ATTN, false>(p, s);
}

template <int NF, bool ATTN>
int wide_launch_groups(const WideMm &p, hipStream_t s) {
  switch (p.n_groups) {
    case 1: return wide_launch_as<NF, 1, ATTN>(p, s);
    case 2: return wide_launch_as<NF, 2, ATTN>(p, s);
    case 3: if (NF <= 4) return wide_launch_as<NF <= 4 ? NF : 4, 3, ATTN>(p, s); break;
    case 4: if (NF <= 4) return wide_launch_as<NF <= 4 ? NF : 4, 4, ATTN>(p, s); break;
  }
  return GA_EUNSUPPORTED;
}

}  // namespace

bool wide_mm_fits(int K, int n_groups) {
  if (K <= 0 || K % 4 != 0 || K > 256 || n_groups < 1 || n_groups > kWideMaxGroups) return false;
  if (K % 8 != 0 && (K > 128 || n_groups > 2)) return false;     // 8-byte row loads: see wide_launch_as
  const int nf = K <= 64 ? 2 : (K <= 128 ? 4 : 8);
  return (size_t)n_groups * wide_group_elems(nf) * sizeof(bf16_t) <= (size_t)kWideMaxLds;
}

int wide_mm_launch(const WideMm &p, hipStream_t s) {
  if (!wide_mm_fits(p.K, p.n_groups)) return GA_EUNSUPPORTED;
  if (p.rows <= 0) return GA_OK;
  if (p.rows > 0x7fffffff || !aligned(p.X, p.K % 8 == 0 ? 16 : 8)) return GA_EUNSUPPORTED;
  if (p.row_scale && (!aligned(p.row_scale, 4) || p.a_l[0])) return GA_EUNSUPPORTED;
  if (p.type_gate && (!aligned(p.type_gate, 4) || p.a_l[0])) return GA_EUNSUPPORTED;
  const bool attn = p.a_l[0] != nullptr;
  if (attn && p.dph != 32 && p.dph != 64 && p.dph != 128) return GA_EUNSUPPORTED;
  for (int g = 0; g < p.n_groups; ++g) {
    if (!p.W[g] || !p.Y[g] || !aligned(p.Y[g], 16) || p.ldy[g] % 8 != 0) return GA_EUNSUPPORTED;
    if (attn && (!p.a_l[g] || !p.a_r[g] || !p.el[g] || !p.er[g] || !aligned(p.a_l[g], 16) ||
                 !aligned(p.a_r[g], 16)))
      return GA_EUNSUPPORTED;
  }
  WideMm a = p;
  a.w_wide = true;
  for (int g = 0; g < p.n_groups; ++g)
    if (!aligned(p.W[g], 16) || p.ldw[g] % 8 != 0 || p.w_type_stride[g] % 8 != 0) a.w_wide = false;
  const int nf = p.K <= 64 ? 2 : (p.K <= 128 ? 4 : 8);
  if (attn) {
    if (nf == 2) return wide_launch_groups<2, true>(a, s);
    if (nf == 4) return wide_launch_groups<4, true>(a, s);
    return wide_launch_groups<8, true>(a, s);
  }
  if (nf == 2) return wide_launch_groups<2, false>(a, s);
  if (nf == 4) return wide_launch_groups<4, false>(a, s);
  return wide_launch_groups<8, false>(a, s);
}

}  // namespace ga
