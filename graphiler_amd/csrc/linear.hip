// Dense node projection with the GAT attention terms in its epilogue (fp32):
//   Z = X @ W,  el[n, h] = <Z[n, h, :], a_l[h, :]>,  er[n, h] = <Z[n, h, :], a_r[h, :]>
// i.e. the dense operators that precede the graph chain in the reference's GAT
// plan (mm(h, fc_weight) and the two halves of mm(z2, attn_weight),
// examples/GAT/GAT.py:25-29 after the split / reorder passes) as one kernel, so
// Z is written once and never re-read for the attention terms.
//
// Tall-skinny GEMM with fp32 operands and fp32 results on the bf16 matrix
// instruction (v_mfma_f32_16x16x32_bf16, 16x the rate of the fp32 one): every
// operand value is split exactly into three bf16 pieces, x = x0 + x1 + x2 (8
// significant bits each, 24 in all), and the product is accumulated in fp32 from
// the six piece products of weight >= 2^-16, x0w0 + x0w1 + x1w0 + x1w1 + x0w2 +
// x2w0; each piece product is exact in fp32 and the three dropped ones are below
// 2^-24 of |x||w|, i.e. below the rounding of an fp32 product.  Measured against
// float64 the result is as close as the fp32 instruction's (max error / max |Z|
// 8e-7 against 1.2e-6 at K = 602).  Non-finite inputs give NaN (inf - inf in the
// split) where fp32 products may give inf.
//
// A workgroup (4 waves) owns 128 rows, each wave 32 rows (2 tiles of 16) x 64
// columns per pass.  Both operands go global -> registers -> LDS in
// slices of 32 k: the MFMA operand layout puts the 16 rows of a tile on 16
// adjacent lanes, so loading X straight into that layout makes every lane its
// own cache access; staged through LDS, adjacent lanes read adjacent addresses
// of a row.  X is staged as fp32 and split after the operand read (each value is
// consumed by exactly one lane); W is split when it is committed to LDS, as three
// [column][k] bf16 arrays, so an operand read is one 16-byte LDS read per piece.
// Loads go through buffer descriptors (fixed lane offsets, the slice as the scalar
// offset), so the loop has no address arithmetic.  Two register sets hold the slices
// one and two ahead of the one being multiplied.  Every wave stages the rows it
// multiplies itself, so the X tile needs one LDS buffer and no barrier (a wave's LDS
// accesses execute in order: the next slice is written after the current one has
// been read); the W pieces, shared by the four waves, have two buffers and cost the
// one barrier per slice.  The W operands of a column block are read while the block
// before it multiplies.  49 KB of LDS and under 168 registers: three workgroups per
// CU when the grid has at least one per CU; smaller grids are latency-bound and run
// the build with the two-per-CU register budget, which is faster there.
// Accumulators come out as D[row][col] with 16 adjacent lanes on 16 adjacent
// columns: Z stores coalesce, and the per-head dot products need one 16-lane DPP
// sum per row and head.
#include "common.h"

namespace ga {
namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

// x = p0 + p1 + p2 exactly, each piece a bf16 (the top 8 significant bits of
// what the pieces before it leave); eight values -> three packed operands.
__device__ __forceinline__ void split8(const float (&v)[8], uint4 &p0, uint4 &p1, uint4 &p2) {
  uint32_t a[8], b[8], c[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    a[j] = __float_as_uint(v[j]);
    const float r1 = v[j] - __uint_as_float(a[j] & 0xffff0000u);
    b[j] = __float_as_uint(r1);
    const float r2 = r1 - __uint_as_float(b[j] & 0xffff0000u);
    c[j] = __float_as_uint(r2);
  }
  constexpr uint32_t hi = 0x07060302u;                   // high halves of (S1, S0)
  p0 = uint4{__builtin_amdgcn_perm(a[1], a[0], hi), __builtin_amdgcn_perm(a[3], a[2], hi),
             __builtin_amdgcn_perm(a[5], a[4], hi), __builtin_amdgcn_perm(a[7], a[6], hi)};
  p1 = uint4{__builtin_amdgcn_perm(b[1], b[0], hi), __builtin_amdgcn_perm(b[3], b[2], hi),
             __builtin_amdgcn_perm(b[5], b[4], hi), __builtin_amdgcn_perm(b[7], b[6], hi)};
  p2 = uint4{__builtin_amdgcn_perm(c[1], c[0], hi), __builtin_amdgcn_perm(c[3], c[2], hi),
             __builtin_amdgcn_perm(c[5], c[4], hi), __builtin_amdgcn_perm(c[7], c[6], hi)};
}

constexpr int kRT = 2;                                   // 16-row tiles per wave
constexpr int kWaveRows = kRT * 16;                      // 32
constexpr int kWgRows = kWaveRows * (kBlock / kWave);    // 128
constexpr int kCB = 4;                                   // 16-column blocks per pass
constexpr int kPassCols = kCB * 16;                      // 64
constexpr int kSliceK = 32;                              // k per LDS slice
constexpr int kXs = kSliceK + 4;                         // LDS row stride of the X tile
constexpr int kWb = kSliceK / 2 + 4;                      // LDS column stride of a W piece, in bf16 pairs

template <int VK> struct XVec;
template <> struct XVec<4> { using type = float4; };
template <> struct XVec<2> { using type = float2; };
template <> struct XVec<1> { using type = float; };

// HAS_ATTN: also produce el / er; requires heads to tile a pass exactly
// (dph = M / heads in {16, 32, 64}).
// VK = widest aligned vector (floats) of a row of X: 4 when K % 4 == 0, 2 when
// K % 2 == 0, else 1.  K % VK == 0, so such a vector lies wholly inside or
// wholly outside a row: ragged edges clamp the address at fetch time (a valid
// one, the row's last vector) and zero by select at commit time, where the
// value is consumed anyway; no lane is ever predicated off in the k loop.
// WAVES: waves per SIMD the register allocation aims at (3 or 2)
// NCB: column blocks multiplied and stored, 4 or -- the plain projection onto at most 16
// columns (a GCN layer's hidden width) -- 1; the W tile is staged 64 columns wide either
// way, what shrinks is the matrix work and the operand reads.
template <bool HAS_ATTN, int VK, int WAVES, int NCB = kCB>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(WAVES, WAVES))) void
linear_attn_kernel(
    const float *__restrict__ X, const float *__restrict__ W,
    const float *__restrict__ a_l, const float *__restrict__ a_r,
    float *__restrict__ Z, float *__restrict__ el, float *__restrict__ er,
    const float *__restrict__ row_scale, int64_t rows, int K, int M, int heads) {
  static_assert(NCB == kCB || !HAS_ATTN, "the attention epilogue pairs up all four column blocks");
  using xvec_t = typename XVec<VK>::type;
  __shared__ __attribute__((aligned(16))) float xs[kWgRows * kXs];   // wave-private rows, one buffer
  __shared__ __attribute__((aligned(16))) uint32_t wb[2][3][kPassCols * kWb];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);   // in a scalar register
  const int lr = lane & 15, lk = lane >> 4;
  const int col0 = blockIdx.y * kPassCols;               // first column of the pass
  const int64_t wg_row0 = (int64_t)blockIdx.x * kWgRows;
  const int64_t wrow0 = wg_row0 + wave * kWaveRows;
  const int n_slices = (K + kSliceK - 1) / kSliceK;

  // X slice of a wave: its 32 rows x 32 k in vectors of VK floats, kVpr per row; lane
  // i owns vectors i, i + 64, ...: a wave instruction reads 64 * VK * 4
  // contiguous-by-row bytes (2 * VK rows of 128 bytes).  Slices past the last
  // are fetched too (from the clamped address) and never multiplied.
  constexpr int kVpr = kSliceK / VK;                     // vectors per row and slice
  constexpr int kXPieces = kWaveRows * kVpr / kWave;     // 4 / 8 / 16 per thread
  constexpr int kRowStep = kWave / kVpr;                 // rows between a thread's vectors
  struct Stage {
    xvec_t x[kXPieces];
    float w[8];
  };
  // Lane offsets (bytes) never change; the slice / the row of W is the scalar offset.
  // Slices that lie wholly inside the rows (all but the last, and that one too when
  // K % 32 == 0) take paths without clamps and selects.
  const int wc = threadIdx.x & 63, wkg = wave;               // column, group of 8 k
  const int xr = wave * kWaveRows + lane / kVpr, xc = (lane % kVpr) * VK;   // each wave stages its own rows
  const rsrc_t xrs = make_rsrc(X + wg_row0 * K, (uint64_t)(rows - wg_row0) * K * 4);
  const rsrc_t wrs = make_rsrc(W, (uint64_t)K * M * 4);
  uint32_t xoff[kXPieces];                               // the piece in slice 0
#pragma unroll
  for (int j = 0; j < kXPieces; ++j)
    xoff[j] = (uint32_t)((min(wg_row0 + xr + j * kRowStep, rows - 1) - wg_row0) * K + xc) * 4u;
  const uint32_t woff = (uint32_t)min(col0 + wc, M - 1) * 4u;
  const bool w_cols_full = col0 + kPassCols <= M;        // uniform

  auto fetch = [&](int sl, Stage &st) {
    if (sl * kSliceK + kSliceK <= K) {
#pragma unroll
      for (int j = 0; j < kXPieces; ++j)
        st.x[j] = BufLoad<VK>::at(xrs, xoff[j], (uint32_t)sl * (kSliceK * 4));
    } else {
      // clamped to the row's last vector (a valid address); zeroed at commit
      const uint32_t dk = (uint32_t)(min(sl * kSliceK + xc, K - VK) - xc) * 4u;
#pragma unroll
      for (int j = 0; j < kXPieces; ++j) st.x[j] = BufLoad<VK>::at(xrs, xoff[j] + dk, 0);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j)
      st.w[j] = BufLoad<1>::at(wrs, woff, (uint32_t)min(sl * kSliceK + wkg * 8 + j, K - 1) * (uint32_t)M * 4u);
  };
  auto commit = [&](int sl, const Stage &st) {
    const int buf = sl & 1;
    const bool inside = sl * kSliceK + kSliceK <= K;     // uniform
    if (inside) {
#pragma unroll
      for (int j = 0; j < kXPieces; ++j)
        *reinterpret_cast<xvec_t *>(&xs[(xr + j * kRowStep) * kXs + xc]) = st.x[j];
    } else {
      const bool xin = sl * kSliceK + xc < K;
#pragma unroll
      for (int j = 0; j < kXPieces; ++j) {
        xvec_t v = st.x[j];
        if (!xin) v = xvec_t{};
        *reinterpret_cast<xvec_t *>(&xs[(xr + j * kRowStep) * kXs + xc]) = v;
      }
    }
    float wv[8];
    if (inside && w_cols_full) {
#pragma unroll
      for (int j = 0; j < 8; ++j) wv[j] = st.w[j];
    } else {
      const bool cin = col0 + wc < M;
#pragma unroll
      for (int j = 0; j < 8; ++j)
        wv[j] = cin && sl * kSliceK + wkg * 8 + j < K ? st.w[j] : 0.0f;
    }
    uint4 p0, p1, p2;
    split8(wv, p0, p1, p2);
    *reinterpret_cast<uint4 *>(&wb[buf][0][wc * kWb + wkg * 4]) = p0;
    *reinterpret_cast<uint4 *>(&wb[buf][1][wc * kWb + wkg * 4]) = p1;
    *reinterpret_cast<uint4 *>(&wb[buf][2][wc * kWb + wkg * 4]) = p2;
  };

  floatx4 acc[kRT][NCB];
#pragma unroll
  for (int t = 0; t < kRT; ++t)
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) acc[t][cb] = floatx4{0, 0, 0, 0};

  const int xl_ofs = (wave * kWaveRows + lr) * kXs + lk * 8;
  const int wl_ofs = lr * kWb + lk * 4;                  // in uint32 (pairs of bf16)
  auto step = [&](int sl, Stage &next) {
    const int buf = sl & 1;
    float4 xa[kRT][2];
    uint4 wf[2][3];
#pragma unroll
    for (int t = 0; t < kRT; ++t) {
      xa[t][0] = *reinterpret_cast<const float4 *>(&xs[xl_ofs + t * 16 * kXs]);
      xa[t][1] = *reinterpret_cast<const float4 *>(&xs[xl_ofs + t * 16 * kXs + 4]);
    }
    auto read_w = [&](int cb, uint4 (&f)[3]) {
#pragma unroll
      for (int p = 0; p < 3; ++p)
        f[p] = *reinterpret_cast<const uint4 *>(&wb[buf][p][wl_ofs + cb * 16 * kWb]);
    };
    read_w(0, wf[0]);
    commit(sl + 1, next);
    fetch(sl + 3, next);
    uint4 xp[kRT][3];
#pragma unroll
    for (int t = 0; t < kRT; ++t) {
      const float v[8] = {xa[t][0].x, xa[t][0].y, xa[t][0].z, xa[t][0].w,
                          xa[t][1].x, xa[t][1].y, xa[t][1].z, xa[t][1].w};
      split8(v, xp[t][0], xp[t][1], xp[t][2]);
    }
    constexpr int px[6] = {2, 0, 1, 1, 0, 0}, pw[6] = {0, 2, 1, 0, 1, 0};
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
      if (cb + 1 < NCB) read_w(cb + 1, wf[(cb + 1) & 1]);
#pragma unroll
      for (int q = 0; q < 6; ++q)
#pragma unroll
        for (int t = 0; t < kRT; ++t)
          acc[t][cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              __builtin_bit_cast(bf16x8, xp[t][px[q]]), __builtin_bit_cast(bf16x8, wf[cb & 1][pw[q]]),
              acc[t][cb], 0, 0, 0);
    }
    __syncthreads();
  };

  Stage sa, sb;                                          // even / odd slices
  fetch(0, sa);
  fetch(1, sb);
  commit(0, sa);
  fetch(2, sa);
  __syncthreads();
  int sl = 0;
  for (; sl + 1 < n_slices; sl += 2) {
    step(sl, sb);
    step(sl + 1, sa);
  }
  if (sl < n_slices) step(sl, sb);

  // epilogue: lane holds rows wrow0 + t*16 + 4*lk + r, column col0 + cb*16 + lr
  // the row factors of the plain projection, all requested before the first store
  float rsv[kRT][4];
  if (!HAS_ATTN) {
#pragma unroll
    for (int t = 0; t < kRT; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int64_t row = wrow0 + t * 16 + lk * 4 + r;
        rsv[t][r] = row_scale && row < rows ? row_scale[row] : 1.0f;
      }
  }
  float al[kCB], ar[kCB];
  const int dph = M / heads;
  const int bph = dph >> 4;                              // column blocks per head
  if constexpr (HAS_ATTN) {
#pragma unroll
    for (int cb = 0; cb < kCB; ++cb) {
      const int c = col0 + cb * 16 + lr;
      al[cb] = c < M ? a_l[c] : 0.0f;                    // (heads, dph) is (M,) flat
      ar[cb] = c < M ? a_r[c] : 0.0f;
    }
  }
#pragma unroll
  for (int t = 0; t < kRT; ++t) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int64_t row = wrow0 + t * 16 + lk * 4 + r;
      const bool live = row < rows;
      if (!HAS_ATTN && row_scale) {                      // the plain projection only
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb) acc[t][cb][r] *= rsv[t][r];
      }
#pragma unroll
      for (int cb = 0; cb < NCB; ++cb) {
        const int c = col0 + cb * 16 + lr;
        if (live && c < M) Z[row * M + c] = acc[t][cb][r];
      }
      if constexpr (HAS_ATTN) {
        // lane-local products, blocks of one head added, then one 16-lane tree
        float pl[kCB], pr[kCB];
#pragma unroll
        for (int cb = 0; cb < kCB; ++cb) {
          pl[cb] = acc[t][cb][r] * al[cb];
          pr[cb] = acc[t][cb][r] * ar[cb];
        }
        if (bph >= 2) {
          pl[0] += pl[1]; pr[0] += pr[1];
          pl[2] += pl[3]; pr[2] += pr[3];
        }
        if (bph == 4) { pl[0] += pl[2]; pr[0] += pr[2]; }
#pragma unroll
        for (int cb = 0; cb < kCB; ++cb) {
          if (cb % bph == 0) {                           // first block of a head
            const float sl_ = row16_sum(pl[cb]), sr_ = row16_sum(pr[cb]);
            const int head = (col0 + cb * 16) / dph;
            if (live && lr == 0 && head < heads) {
              el[row * heads + head] = sl_;
              er[row * heads + head] = sr_;
            }
          }
        }
      }
    }
  }
}

}  // namespace
}  // namespace ga

namespace ga {
namespace {
int launch_linear(const float *X, const float *W, const float *a_l, const float *a_r, float *Z,
                  float *el, float *er, const float *row_scale, int64_t rows, int64_t K,
                  int64_t M, int64_t heads, ga_stream_t stream) {
  if (rows < 0 || K <= 0 || M <= 0 || heads <= 0 || M % heads) return GA_EINVAL;
  if (rows > 0x7fffffff || K > 0x7fffffff || M > 0x7fffffff) return GA_EINVAL;
  if (rows == 0) return GA_OK;
  if (!X || !W || !Z) return GA_EINVAL;
  // 32-bit byte offsets: 128 rows of K floats, and all of W
  if (K > (1 << 22) || K * M >= ((int64_t)1 << 30)) return GA_EUNSUPPORTED;
  const bool attn = el != nullptr || er != nullptr;
  if (attn && (!el || !er || !a_l || !a_r)) return GA_EINVAL;
  if (attn && row_scale) return GA_EINVAL;
  if (!aligned(X, 4) || !aligned(W, 4) || !aligned(Z, 4) || (row_scale && !aligned(row_scale, 4)))
    return GA_EALIGN;
  const int vk = (K % 4 == 0 && aligned(X, 16)) ? 4 : ((K % 2 == 0 && aligned(X, 8)) ? 2 : 1);
  const int64_t dph = M / heads;
  if (attn && !(dph == 16 || dph == 32 || dph == 64)) return GA_EUNSUPPORTED;
  const int64_t gx = (rows + kWgRows - 1) / kWgRows;
  const int64_t gy = (M + kPassCols - 1) / kPassCols;
  if (gx > 0x7fffffff || gy > 65535) return GA_EUNSUPPORTED;
  hipStream_t s = (hipStream_t)stream;
#define GA_LAUNCH_LINEAR_NCB(ATTN, VK, WAVES, NCB)                                  \
  hipLaunchKernelGGL((linear_attn_kernel<ATTN, VK, WAVES, NCB>),                   \
                     dim3((unsigned)gx, (unsigned)gy), dim3(kBlock), 0, s, X, W, a_l, a_r, Z, el, \
                     er, row_scale, rows, (int)K, (int)M, (int)heads)
#define GA_LAUNCH_LINEAR(ATTN, VK, WAVES)                           \
  do {                                                              \
    if (!ATTN && M <= 16) GA_LAUNCH_LINEAR_NCB(false, VK, WAVES, 1); \
    else GA_LAUNCH_LINEAR_NCB(ATTN, VK, WAVES, kCB);                 \
  } while (0)
#define GA_LAUNCH_LINEAR_VK(ATTN, WAVES)                 \
  do {                                                   \
    if (vk == 4) GA_LAUNCH_LINEAR(ATTN, 4, WAVES);       \
    else if (vk == 2) GA_LAUNCH_LINEAR(ATTN, 2, WAVES);  \
    else GA_LAUNCH_LINEAR(ATTN, 1, 2);                   \
  } while (0)
  // three workgroups per CU once there is at least one per CU to start with; below
  // that the kernel is latency-bound and the build with the larger register budget
  // (two per CU) has the shorter dependent chain per slice.  Rows that are only
  // 4-byte aligned (odd K) are staged one float per load: that build holds 32 staged
  // registers per lane, does not fit the three-workgroup budget without spilling
  // (measured 4x slower there), and always runs two per CU.
  constexpr int64_t kDeviceCUs = 256;                    // MI355X
  const bool dense_grid = gx * gy >= kDeviceCUs;
  if (attn) {
    if (dense_grid) GA_LAUNCH_LINEAR_VK(true, 3);
    else GA_LAUNCH_LINEAR_VK(true, 2);
  } else {
    if (dense_grid) GA_LAUNCH_LINEAR_VK(false, 3);
    else GA_LAUNCH_LINEAR_VK(false, 2);
  }
#undef GA_LAUNCH_LINEAR_VK
#undef GA_LAUNCH_LINEAR
#undef GA_LAUNCH_LINEAR_NCB
  return launch_status();
}
}  // namespace
}  // namespace ga

extern "C" int ga_linear_attn(const float *X, const float *W, const float *a_l,
                              const float *a_r, float *Z, float *el, float *er,
                              int64_t rows, int64_t K, int64_t M, int64_t heads,
                              ga_stream_t stream) {
  return ga::launch_linear(X, W, a_l, a_r, Z, el, er, nullptr, rows, K, M, heads, stream);
}

extern "C" int ga_linear_rows_scaled(const float *X, const float *W, const float *row_scale,
                                     float *Z, int64_t rows, int64_t K, int64_t M,
                                     ga_stream_t stream) {
  return ga::launch_linear(X, W, nullptr, nullptr, Z, nullptr, nullptr, row_scale, rows, K, M, 1,
                           stream);
}
