// Dense node projection with the GAT attention terms in its epilogue (fp32):
//   Z = X @ W,  el[n, h] = <Z[n, h, :], a_l[h, :]>,  er[n, h] = <Z[n, h, :], a_r[h, :]>
// i.e. the dense operators that precede the graph chain in the reference's GAT
// plan (mm(h, fc_weight) and the two halves of mm(z2, attn_weight),
// examples/GAT/GAT.py:25-29 after the split / reorder passes) as one kernel, so
// Z is written once and never re-read for the attention terms.
//
// Tall-skinny GEMM on v_mfma_f32_16x16x4_f32: a workgroup (4 waves) owns 128
// rows, each wave 32 rows (2 tiles of 16) x 64 columns per pass.  Both operands
// go global -> registers -> LDS in slices of 32 k: the MFMA operand layout puts
// the 16 rows of a tile on 16 adjacent lanes, so loading X straight into that
// layout makes every lane its own cache access (the address unit then bounds
// the kernel at well under half the MFMA rate); staged through LDS, adjacent
// lanes read adjacent addresses of a row and the layout change costs one
// 16-byte LDS read per lane and 16 k.  Two register sets hold the slices one
// and two ahead of the one being multiplied, two LDS buffers the current and
// the next slice, so a slice costs one barrier and its global loads have two
// slices of MFMAs to arrive.  Accumulators come out as D[row][col] with 16
// adjacent lanes on 16 adjacent columns: Z stores coalesce, and the per-head
// dot products need one 16-lane DPP sum per row and head.
#include "common.h"

namespace ga {
namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kRT = 2;                                   // 16-row tiles per wave
constexpr int kWaveRows = kRT * 16;                      // 32
constexpr int kWgRows = kWaveRows * (kBlock / kWave);    // 128
constexpr int kCB = 4;                                   // 16-column blocks per pass
constexpr int kPassCols = kCB * 16;                      // 64
constexpr int kSliceK = 32;                              // k per LDS slice
constexpr int kXs = kSliceK + 4;                         // LDS row stride of the X tile
constexpr int kWs = kPassCols + 4;                       // LDS row stride of the W tile

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
template <bool HAS_ATTN, int VK>
// two waves per SIMD: with that register budget the accumulators stay in place
// across the loop (left to itself the allocator splits them over both register
// files and copies 48 of them every trip)
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(2, 2))) void
linear_attn_kernel(
    const float *__restrict__ X, const float *__restrict__ W,
    const float *__restrict__ a_l, const float *__restrict__ a_r,
    float *__restrict__ Z, float *__restrict__ el, float *__restrict__ er,
    int64_t rows, int K, int M, int heads) {
  using xvec_t = typename XVec<VK>::type;
  __shared__ __attribute__((aligned(16))) float xs[2][kWgRows * kXs];
  __shared__ __attribute__((aligned(16))) float ws[2][kSliceK * kWs];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int lr = lane & 15, lk = lane >> 4;
  const int col0 = blockIdx.y * kPassCols;               // first column of the pass
  const int64_t wg_row0 = (int64_t)blockIdx.x * kWgRows;
  const int64_t wrow0 = wg_row0 + wave * kWaveRows;
  const bool vec_w = (M & 3) == 0 && (reinterpret_cast<uintptr_t>(W) & 15) == 0;
  const int n_slices = (K + kSliceK - 1) / kSliceK;

  // X slice: 128 rows x 32 k in vectors of VK floats, kVpr per row; thread i
  // owns vectors i, i + 256, ...: a wave instruction reads 64 * VK * 4
  // contiguous-by-row bytes (8 * VK rows of 128 bytes).  Slices past the last
  // are fetched too (from the clamped address) and never multiplied.
  constexpr int kVpr = kSliceK / VK;                     // vectors per row and slice
  constexpr int kXPieces = kWgRows * kVpr / kBlock;      // 4 / 8 / 16 per thread
  constexpr int kRowStep = kBlock / kVpr;                // rows between a thread's vectors
  constexpr int kWPieces = kSliceK * (kPassCols / 4) / kBlock;  // float4 of W: 2
  struct Stage {
    xvec_t x[kXPieces];
    float4 w[kWPieces];
  };
  const int xr = threadIdx.x / kVpr, xc = (threadIdx.x % kVpr) * VK;
  const float *xbase[kXPieces];
#pragma unroll
  for (int j = 0; j < kXPieces; ++j)
    xbase[j] = X + min(wg_row0 + xr + j * kRowStep, rows - 1) * K;
  const bool w_cols_plain = vec_w && col0 + kPassCols <= M;     // uniform

  auto fetch = [&](int sl, Stage &st) {
    const int kc = min(sl * kSliceK + xc, K - VK);
#pragma unroll
    for (int j = 0; j < kXPieces; ++j)
      st.x[j] = *reinterpret_cast<const xvec_t *>(xbase[j] + kc);
#pragma unroll
    for (int j = 0; j < kWPieces; ++j) {
      const int i = threadIdx.x + j * kBlock;
      const int kk = min(sl * kSliceK + (i >> 4), K - 1), cc = col0 + (i & 15) * 4;
      const float *src = W + (int64_t)kk * M;
      if (w_cols_plain) {
        st.w[j] = *reinterpret_cast<const float4 *>(src + cc);
      } else {
        st.w[j].x = src[min(cc, M - 1)];
        st.w[j].y = src[min(cc + 1, M - 1)];
        st.w[j].z = src[min(cc + 2, M - 1)];
        st.w[j].w = src[min(cc + 3, M - 1)];
      }
    }
  };
  auto commit = [&](int sl, const Stage &st) {
    const int buf = sl & 1;
    const bool xin = sl * kSliceK + xc < K;
#pragma unroll
    for (int j = 0; j < kXPieces; ++j) {
      xvec_t v = st.x[j];
      if (!xin) v = xvec_t{};
      *reinterpret_cast<xvec_t *>(&xs[buf][(xr + j * kRowStep) * kXs + xc]) = v;
    }
#pragma unroll
    for (int j = 0; j < kWPieces; ++j) {
      const int i = threadIdx.x + j * kBlock;
      float4 v = st.w[j];
      const int cc = col0 + (i & 15) * 4;
      const bool kin = sl * kSliceK + (i >> 4) < K;
      v.x = kin && cc < M ? v.x : 0.0f;
      v.y = kin && cc + 1 < M ? v.y : 0.0f;
      v.z = kin && cc + 2 < M ? v.z : 0.0f;
      v.w = kin && cc + 3 < M ? v.w : 0.0f;
      *reinterpret_cast<float4 *>(&ws[buf][(i >> 4) * kWs + (i & 15) * 4]) = v;
    }
  };

  floatx4 acc[kRT][kCB];
#pragma unroll
  for (int t = 0; t < kRT; ++t)
#pragma unroll
    for (int cb = 0; cb < kCB; ++cb) acc[t][cb] = floatx4{0, 0, 0, 0};

  // MFMA operands of the lane: X[row lr of tile t][k = kb*16 + lk*4 + q] against
  // W[k = kb*16 + lk*4 + q][column cb*16 + lr], q = 0..3 (the k order inside a
  // block of 16 is permuted identically for both operands)
  const int xl_ofs = (wave * kWaveRows + lr) * kXs + lk * 4;
  const int wl_ofs = lk * 4 * kWs + lr;
  struct Frag {
    float4 x[kRT];
    float w[4][kCB];
  };
  auto read_frag = [&](int buf, int kb, Frag &f) {
    const float *xl = &xs[buf][xl_ofs + kb * 16];
    const float *wl = &ws[buf][wl_ofs + kb * 16 * kWs];
#pragma unroll
    for (int t = 0; t < kRT; ++t) f.x[t] = *reinterpret_cast<const float4 *>(xl + t * 16 * kXs);
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int cb = 0; cb < kCB; ++cb) f.w[q][cb] = wl[q * kWs + cb * 16];
  };
  auto mma = [&](const Frag &f) {
#pragma unroll
    for (int t = 0; t < kRT; ++t) {
      const float xv[4] = {f.x[t].x, f.x[t].y, f.x[t].z, f.x[t].w};
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int cb = 0; cb < kCB; ++cb)
          acc[t][cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(xv[q], f.w[q][cb], acc[t][cb], 0, 0, 0);
    }
  };
  // One slice.  Waves of one SIMD run this loop in step with each other, so a
  // stall is not covered by another wave's MFMAs: each wave hides its own.  The
  // fragments of a block are read from LDS while the block before it multiplies;
  // the next slice's registers go to the other LDS buffer (last read a slice ago,
  // before that slice's barrier) and the slice three ahead is fetched into the
  // registers just freed, all under the first block's MFMAs.
  Frag f0, f1;
  auto step = [&](int sl, Stage &next) {
    read_frag(sl & 1, 1, f1);
    __builtin_amdgcn_sched_barrier(0);
    mma(f0);
    commit(sl + 1, next);
    fetch(sl + 3, next);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    read_frag((sl + 1) & 1, 0, f0);
    __builtin_amdgcn_sched_barrier(0);
    mma(f1);
    __builtin_amdgcn_sched_barrier(0);
  };

  Stage sa, sb;                                          // even / odd slices
  fetch(0, sa);
  fetch(1, sb);
  commit(0, sa);
  fetch(2, sa);
  __syncthreads();
  read_frag(0, 0, f0);
  // slices in pairs (the register sets alternate), an odd last one on its own:
  // a conditional second half inside the loop would make the allocator copy
  // the accumulators around on every trip
  int sl = 0;
  for (; sl + 1 < n_slices; sl += 2) {
    step(sl, sb);
    step(sl + 1, sa);
  }
  if (sl < n_slices) step(sl, sb);

  // epilogue: lane holds rows wrow0 + t*16 + 4*lk + r, column col0 + cb*16 + lr
  float al[kCB], ar[kCB];
  const int dph = M / heads;
  const int bph = dph >> 4;                              // column blocks per head
  if (HAS_ATTN) {
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
#pragma unroll
      for (int cb = 0; cb < kCB; ++cb) {
        const int c = col0 + cb * 16 + lr;
        if (live && c < M) Z[row * M + c] = acc[t][cb][r];
      }
      if (HAS_ATTN) {
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

extern "C" int ga_linear_attn(const float *X, const float *W, const float *a_l,
                              const float *a_r, float *Z, float *el, float *er,
                              int64_t rows, int64_t K, int64_t M, int64_t heads,
                              ga_stream_t stream) {
  using namespace ga;
  if (rows < 0 || K <= 0 || M <= 0 || heads <= 0 || M % heads) return GA_EINVAL;
  if (rows > 0x7fffffff || K > 0x7fffffff || M > 0x7fffffff) return GA_EINVAL;
  if (rows == 0) return GA_OK;
  if (!X || !W || !Z) return GA_EINVAL;
  const bool attn = el != nullptr || er != nullptr;
  if (attn && (!el || !er || !a_l || !a_r)) return GA_EINVAL;
  if (!aligned(X, 4) || !aligned(W, 4) || !aligned(Z, 4)) return GA_EALIGN;
  const int vk = (K % 4 == 0 && aligned(X, 16)) ? 4 : ((K % 2 == 0 && aligned(X, 8)) ? 2 : 1);
  const int64_t dph = M / heads;
  if (attn && !(dph == 16 || dph == 32 || dph == 64)) return GA_EUNSUPPORTED;
  const int64_t gx = (rows + kWgRows - 1) / kWgRows;
  const int64_t gy = (M + kPassCols - 1) / kPassCols;
  if (gx > 0x7fffffff || gy > 65535) return GA_EUNSUPPORTED;
  hipStream_t s = (hipStream_t)stream;
#define GA_LAUNCH_LINEAR(ATTN, VK)                                                 \
  hipLaunchKernelGGL((linear_attn_kernel<ATTN, VK>), dim3((unsigned)gx, (unsigned)gy), \
                     dim3(kBlock), 0, s, X, W, a_l, a_r, Z, el, er, rows, (int)K,   \
                     (int)M, (int)heads)
  if (attn) {
    if (vk == 4) GA_LAUNCH_LINEAR(true, 4);
    else if (vk == 2) GA_LAUNCH_LINEAR(true, 2);
    else GA_LAUNCH_LINEAR(true, 1);
  } else {
    if (vk == 4) GA_LAUNCH_LINEAR(false, 4);
    else if (vk == 2) GA_LAUNCH_LINEAR(false, 2);
    else GA_LAUNCH_LINEAR(false, 1);
  }
#undef GA_LAUNCH_LINEAR
  return launch_status();
}
