// Dense node projection with the GAT attention terms in its epilogue (fp32):
//   Z = X @ W,  el[n, h] = <Z[n, h, :], a_l[h, :]>,  er[n, h] = <Z[n, h, :], a_r[h, :]>
// i.e. the dense operators that precede the graph chain in the reference's GAT
// plan (mm(h, fc_weight) and the two halves of mm(z2, attn_weight),
// examples/GAT/GAT.py:25-29 after the split / reorder passes) as one kernel, so
// Z is written once and never re-read for the attention terms.
//
// Tall-skinny GEMM on v_mfma_f32_16x16x4_f32: a workgroup (4 waves) owns 256
// rows, each wave 64 rows (4 tiles of 16) x 64 columns per pass; W is streamed
// through LDS in double-buffered slices of 64 k, X fragments go global ->
// registers (one 16-byte load per lane covers 16 k of a row, the k order inside
// a block being permuted identically for X and W).  Per slice and wave:
// 16 X loads, 64 LDS reads, 256 MFMAs.  Accumulators come out as D[row][col]
// with 16 adjacent lanes on 16 adjacent columns: Z stores coalesce, and the
// per-head dot products need one 16-lane shuffle tree per row and head.
#include "common.h"

namespace ga {
namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kRT = 4;                                   // 16-row tiles per wave
constexpr int kWaveRows = kRT * 16;                      // 64
constexpr int kWgRows = kWaveRows * (kBlock / kWave);    // 256
constexpr int kCB = 4;                                   // 16-column blocks per pass
constexpr int kPassCols = kCB * 16;                      // 64
constexpr int kSliceK = 64;                              // k per LDS slice
constexpr int kWs = kPassCols + 4;                       // padded LDS row stride

// HAS_ATTN: also produce el / er; requires heads to tile a pass exactly
// (dph = M / heads in {16, 32, 64}).
// VK = widest aligned vector (floats) a lane may use for its four k values:
// 4 when K % 4 == 0, 2 when K % 2 == 0, else 1.
template <bool HAS_ATTN, int VK>
__global__ __launch_bounds__(kBlock) void linear_attn_kernel(
    const float *__restrict__ X, const float *__restrict__ W,
    const float *__restrict__ a_l, const float *__restrict__ a_r,
    float *__restrict__ Z, float *__restrict__ el, float *__restrict__ er,
    int64_t rows, int K, int M, int heads) {
  __shared__ __attribute__((aligned(16))) float wt[2][kSliceK * kWs];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int lr = lane & 15, lk = lane >> 4;
  const int col0 = blockIdx.y * kPassCols;               // first column of the pass
  const int64_t wrow0 = (int64_t)blockIdx.x * kWgRows + wave * kWaveRows;
  const bool vec_w = (M & 3) == 0 && (reinterpret_cast<uintptr_t>(W) & 15) == 0;

  // slice sl (k in [sl*64, sl*64+64)) of W[:, col0:col0+64] -> wt[buf], zero padded
  auto stage = [&](int sl, int buf) {
    const int k0 = sl * kSliceK;
    for (int i = threadIdx.x; i < kSliceK * (kPassCols / 4); i += kBlock) {
      const int k = i >> 4, c4 = (i & 15) * 4;
      const int kk = k0 + k, cc = col0 + c4;
      float4 v = make_float4(0, 0, 0, 0);
      if (kk < K) {
        const float *src = W + (int64_t)kk * M + cc;
        if (vec_w && cc + 3 < M) {
          v = *reinterpret_cast<const float4 *>(src);
        } else {
          if (cc < M) v.x = src[0];
          if (cc + 1 < M) v.y = src[1];
          if (cc + 2 < M) v.z = src[2];
          if (cc + 3 < M) v.w = src[3];
        }
      }
      *reinterpret_cast<float4 *>(&wt[buf][k * kWs + c4]) = v;
    }
  };

  floatx4 acc[kRT][kCB];
#pragma unroll
  for (int t = 0; t < kRT; ++t)
#pragma unroll
    for (int cb = 0; cb < kCB; ++cb) acc[t][cb] = floatx4{0, 0, 0, 0};

  const float *xrow[kRT];
  bool xlive[kRT];
#pragma unroll
  for (int t = 0; t < kRT; ++t) {
    const int64_t r = wrow0 + t * 16 + lr;
    xlive[t] = r < rows;
    xrow[t] = X + (xlive[t] ? r : 0) * (int64_t)K + lk * 4;
  }

  // X fragments of k block kb (16 k): the lane's four values of each row tile
  auto load_frags = [&](int kofs, float4 (&xa)[kRT]) {
#pragma unroll
    for (int t = 0; t < kRT; ++t) {
      xa[t] = make_float4(0, 0, 0, 0);
      const int k0 = kofs + lk * 4;
      const float *px = xrow[t] + kofs;
      if (xlive[t] && k0 < K) {
        if (VK == 4) {
          xa[t] = *reinterpret_cast<const float4 *>(px);
        } else if (VK == 2) {
          const float2 lo = *reinterpret_cast<const float2 *>(px);
          xa[t].x = lo.x; xa[t].y = lo.y;
          if (k0 + 2 < K) {
            const float2 hi = *reinterpret_cast<const float2 *>(px + 2);
            xa[t].z = hi.x; xa[t].w = hi.y;
          }
        } else {
          xa[t].x = px[0];
          if (k0 + 1 < K) xa[t].y = px[1];
          if (k0 + 2 < K) xa[t].z = px[2];
          if (k0 + 3 < K) xa[t].w = px[3];
        }
      }
    }
  };

  const int n_slices = (K + kSliceK - 1) / kSliceK;
  stage(0, 0);
  float4 xn[kRT];
  load_frags(0, xn);                                     // software pipeline: the
  __syncthreads();                                       // next block's X is in
  for (int sl = 0; sl < n_slices; ++sl) {                // flight during the MFMAs
    const int buf = sl & 1;
    if (sl + 1 < n_slices) stage(sl + 1, buf ^ 1);       // other buffer: free since
    const float *wl = &wt[buf][lk * 4 * kWs + lr];       // the barrier of slice sl-1
#pragma unroll
    for (int kb = 0; kb < kSliceK / 16; ++kb) {
      const int kofs = sl * kSliceK + kb * 16;
      float4 xa[kRT];
#pragma unroll
      for (int t = 0; t < kRT; ++t) xa[t] = xn[t];
      load_frags(kofs + 16, xn);                         // zero beyond K
      float wv[4][kCB];
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int cb = 0; cb < kCB; ++cb) wv[q][cb] = wl[(kb * 16 + q) * kWs + cb * 16];
#pragma unroll
      for (int t = 0; t < kRT; ++t) {
        const float xv[4] = {xa[t].x, xa[t].y, xa[t].z, xa[t].w};
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int cb = 0; cb < kCB; ++cb)
            acc[t][cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(xv[q], wv[q][cb],
                                                              acc[t][cb], 0, 0, 0);
      }
    }
    __syncthreads();
  }

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
            float sl_ = pl[cb], sr_ = pr[cb];
            for (int o = 8; o > 0; o >>= 1) {
              sl_ += __shfl_xor(sl_, o);
              sr_ += __shfl_xor(sr_, o);
            }
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
