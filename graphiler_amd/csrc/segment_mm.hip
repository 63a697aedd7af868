// segment_mm (typed linear) for gfx950 on the matrix cores.
//
//   Y[r, h, :] = X[r, h, :] @ W[type(r), h, :, :]      rows sorted by type
//
// Every configured shape (K, M <= 128) is bound by streaming X in and Y out, so
// the kernel is organised around the row stream: a workgroup (4 waves) takes a
// chunk of consecutive rows of ONE type, keeps that type's weights for all heads
// in LDS, and each wave pushes 16-row tiles through MFMA with fp32 accumulation:
//   fp32: v_mfma_f32_16x16x4_f32, one 16-byte X load per lane covers K = 16
//         (the four components feed four MFMAs; the k order inside a block is
//         permuted identically for X and W, which a dot product allows);
//   bf16: v_mfma_f32_16x16x32_bf16, one 16-byte X load per lane covers K = 32.
// The product is formed transposed (D = W^T X^T) so that each lane ends up with
// four consecutive output columns of one row and stores them as one vector.
// The type of a chunk is found on the device from type_pointer (block-wide
// prefix sum of chunks per type): no host copy, no synchronisation.
#include "common.h"

namespace ga {
namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kTileRows = 16;              // rows per wave tile (MFMA N)
constexpr int kWaves = kBlock / kWave;     // 4
constexpr int kTileBlock = kTileRows * kWaves;  // 64 rows per workgroup step
constexpr int kMaxLds = 64 * 1024;

template <typename T>
struct MmTraits;
template <>
struct MmTraits<float> {
  static constexpr int kColGroup = 4;  // 16-column blocks accumulated per pass
  static __host__ __device__ int w_stride(int kb, int mb) { return mb * 16 + 4; }
  static __host__ __device__ size_t lds_bytes(int heads, int kb, int mb) {
    return (size_t)heads * kb * 16 * w_stride(kb, mb) * sizeof(float);
  }
};
template <>
struct MmTraits<bf16_t> {
  static constexpr int kColGroup = 8;
  static __host__ __device__ int w_stride(int kb, int mb) { return kb * 32 + 8; }
  static __host__ __device__ size_t lds_bytes(int heads, int kb, int mb) {
    return (size_t)heads * mb * 16 * w_stride(kb, mb) * sizeof(bf16_t);
  }
};

// Which chunk of which type does this workgroup own?  chunks(t) =
// ceil(rows_t / chunk_rows); workgroup id -> (t, first row, end row).
__device__ __forceinline__ bool locate_chunk(const int32_t *__restrict__ tp,
                                             int n_types, int chunk_rows,
                                             int &type, int &row0, int &row1) {
  __shared__ int scan[kBlock];
  __shared__ int found[3];
  if (threadIdx.x == 0) found[0] = -1;
  const int target = blockIdx.x;
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

// ---- fp32 ----------------------------------------------------------------
__global__ __launch_bounds__(kBlock) void segment_mm_f32_kernel(
    const int32_t *__restrict__ tp, int n_types, const float *__restrict__ X,
    const float *__restrict__ W, float *__restrict__ Y, int heads, int K, int M,
    int KB, int MB, int chunk_rows) {
  typedef MmTraits<float> Tr;
  extern __shared__ __attribute__((aligned(16))) float ldsw[];
  int type, row0, row1;
  if (!locate_chunk(tp, n_types, chunk_rows, type, row0, row1)) return;

  const int ws = Tr::w_stride(KB, MB);
  const int kpad = KB * 16, mpad = MB * 16;
  // weights of this type, all heads: ldsw[h][k][m], zero padded
  for (int i = threadIdx.x; i < heads * kpad * mpad; i += kBlock) {
    const int m = i % mpad;
    const int k = (i / mpad) % kpad;
    const int h = i / (mpad * kpad);
    float v = 0.0f;
    if (k < K && m < M) v = W[(((int64_t)type * heads + h) * K + k) * M + m];
    ldsw[(h * kpad + k) * ws + m] = v;
  }
  __syncthreads();

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int lr = lane & 15;   // row inside the tile / column inside a block
  const int lk = lane >> 4;   // k slot (0..3)
  const int64_t ldx = (int64_t)heads * K, ldy = (int64_t)heads * M;
  const bool vec_store = (M & 3) == 0;

  for (int tile0 = row0 + wave * kTileRows; tile0 < row1; tile0 += kTileBlock) {
    const int row = tile0 + lr;
    const bool live = row < row1;
    for (int h = 0; h < heads; ++h) {
      const float *xrow = X + (int64_t)row * ldx + (int64_t)h * K;
      const float *wh = ldsw + h * kpad * ws;
      for (int cg = 0; cg < MB; cg += Tr::kColGroup) {
        floatx4 acc[Tr::kColGroup];
#pragma unroll
        for (int cb = 0; cb < Tr::kColGroup; ++cb) acc[cb] = floatx4{0, 0, 0, 0};
        for (int kb = 0; kb < KB; ++kb) {
          const int k0 = kb * 16 + lk * 4;
          float4 xa = make_float4(0, 0, 0, 0);
          if (live && k0 < K) xa = *reinterpret_cast<const float4 *>(xrow + k0);
          const float xv[4] = {xa.x, xa.y, xa.z, xa.w};
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const float *wk = wh + (k0 + q) * ws + lr;
#pragma unroll
            for (int cb = 0; cb < Tr::kColGroup; ++cb) {
              if (cg + cb < MB)
                acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                    wk[(cg + cb) * 16], xv[q], acc[cb], 0, 0, 0);
            }
          }
        }
        if (live) {
          float *yrow = Y + (int64_t)row * ldy + (int64_t)h * M;
#pragma unroll
          for (int cb = 0; cb < Tr::kColGroup; ++cb) {
            const int m0 = (cg + cb) * 16 + lk * 4;
            if (cg + cb < MB && m0 < M) {
              if (vec_store) {
                *reinterpret_cast<float4 *>(yrow + m0) =
                    make_float4(acc[cb][0], acc[cb][1], acc[cb][2], acc[cb][3]);
              } else {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                  if (m0 + r < M) yrow[m0 + r] = acc[cb][r];
              }
            }
          }
        }
      }
    }
  }
}

// ---- bf16 ----------------------------------------------------------------
__global__ __launch_bounds__(kBlock) void segment_mm_bf16_kernel(
    const int32_t *__restrict__ tp, int n_types, const bf16_t *__restrict__ X,
    const bf16_t *__restrict__ W, bf16_t *__restrict__ Y, int heads, int K, int M,
    int KB, int MB, int chunk_rows) {
  typedef MmTraits<bf16_t> Tr;
  extern __shared__ __attribute__((aligned(16))) float ldsw_raw[];
  bf16_t *ldsw = reinterpret_cast<bf16_t *>(ldsw_raw);
  int type, row0, row1;
  if (!locate_chunk(tp, n_types, chunk_rows, type, row0, row1)) return;

  const int ws = Tr::w_stride(KB, MB);
  const int kpad = KB * 32, mpad = MB * 16;
  // weights of this type, all heads, transposed: ldsw[h][m][k], zero padded
  for (int i = threadIdx.x; i < heads * kpad * mpad; i += kBlock) {
    const int m = i % mpad;
    const int k = (i / mpad) % kpad;
    const int h = i / (mpad * kpad);
    bf16_t v = 0;
    if (k < K && m < M) v = W[(((int64_t)type * heads + h) * K + k) * M + m];
    ldsw[(h * mpad + m) * ws + k] = v;
  }
  __syncthreads();

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int lr = lane & 15;
  const int lk = lane >> 4;
  const int64_t ldx = (int64_t)heads * K, ldy = (int64_t)heads * M;
  const bool vec_store = (M & 3) == 0;

  for (int tile0 = row0 + wave * kTileRows; tile0 < row1; tile0 += kTileBlock) {
    const int row = tile0 + lr;
    const bool live = row < row1;
    for (int h = 0; h < heads; ++h) {
      const bf16_t *xrow = X + (int64_t)row * ldx + (int64_t)h * K;
      const bf16_t *wh = ldsw + h * mpad * ws;
      for (int cg = 0; cg < MB; cg += Tr::kColGroup) {
        floatx4 acc[Tr::kColGroup];
#pragma unroll
        for (int cb = 0; cb < Tr::kColGroup; ++cb) acc[cb] = floatx4{0, 0, 0, 0};
        for (int kb = 0; kb < KB; ++kb) {
          const int k0 = kb * 32 + lk * 8;
          uint4 xa = make_uint4(0, 0, 0, 0);
          if (live && k0 < K) xa = *reinterpret_cast<const uint4 *>(xrow + k0);
          const bf16x8 xv = __builtin_bit_cast(bf16x8, xa);
#pragma unroll
          for (int cb = 0; cb < Tr::kColGroup; ++cb) {
            if (cg + cb < MB) {
              const uint4 wa = *reinterpret_cast<const uint4 *>(
                  wh + ((cg + cb) * 16 + lr) * ws + k0);
              acc[cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                  __builtin_bit_cast(bf16x8, wa), xv, acc[cb], 0, 0, 0);
            }
          }
        }
        if (live) {
          bf16_t *yrow = Y + (int64_t)row * ldy + (int64_t)h * M;
#pragma unroll
          for (int cb = 0; cb < Tr::kColGroup; ++cb) {
            const int m0 = (cg + cb) * 16 + lk * 4;
            if (cg + cb < MB && m0 < M) {
              if (vec_store) {
                uint2 o;
                o.x = pack_bf16(acc[cb][0], acc[cb][1]);
                o.y = pack_bf16(acc[cb][2], acc[cb][3]);
                *reinterpret_cast<uint2 *>(yrow + m0) = o;
              } else {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                  if (m0 + r < M) yrow[m0 + r] = (bf16_t)f32_to_bf16_bits(acc[cb][r]);
              }
            }
          }
        }
      }
    }
  }
}

// ---- any shape: one thread per output element ------------------------------
template <typename T>
__device__ __forceinline__ float ldf(const T *p);
template <>
__device__ __forceinline__ float ldf<float>(const float *p) { return *p; }
template <>
__device__ __forceinline__ float ldf<bf16_t>(const bf16_t *p) { return bf16_lo(*p); }
__device__ __forceinline__ void stf(float *p, float v) { *p = v; }
__device__ __forceinline__ void stf(bf16_t *p, float v) { *p = (bf16_t)f32_to_bf16_bits(v); }

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

}  // namespace
}  // namespace ga

extern "C" int ga_segment_mm(const int32_t *type_pointer, int64_t n_types,
                             const void *X, const void *W, void *Y, int64_t rows,
                             int64_t heads, int64_t K, int64_t M, int dtype,
                             ga_stream_t stream) {
  using namespace ga;
  if (n_types < 0 || rows < 0 || heads <= 0 || K <= 0 || M <= 0) return GA_EINVAL;
  if (dtype != GA_F32 && dtype != GA_BF16) return GA_EINVAL;
  if (rows > 0x7fffffff || n_types > 0x7fffffff || heads * K > 0x7fffffff ||
      heads * M > 0x7fffffff)
    return GA_EINVAL;
  if (rows == 0 || n_types == 0) return GA_OK;
  if (!type_pointer || !X || !W || !Y) return GA_EINVAL;
  const size_t esz = dtype == GA_F32 ? 4 : 2;
  if (!aligned(X, esz) || !aligned(W, esz) || !aligned(Y, esz)) return GA_EALIGN;
  hipStream_t s = (hipStream_t)stream;

  const int kblk = dtype == GA_F32 ? 16 : 32;
  const int vec = dtype == GA_F32 ? 4 : 8;
  const int KB = (int)((K + kblk - 1) / kblk), MB = (int)((M + 15) / 16);
  const size_t lds = dtype == GA_F32 ? MmTraits<float>::lds_bytes((int)heads, KB, MB)
                                     : MmTraits<bf16_t>::lds_bytes((int)heads, KB, MB);
  const bool mfma_ok = K % vec == 0 && aligned(X, 16) && aligned(Y, 16) &&
                       lds <= (size_t)kMaxLds;
  if (mfma_ok) {
    // rows per workgroup: a multiple of the 64-row step, large enough to
    // amortise the weight load, small enough to keep every CU busy
    int64_t steps = rows / (kTileBlock * 1024);
    if (steps < 1) steps = 1;
    if (steps > 16) steps = 16;
    const int chunk_rows = (int)steps * kTileBlock;
    const int64_t grid = (rows + chunk_rows - 1) / chunk_rows + n_types;
    if (grid > 0x7fffffff) return GA_EUNSUPPORTED;
    if (dtype == GA_F32)
      hipLaunchKernelGGL(segment_mm_f32_kernel, dim3((unsigned)grid), dim3(kBlock),
                         lds, s, type_pointer, (int)n_types, (const float *)X,
                         (const float *)W, (float *)Y, (int)heads, (int)K, (int)M,
                         KB, MB, chunk_rows);
    else
      hipLaunchKernelGGL(segment_mm_bf16_kernel, dim3((unsigned)grid), dim3(kBlock),
                         lds, s, type_pointer, (int)n_types, (const bf16_t *)X,
                         (const bf16_t *)W, (bf16_t *)Y, (int)heads, (int)K, (int)M,
                         KB, MB, chunk_rows);
    return launch_status();
  }
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
