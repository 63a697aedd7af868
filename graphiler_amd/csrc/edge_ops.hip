// Per-edge streaming kernels for gfx950: SDDMM (u_add_v, u_dot_v) and the row
// gather behind the Broadcast* operators.  All are bandwidth bound: index
// columns and outputs are read/written once, fully coalesced; the node rows are
// gathered with 16-byte accesses where the shapes allow.
#include "common.h"

namespace ga {
namespace {

template <typename T>
__device__ __forceinline__ float load_f32(const T *p);
template <>
__device__ __forceinline__ float load_f32<float>(const float *p) { return *p; }
template <>
__device__ __forceinline__ float load_f32<bf16_t>(const bf16_t *p) {
  return bf16_lo(*p);
}

// a / b for 0 <= a, 0 < b: the 32-bit division when the numerator fits, which is
// several times shorter than the 64-bit one the flat indexings would otherwise pay
// per element.
__device__ __forceinline__ int64_t div_pos(int64_t a, int b) {
  return (a >> 32) == 0 ? (int64_t)((uint32_t)a / (uint32_t)b) : a / b;
}

// ---- u (op) v --------------------------------------------------------------
// One thread per output element; FEAT1 specialisation handles four consecutive
// edges per thread so index and output accesses are 16 bytes wide.  OP is the
// binary functor (functor.cuh:19-72): one fp32 operation per element.
template <int OP>
__device__ __forceinline__ float edge_op(float a, float b) {
  if (OP == GA_SDDMM_SUB) return a - b;
  if (OP == GA_SDDMM_MUL) return a * b;
  if (OP == GA_SDDMM_DIV) return a / b;
  return a + b;
}

template <typename IdxT, typename T, int OP>
__global__ __launch_bounds__(kBlock) void u_add_v_kernel(
    const IdxT *__restrict__ lhs, const IdxT *__restrict__ rhs,
    const T *__restrict__ u, const T *__restrict__ v, float *__restrict__ out,
    int64_t n_edges, int feat) {
  const int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (t >= n_edges * feat) return;
  const int64_t i = div_pos(t, feat);
  const int k = (int)(t - i * feat);
  out[t] = edge_op<OP>(load_f32(u + (int64_t)lhs[i] * feat + k),
                       load_f32(v + (int64_t)rhs[i] * feat + k));
}

template <typename IdxT, typename T, int OP>
__global__ __launch_bounds__(kBlock) void u_add_v_feat1_kernel(
    const IdxT *__restrict__ lhs, const IdxT *__restrict__ rhs,
    const T *__restrict__ u, const T *__restrict__ v, float *__restrict__ out,
    int64_t n_edges) {
  const int64_t i0 = ((int64_t)blockIdx.x * kBlock + threadIdx.x) * 4;
  if (i0 >= n_edges) return;
  if (i0 + 4 <= n_edges) {
    IdxT l[4], r[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) { l[q] = lhs[i0 + q]; r[q] = rhs[i0 + q]; }
    float o[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) o[q] = edge_op<OP>(load_f32(u + l[q]), load_f32(v + r[q]));
    *reinterpret_cast<float4 *>(out + i0) = make_float4(o[0], o[1], o[2], o[3]);
  } else {
    for (int64_t i = i0; i < n_edges; ++i)
      out[i] = edge_op<OP>(load_f32(u + lhs[i]), load_f32(v + rhs[i]));
  }
}

// ---- u_dot_v ---------------------------------------------------------------
// A group of `gl` lanes covers the heads*dim elements of one edge with 16-byte
// loads; the `lph` lanes of a head are combined with xor shuffles (fixed tree).
template <typename IdxT, typename T, int VEC>
__global__ __launch_bounds__(kBlock) void u_dot_v_vec_kernel(
    const IdxT *__restrict__ lhs, const IdxT *__restrict__ rhs,
    const T *__restrict__ u, const T *__restrict__ v, float *__restrict__ out,
    int64_t n_edges, int heads, int dim, int gl_shift, int lph) {
  typedef Frag<T, VEC> IO;
  const int gl = 1 << gl_shift;
  const int lane = threadIdx.x & (gl - 1);
  const int64_t i = ((int64_t)blockIdx.x * kBlock + threadIdx.x) >> gl_shift;
  const int feat = heads * dim;
  const bool live = i < n_edges && lane * VEC < feat;
  float s = 0.0f;
  if (live) {
    const typename IO::raw_t a = IO::load(u + (int64_t)lhs[i] * feat + lane * VEC);
    const typename IO::raw_t b = IO::load(v + (int64_t)rhs[i] * feat + lane * VEC);
    float af[VEC], bf[VEC];
    IO::widen(a, af);
    IO::widen(b, bf);
#pragma unroll
    for (int q = 0; q < VEC; ++q) s = fmaf(af[q], bf[q], s);
  }
  for (int off = lph >> 1; off > 0; off >>= 1) s += __shfl_xor(s, off);
  if (live && (lane & (lph - 1)) == 0) out[i * heads + lane / lph] = s;
}

// Shapes the kernel above does not take (a row wider than a wavefront's 16-byte
// loads, a head width that is not a power-of-two number of such loads, unaligned
// storage): a group of 2^lpu_shift lanes per (edge, head) walks the head's `dim`
// elements, VEC at a time (VEC > 1: dim % VEC == 0 and 16-byte aligned rows), the
// lanes reading consecutive pieces; combined with xor shuffles (fixed tree).
template <typename IdxT, typename T, int VEC>
__global__ __launch_bounds__(kBlock) void u_dot_v_group_kernel(
    const IdxT *__restrict__ lhs, const IdxT *__restrict__ rhs,
    const T *__restrict__ u, const T *__restrict__ v, float *__restrict__ out,
    int64_t n_units, int heads, int dim, int lpu_shift) {
  typedef Frag<T, VEC> IO;
  const int lpu = 1 << lpu_shift;
  const int lane = threadIdx.x & (lpu - 1);
  const int64_t unit = ((int64_t)blockIdx.x * kBlock + threadIdx.x) >> lpu_shift;
  const bool live = unit < n_units;
  float s = 0.0f;
  if (live) {
    const int64_t i = div_pos(unit, heads);
    const int h = (int)(unit - i * heads);
    const T *a = u + ((int64_t)lhs[i] * heads + h) * dim;
    const T *b = v + ((int64_t)rhs[i] * heads + h) * dim;
    for (int q = lane * VEC; q < dim; q += lpu * VEC) {
      float af[VEC], bf[VEC];
      IO::widen(IO::load(a + q), af);
      IO::widen(IO::load(b + q), bf);
#pragma unroll
      for (int t = 0; t < VEC; ++t) s = fmaf(af[t], bf[t], s);
    }
  }
  for (int off = lpu >> 1; off > 0; off >>= 1) s += __shfl_xor(s, off);
  if (live && lane == 0) out[unit] = s;
}

// ---- row gather --------------------------------------------------------------
template <typename IdxT, typename UnitT>
__global__ __launch_bounds__(kBlock) void gather_rows_kernel(
    const IdxT *__restrict__ idx, const UnitT *__restrict__ x,
    UnitT *__restrict__ y, int64_t n_out, int64_t units, int gl_shift) {
  const int gl = 1 << gl_shift;
  const int lane = threadIdx.x & (gl - 1);
  const int64_t i = ((int64_t)blockIdx.x * kBlock + threadIdx.x) >> gl_shift;
  if (i >= n_out) return;
  const UnitT *src = x + (int64_t)idx[i] * units;
  UnitT *dst = y + i * units;
  for (int64_t q = lane; q < units; q += gl) dst[q] = src[q];
}

// Rows whose unit count leaves many lanes of a power-of-two lane group idle: one
// thread per output unit instead, so reads and writes are contiguous over the
// whole wavefront whatever the row length.
template <typename IdxT, typename UnitT>
__global__ __launch_bounds__(kBlock) void gather_units_kernel(
    const IdxT *__restrict__ idx, const UnitT *__restrict__ x,
    UnitT *__restrict__ y, int64_t n_units_total, int units) {
  const int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (t >= n_units_total) return;
  const int64_t i = div_pos(t, units);
  const int k = (int)(t - i * units);
  y[t] = x[(int64_t)idx[i] * units + k];
}

// Rows of 256 bytes or more that are only 4- or 2-byte aligned (129 floats, 129 bf16
// values): 16-byte pieces moved through a type of that alignment -- the load / store
// unit takes such addresses, and a fraction of the accesses beats aligned narrow ones
// -- and the few units left over at the end of the row by the group's first lanes.
template <typename UnitT>
struct __attribute__((packed, aligned(sizeof(UnitT)))) Piece16 {
  UnitT u[16 / sizeof(UnitT)];
};

template <typename IdxT, typename UnitT>
__global__ __launch_bounds__(kBlock) void gather_rows_pieces_kernel(
    const IdxT *__restrict__ idx, const UnitT *__restrict__ x,
    UnitT *__restrict__ y, int64_t n_out, int64_t units, int gl_shift) {
  constexpr int kPer = 16 / sizeof(UnitT);    // units per piece; the tail is shorter
  const int gl = 1 << gl_shift;               // >= 16 lanes: rows have >= 16 pieces
  const int lane = threadIdx.x & (gl - 1);
  const int64_t i = ((int64_t)blockIdx.x * kBlock + threadIdx.x) >> gl_shift;
  if (i >= n_out) return;
  const UnitT *src = x + (int64_t)idx[i] * units;
  UnitT *dst = y + i * units;
  const int64_t pieces = units / kPer;
  for (int64_t q = lane; q < pieces; q += gl)
    *reinterpret_cast<Piece16<UnitT> *>(dst + kPer * q) =
        *reinterpret_cast<const Piece16<UnitT> *>(src + kPer * q);
  const int64_t t = kPer * pieces + lane;
  if (t < units) dst[t] = src[t];
}

template <typename IdxT, typename UnitT>
int launch_gather_pieces(const void *idx, const void *x, void *y, int64_t n_out,
                         int64_t row_bytes, hipStream_t s) {
  const int64_t units = row_bytes / (int64_t)sizeof(UnitT), pieces = row_bytes / 16;
  const int gl_shift = ilog2_ceil((uint64_t)(pieces > kWave ? kWave : pieces));
  const int64_t per_block = kBlock >> gl_shift;
  const int64_t blocks = (n_out + per_block - 1) / per_block;
  if (blocks > 0x7fffffff) return GA_EUNSUPPORTED;
  hipLaunchKernelGGL((gather_rows_pieces_kernel<IdxT, UnitT>), dim3((unsigned)blocks),
                     dim3(kBlock), 0, s, (const IdxT *)idx, (const UnitT *)x, (UnitT *)y, n_out,
                     units, gl_shift);
  return launch_status();
}

template <typename IdxT, typename UnitT>
int launch_gather(const void *idx, const void *x, void *y, int64_t n_out,
                  int64_t units, hipStream_t s) {
  const int gl_shift = ilog2_ceil((uint64_t)(units > kWave ? kWave : units));
  const int64_t gl = (int64_t)1 << gl_shift;
  const int64_t lane_slots = (units + gl - 1) / gl * gl;   // lanes x iterations per row
  // more than 1/9 of them idle; longer rows amortise the idle tail and lose more to
  // the per-element index arithmetic (measured: 129 units 15 % slower this way)
  if (lane_slots * 8 > units * 9 && units < kWave) {
    const int64_t total = n_out * units;
    const int64_t fblocks = (total + kBlock - 1) / kBlock;
    if (fblocks > 0x7fffffff) return GA_EUNSUPPORTED;
    hipLaunchKernelGGL((gather_units_kernel<IdxT, UnitT>), dim3((unsigned)fblocks),
                       dim3(kBlock), 0, s, (const IdxT *)idx, (const UnitT *)x,
                       (UnitT *)y, total, (int)units);
    return launch_status();
  }
  const int64_t per_block = kBlock >> gl_shift;
  const int64_t blocks = (n_out + per_block - 1) / per_block;
  if (blocks > 0x7fffffff) return GA_EUNSUPPORTED;
  hipLaunchKernelGGL((gather_rows_kernel<IdxT, UnitT>), dim3((unsigned)blocks),
                     dim3(kBlock), 0, s, (const IdxT *)idx, (const UnitT *)x,
                     (UnitT *)y, n_out, units, gl_shift);
  return launch_status();
}

template <typename IdxT>
int pick_gather_unit(const void *idx, const void *x, void *y, int64_t n_out,
                     int64_t row_bytes, hipStream_t s) {
  const uintptr_t bits = reinterpret_cast<uintptr_t>(x) |
                         reinterpret_cast<uintptr_t>(y) | (uintptr_t)row_bytes;
  if ((bits & 15) == 0)
    return launch_gather<IdxT, uint4>(idx, x, y, n_out, row_bytes / 16, s);
  if ((bits & 7) == 0)
    return launch_gather<IdxT, uint2>(idx, x, y, n_out, row_bytes / 8, s);
  if ((bits & 3) == 0) {
    if (row_bytes >= 256) return launch_gather_pieces<IdxT, uint32_t>(idx, x, y, n_out, row_bytes, s);
    return launch_gather<IdxT, uint32_t>(idx, x, y, n_out, row_bytes / 4, s);
  }
  if ((bits & 1) == 0) {
    if (row_bytes >= 256) return launch_gather_pieces<IdxT, uint16_t>(idx, x, y, n_out, row_bytes, s);
    return launch_gather<IdxT, uint16_t>(idx, x, y, n_out, row_bytes / 2, s);
  }
  return launch_gather<IdxT, uint8_t>(idx, x, y, n_out, row_bytes, s);
}

template <typename IdxT, typename T, int OP>
int launch_u_op_v(const void *lhs, const void *rhs, const void *u,
                   const void *v, float *out, int64_t n_edges, int feat,
                   hipStream_t s) {
  if (feat == 1 && aligned(out, 16)) {
    const int64_t threads = (n_edges + 3) / 4;
    const int64_t blocks = (threads + kBlock - 1) / kBlock;
    hipLaunchKernelGGL((u_add_v_feat1_kernel<IdxT, T, OP>), dim3((unsigned)blocks),
                       dim3(kBlock), 0, s, (const IdxT *)lhs, (const IdxT *)rhs,
                       (const T *)u, (const T *)v, out, n_edges);
  } else {
    const int64_t blocks = (n_edges * feat + kBlock - 1) / kBlock;
    if (blocks > 0x7fffffff) return GA_EUNSUPPORTED;
    hipLaunchKernelGGL((u_add_v_kernel<IdxT, T, OP>), dim3((unsigned)blocks),
                       dim3(kBlock), 0, s, (const IdxT *)lhs, (const IdxT *)rhs,
                       (const T *)u, (const T *)v, out, n_edges, feat);
  }
  return launch_status();
}

template <typename IdxT, typename T, int VEC>
int launch_u_dot_v_group(const void *lhs, const void *rhs, const void *u, const void *v,
                         float *out, int64_t n_edges, int heads, int dim, hipStream_t s) {
  // 16-byte pieces: one per lane and step, so a step reads the head's row contiguously;
  // single elements: about four steps per lane (measured: one lane per element loses to
  // a single lane per head at dim 5 and 17)
  const int64_t pieces = (dim + VEC - 1) / VEC;
  const int lpu_shift = VEC > 1 ? ilog2_ceil((uint64_t)(pieces > kWave ? kWave : pieces))
                                : ilog2_floor((uint64_t)(pieces >= 4 * kWave ? kWave
                                                         : (pieces >= 4 ? pieces / 4 : 1)));
  const int64_t n_units = n_edges * heads;
  const int64_t per_block = kBlock >> lpu_shift;
  const int64_t blocks = (n_units + per_block - 1) / per_block;
  if (blocks > 0x7fffffff) return GA_EUNSUPPORTED;
  hipLaunchKernelGGL((u_dot_v_group_kernel<IdxT, T, VEC>), dim3((unsigned)blocks),
                     dim3(kBlock), 0, s, (const IdxT *)lhs, (const IdxT *)rhs,
                     (const T *)u, (const T *)v, out, n_units, heads, dim, lpu_shift);
  return launch_status();
}

template <typename IdxT, typename T, int VEC>
int launch_u_dot_v(const void *lhs, const void *rhs, const void *u,
                   const void *v, float *out, int64_t n_edges, int heads,
                   int dim, hipStream_t s) {
  const int64_t feat = (int64_t)heads * dim;
  const int lph = dim / VEC;  // lanes per head
  const bool vec = VEC > 1 && dim % VEC == 0 && (lph & (lph - 1)) == 0 &&
                   feat / VEC <= kWave && aligned(u, 16) && aligned(v, 16);
  if (vec) {
    const int gl_shift = ilog2_ceil((uint64_t)(feat / VEC));
    const int64_t per_block = kBlock >> gl_shift;
    const int64_t blocks = (n_edges + per_block - 1) / per_block;
    if (blocks > 0x7fffffff) return GA_EUNSUPPORTED;
    hipLaunchKernelGGL((u_dot_v_vec_kernel<IdxT, T, VEC>),
                       dim3((unsigned)blocks), dim3(kBlock), 0, s,
                       (const IdxT *)lhs, (const IdxT *)rhs, (const T *)u,
                       (const T *)v, out, n_edges, heads, dim, gl_shift, lph);
  } else if (VEC > 1 && dim % VEC == 0 && aligned(u, 16) && aligned(v, 16)) {
    return launch_u_dot_v_group<IdxT, T, VEC>(lhs, rhs, u, v, out, n_edges, heads, dim, s);
  } else {
    return launch_u_dot_v_group<IdxT, T, 1>(lhs, rhs, u, v, out, n_edges, heads, dim, s);
  }
  return launch_status();
}

int check_edge_args(const void *lhs, const void *rhs, int idx_bits,
                    const void *u, const void *v, const float *out,
                    int64_t n_edges, int dtype) {
  if (n_edges < 0 || n_edges > 0x7fffffff) return GA_EINVAL;
  if (idx_bits != 32 && idx_bits != 64) return GA_EINVAL;
  if (dtype != GA_F32 && dtype != GA_BF16) return GA_EINVAL;
  if (n_edges == 0) return GA_OK;
  if (!lhs || !rhs || !u || !v || !out) return GA_EINVAL;
  const size_t esz = dtype == GA_F32 ? 4 : 2;
  if (!aligned(lhs, idx_bits / 8) || !aligned(rhs, idx_bits / 8) ||
      !aligned(u, esz) || !aligned(v, esz) || !aligned(out, 4))
    return GA_EALIGN;
  return GA_OK;
}

}  // namespace
}  // namespace ga

extern "C" {

int ga_sddmm_u_op_v(const void *lhs, const void *rhs, int idx_bits,
                    const void *u, const void *v, float *out, int64_t n_edges,
                    int64_t feat, int op, int dtype, ga_stream_t stream) {
  if (feat <= 0 || feat > 0x7fffffff) return GA_EINVAL;
  if (op < GA_SDDMM_ADD || op > GA_SDDMM_DIV) return GA_EINVAL;
  int rc = ga::check_edge_args(lhs, rhs, idx_bits, u, v, out, n_edges, dtype);
  if (rc != GA_OK || n_edges == 0) return rc;
  hipStream_t s = (hipStream_t)stream;
#define GA_U_OP_V(IDX, T)                                                             \
  switch (op) {                                                                       \
    case GA_SDDMM_SUB:                                                                \
      return ga::launch_u_op_v<IDX, T, GA_SDDMM_SUB>(lhs, rhs, u, v, out, n_edges, (int)feat, s); \
    case GA_SDDMM_MUL:                                                                \
      return ga::launch_u_op_v<IDX, T, GA_SDDMM_MUL>(lhs, rhs, u, v, out, n_edges, (int)feat, s); \
    case GA_SDDMM_DIV:                                                                \
      return ga::launch_u_op_v<IDX, T, GA_SDDMM_DIV>(lhs, rhs, u, v, out, n_edges, (int)feat, s); \
    default:                                                                          \
      return ga::launch_u_op_v<IDX, T, GA_SDDMM_ADD>(lhs, rhs, u, v, out, n_edges, (int)feat, s); \
  }
  if (idx_bits == 64) {
    if (dtype == GA_F32) GA_U_OP_V(int64_t, float)
    GA_U_OP_V(int64_t, ga::bf16_t)
  }
  if (dtype == GA_F32) GA_U_OP_V(int32_t, float)
  GA_U_OP_V(int32_t, ga::bf16_t)
#undef GA_U_OP_V
}

int ga_sddmm_u_add_v(const void *lhs, const void *rhs, int idx_bits,
                     const void *u, const void *v, float *out, int64_t n_edges,
                     int64_t feat, int dtype, ga_stream_t stream) {
  return ga_sddmm_u_op_v(lhs, rhs, idx_bits, u, v, out, n_edges, feat, GA_SDDMM_ADD, dtype,
                         stream);
}

int ga_sddmm_u_dot_v(const void *lhs, const void *rhs, int idx_bits,
                     const void *u, const void *v, float *out, int64_t n_edges,
                     int64_t heads, int64_t dim, int dtype, ga_stream_t stream) {
  if (heads <= 0 || dim <= 0 || heads * dim > 0x7fffffff) return GA_EINVAL;
  int rc = ga::check_edge_args(lhs, rhs, idx_bits, u, v, out, n_edges, dtype);
  if (rc != GA_OK || n_edges == 0) return rc;
  hipStream_t s = (hipStream_t)stream;
  if (idx_bits == 64)
    return dtype == GA_F32
               ? ga::launch_u_dot_v<int64_t, float, 4>(lhs, rhs, u, v, out,
                                                       n_edges, (int)heads,
                                                       (int)dim, s)
               : ga::launch_u_dot_v<int64_t, ga::bf16_t, 8>(lhs, rhs, u, v, out,
                                                            n_edges, (int)heads,
                                                            (int)dim, s);
  return dtype == GA_F32
             ? ga::launch_u_dot_v<int32_t, float, 4>(lhs, rhs, u, v, out,
                                                     n_edges, (int)heads,
                                                     (int)dim, s)
             : ga::launch_u_dot_v<int32_t, ga::bf16_t, 8>(lhs, rhs, u, v, out,
                                                          n_edges, (int)heads,
                                                          (int)dim, s);
}

int ga_gather_rows(const void *idx, int idx_bits, const void *x, void *y,
                   int64_t n_out, int64_t row_bytes, ga_stream_t stream) {
  if (n_out < 0 || row_bytes < 0 || (idx_bits != 32 && idx_bits != 64))
    return GA_EINVAL;
  if (n_out == 0 || row_bytes == 0) return GA_OK;
  if (!idx || !x || !y) return GA_EINVAL;
  if (!ga::aligned(idx, idx_bits / 8)) return GA_EALIGN;
  hipStream_t s = (hipStream_t)stream;
  return idx_bits == 64
             ? ga::pick_gather_unit<int64_t>(idx, x, y, n_out, row_bytes, s)
             : ga::pick_gather_unit<int32_t>(idx, x, y, n_out, row_bytes, s);
}

}  // extern "C"
