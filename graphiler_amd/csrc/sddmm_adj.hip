// SDDMM u (op) v over a grouped adjacency for gfx950: out[i, :] = u[nbr[i], :] (op)
// v[row(i), :] for every slot i, rows taken from the row pointer.
//
// The generic kernels of edge_ops.hip read two index columns per edge.  Over an
// adjacency the second one is the slot -> row column, 4 bytes per slot that the row
// pointer already implies: here a wavefront owns a chunk of 64 * kS consecutive
// slots (kS = 16 / feat, so a lane owns 64 bytes of output), looks up the rows of
// the chunk's first and last slot in that column (two reads per chunk) and takes
// the row starts in between from the row pointer -- the lane that finds a row start
// inside the chunk leaves the row's id and its v row at that slot in a wave-private
// LDS tile; a lane then reads the marks of its kS slots and carries the last one
// forward (what precedes its first mark is the largest mark of the lanes before it:
// a scan over the lanes).  v is therefore read once per row, coalesced, instead of
// once per slot; the only per-slot gather left is u[nbr[i]].  Index reads and output
// writes are 16 bytes wide.  One fp32 operation per element: bit-exact against the
// functors of functor.cuh:19-72.
#include "common.h"

namespace ga {
namespace {

constexpr int kAdjWaves = 4;      // wavefronts per workgroup (independent of each other)

template <int OP>
__device__ __forceinline__ float adj_op(float a, float b) {
  if (OP == GA_SDDMM_SUB) return a - b;
  if (OP == GA_SDDMM_MUL) return a * b;
  if (OP == GA_SDDMM_DIV) return a / b;
  return a + b;
}

// Tile word of value word e (lane e / 16 owns words 16 (e / 16) .. + 15): four 16-byte
// units per lane, stored at unit position u ^ ((lane >> 1) & 3) so that the eight
// lanes a 16-byte LDS access serves at a time fall on different banks.
__device__ __forceinline__ int adj_unit(int o, int u) {
  return (o << 4) + (((u ^ (o >> 1)) & 3) << 2);
}
__device__ __forceinline__ int adj_word(int e) {
  return adj_unit(e >> 4, (e >> 2) & 3) + (e & 3);
}

template <int F> struct RowVec;
template <> struct RowVec<1> { typedef float type; };
template <> struct RowVec<2> { typedef float2 type; };
template <> struct RowVec<4> { typedef float4 type; };

template <int F>
__device__ __forceinline__ void unpack(const typename RowVec<F>::type &r, float *f);
template <>
__device__ __forceinline__ void unpack<1>(const float &r, float *f) { f[0] = r; }
template <>
__device__ __forceinline__ void unpack<2>(const float2 &r, float *f) { f[0] = r.x; f[1] = r.y; }
template <>
__device__ __forceinline__ void unpack<4>(const float4 &r, float *f) {
  f[0] = r.x; f[1] = r.y; f[2] = r.z; f[3] = r.w;
}

template <int F, int OP>
__global__ __launch_bounds__(kAdjWaves *kWave) void u_op_v_adj_kernel(
    const int32_t *__restrict__ pointer, const int32_t *__restrict__ row_of_slot,
    const int32_t *__restrict__ nbr, const float *__restrict__ u, const float *__restrict__ v,
    float *__restrict__ out, int64_t n_edges) {
  typedef typename RowVec<F>::type row_t;
  constexpr int kS = 16 / F;                 // slots per lane
  constexpr int kChunk = kWave * kS;         // slots per wavefront
  __shared__ int marks_w[kAdjWaves][kChunk];
  __shared__ float vals_w[kAdjWaves][kChunk * F];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t c0 = ((int64_t)blockIdx.x * kAdjWaves + wave) * kChunk;
  if (c0 >= n_edges) return;                 // whole wavefront; no workgroup barrier below
  const int64_t c1 = min(c0 + (int64_t)kChunk, n_edges);
  const bool full = c1 - c0 == kChunk;
  const int64_t s0 = c0 + (int64_t)lane * kS;
  int *marks = marks_w[wave];
  float *vals = vals_w[wave];

  // ---- neighbour ids of my slots (they depend on nothing) ---------------------------
  int nb[kS];
  if (full) {
#pragma unroll
    for (int q = 0; q < kS / 4; ++q) {
      const int4 t = *reinterpret_cast<const int4 *>(nbr + s0 + 4 * q);
      nb[4 * q] = t.x; nb[4 * q + 1] = t.y; nb[4 * q + 2] = t.z; nb[4 * q + 3] = t.w;
    }
  } else {
#pragma unroll
    for (int j = 0; j < kS; ++j) nb[j] = nbr[s0 + j < c1 ? s0 + j : c1 - 1];
  }
  // ---- rows: marks and v rows at the row starts inside the chunk ----------------------
  const int row_first = row_of_slot[c0], row_last = row_of_slot[c1 - 1];
#pragma unroll
  for (int q = 0; q < kS / 4; ++q)
    *reinterpret_cast<int4 *>(marks + (q * kWave + lane) * 4) = make_int4(-1, -1, -1, -1);
  __builtin_amdgcn_wave_barrier();
  for (int r = row_first + 1 + lane; r <= row_last; r += kWave) {
    const int s = pointer[r], e = pointer[r + 1];
    if (e > s) {                               // rows without edges own no slot
      const int q = (int)(s - c0);
      marks[kS == 16 ? adj_word(q) : q] = r;
      *reinterpret_cast<row_t *>(vals + adj_word(q * F)) =
          *reinterpret_cast<const row_t *>(v + (int64_t)r * F);
    }
  }
  __builtin_amdgcn_wave_barrier();
  int mk[kS];
  if (kS == 16) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int4 t = *reinterpret_cast<const int4 *>(marks + adj_unit(lane, q));
      mk[(4 * q) % kS] = t.x; mk[(4 * q + 1) % kS] = t.y;
      mk[(4 * q + 2) % kS] = t.z; mk[(4 * q + 3) % kS] = t.w;
    }
  } else {
#pragma unroll
    for (int q = 0; q < kS / 4; ++q) {
      const int4 t = *reinterpret_cast<const int4 *>(marks + lane * kS + 4 * q);
      mk[4 * q] = t.x; mk[4 * q + 1] = t.y; mk[4 * q + 2] = t.z; mk[4 * q + 3] = t.w;
    }
  }
  float vt[16];                                // my 16 words of the v tile
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const float4 t = *reinterpret_cast<const float4 *>(vals + adj_unit(lane, q));
    vt[4 * q] = t.x; vt[4 * q + 1] = t.y; vt[4 * q + 2] = t.z; vt[4 * q + 3] = t.w;
  }
  int last = -1;
#pragma unroll
  for (int j = 0; j < kS; ++j) last = max(last, mk[j]);
  int inc = last;                              // largest mark of lanes <= me
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const int t = __shfl_up(inc, off);
    if (lane >= off) inc = max(inc, t);
  }
  int before = __shfl_up(inc, 1);
  before = lane >= 1 ? max(before, row_first) : row_first;
  // the row that is open at my first slot: its v row straight from memory
  float cur[F];
  unpack<F>(*reinterpret_cast<const row_t *>(v + (int64_t)before * F), cur);
  // ---- u rows of my slots, the operation, 64 bytes of output ----------------------------
  float o[16];
#pragma unroll
  for (int j = 0; j < kS; ++j) {
    float uf[F];
    unpack<F>(*reinterpret_cast<const row_t *>(u + (int64_t)nb[j] * F), uf);
#pragma unroll
    for (int f = 0; f < F; ++f) {
      cur[f] = mk[j] >= 0 ? vt[j * F + f] : cur[f];
      o[j * F + f] = adj_op<OP>(uf[f], cur[f]);
    }
  }
  float *dst = out + s0 * F;
  if (full) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
      *reinterpret_cast<float4 *>(dst + 4 * q) =
          make_float4(o[4 * q], o[4 * q + 1], o[4 * q + 2], o[4 * q + 3]);
  } else {
#pragma unroll
    for (int j = 0; j < kS; ++j)
      if (s0 + j < c1) {
#pragma unroll
        for (int f = 0; f < F; ++f) dst[j * F + f] = o[j * F + f];
      }
  }
}

template <int F, int OP>
int launch_adj(const int32_t *pointer, const int32_t *row_of_slot, const int32_t *nbr,
               const float *u, const float *v, float *out, int64_t n_edges, hipStream_t s) {
  constexpr int kChunk = kWave * (16 / F);
  const int64_t chunks = (n_edges + kChunk - 1) / kChunk;
  const int64_t blocks = (chunks + kAdjWaves - 1) / kAdjWaves;
  if (blocks > 0x7fffffff) return GA_EUNSUPPORTED;
  hipLaunchKernelGGL((u_op_v_adj_kernel<F, OP>), dim3((unsigned)blocks), dim3(kAdjWaves * kWave), 0,
                     s, pointer, row_of_slot, nbr, u, v, out, n_edges);
  return launch_status();
}

template <int F>
int launch_adj_op(int op, const int32_t *pointer, const int32_t *row_of_slot,
                  const int32_t *nbr, const float *u, const float *v, float *out,
                  int64_t n_edges, hipStream_t s) {
  switch (op) {
    case GA_SDDMM_SUB: return launch_adj<F, GA_SDDMM_SUB>(pointer, row_of_slot, nbr, u, v, out, n_edges, s);
    case GA_SDDMM_MUL: return launch_adj<F, GA_SDDMM_MUL>(pointer, row_of_slot, nbr, u, v, out, n_edges, s);
    case GA_SDDMM_DIV: return launch_adj<F, GA_SDDMM_DIV>(pointer, row_of_slot, nbr, u, v, out, n_edges, s);
    default: return launch_adj<F, GA_SDDMM_ADD>(pointer, row_of_slot, nbr, u, v, out, n_edges, s);
  }
}

}  // namespace
}  // namespace ga

extern "C" {

int ga_sddmm_u_op_v_adj(const int32_t *pointer, const int32_t *row_of_slot, const int32_t *nbr,
                        const float *u, const float *v, float *out, int64_t n_rows,
                        int64_t n_edges, int64_t feat, int op, ga_stream_t stream) {
  using namespace ga;
  if (n_rows < 0 || n_edges < 0 || n_rows > 0x7fffffff || n_edges > 0x7fffffff) return GA_EINVAL;
  if (op < GA_SDDMM_ADD || op > GA_SDDMM_DIV) return GA_EINVAL;
  if (feat != 1 && feat != 2 && feat != 4) return GA_EUNSUPPORTED;
  if (n_edges == 0) return GA_OK;
  if (n_rows == 0 || !pointer || !row_of_slot || !nbr || !u || !v || !out) return GA_EINVAL;
  if (!aligned(pointer, 4) || !aligned(row_of_slot, 4)) return GA_EALIGN;
  // 16-byte index reads and output writes, whole-row reads of u and v
  if (!aligned(nbr, 16) || !aligned(out, 16) || !aligned(u, 4 * (size_t)feat) ||
      !aligned(v, 4 * (size_t)feat))
    return GA_EALIGN;
  hipStream_t s = (hipStream_t)stream;
  if (feat == 1) return launch_adj_op<1>(op, pointer, row_of_slot, nbr, u, v, out, n_edges, s);
  if (feat == 2) return launch_adj_op<2>(op, pointer, row_of_slot, nbr, u, v, out, n_edges, s);
  return launch_adj_op<4>(op, pointer, row_of_slot, nbr, u, v, out, n_edges, s);
}

}  // extern "C"
