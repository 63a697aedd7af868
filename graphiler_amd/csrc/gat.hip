// Fused GAT aggregation for gfx950: u_add_v -> leaky_relu -> edge softmax ->
// u_mul_e sum in one pass over the in-adjacency, nothing per-edge materialised.
//
// Same run-based schedule as the SpMM (row_runs.h: equal runs of slots, one lane
// group per run, rows shared between runs chained in LDS and, across
// workgroups, by a second kernel), with an online softmax state per lane:
// running maximum m, running denominator l and the un-normalised weighted sum
// acc.  Two states merge as
//   M = max(m1, m2); l = l1 e^(m1-M) + l2 e^(m2-M); acc likewise,
// so partial rows combine exactly like partial sums, in run order.
//
// The same pass with per-edge operands (EDGE): the logits are given per edge
// and the weighted rows are per-edge rows, both read through the edge-id
// column: out[v] = sum_e softmax_v(logit)[e] * m[e], the SegmentSoftmax ->
// mul -> SpMMEdge tail of examples/HGT/HGT.py:50-53 with no attention tensor.
#include <mutex>

#include "row_runs.h"

namespace ga {
namespace {

__device__ __forceinline__ float leaky(float t, float slope) {
  return t >= 0.0f ? t : t * slope;
}

// The running maximum as the point the exponentials are taken from: while every
// logit seen so far is -inf (masked edges) the maximum is -inf too and
// exp(-inf - -inf) would be NaN; taken from 0 instead, such edges weigh 0 and a
// later finite logit rescales the (empty) state by exp(-inf) = 0.  A row whose
// logits are all -inf ends with a zero denominator and yields NaN, as the
// reference's softmax does (segment_softmax_kernel.cu:9-49).
__device__ __forceinline__ float finite_or_zero(float m) {
  return m == -INFINITY ? 0.0f : m;
}

// State per lane: VEC un-normalised weighted sums, then the running maximum m
// and the running denominator l of the lane's head.
// MODE selects where the logits come from:
//   kGatNode  el[src] + er[dst] through leaky_relu (the GAT chain),
//   kGatEdge  given per edge (EDGE operands, see the header comment),
//   kGatFromZ <z[src, h, :], a_l[h, :]> + er[dst] through leaky_relu: the source
//             term is recomputed from the row that is gathered anyway instead of
//             being gathered itself -- a separate (N, heads) table costs one more
//             memory sector per edge once it no longer fits the caches.
constexpr int kGatNode = 0, kGatEdge = 1, kGatFromZ = 2;

// Sum over `lanes` adjacent lanes (a power of two <= 16, aligned), in every lane.
__device__ __forceinline__ float lanes_sum(float v, int lanes) {
  if (lanes >= 2) v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xF, 0xF, true));
  if (lanes >= 4) v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xF, 0xF, true));
  if (lanes >= 8) v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x141, 0xF, 0xF, true));
  if (lanes >= 16) v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x140, 0xF, 0xF, true));
  return v;
}

// SPREAD: the lane's features lie a lane-group width apart (rows that 16-byte
// accesses do not tile); they share the lane's one (m, l) pair, i.e. one head.
// ACT: the activation compiled into the row store (GA_ACT_RELU / GA_ACT_ELU), or
// kActRuntime = the one named by Args::act (the less common lane layouts; one build
// for all three).  The compiled-in forms keep the dead branches out of the kernel:
// the store sits at five places of the run loop, under divergence, so its length is
// paid once per closed row and wavefront, not per element.
constexpr int kActRuntime = -1;
template <typename T, int VEC, int MODE = kGatNode, bool SPREAD = false, int ACT = kActRuntime>
struct GatPolicy {
  static constexpr bool EDGE = MODE == kGatEdge;
  typedef T out_t;
  static constexpr int kVec = VEC;
  static constexpr int kState = VEC + 2;
  static constexpr bool kSpread = SPREAD;
  struct Args {
    const int32_t *nbr;   // kGatEdge: the edge-id column, or null when slot = edge id
    const float *el;      // kGatEdge: per-edge logits (E, heads); kGatFromZ: a_l (heads*dph)
    const float *er;      // kGatEdge: unused
    const T *z;           // kGatEdge: per-edge rows (E, heads*dph)
    int heads;
    int dph;
    float slope;
    bool ids_vec;   // row_of_slot and nbr are 16-byte aligned
    int head_lanes; // kGatFromZ: lanes that share a head (dph / VEC)
    int stride_shift;   // SPREAD: log2 of the lanes per group, set by the launcher
    int act;            // GA_ACT_*: applied to the finished row before it is stored
  };
  static __device__ __forceinline__ void init(float (&st)[VEC + 2]) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) st[v] = 0.0f;
    st[VEC] = -INFINITY;
    st[VEC + 1] = 0.0f;
  }
  static __device__ __forceinline__ void merge(float (&dst)[VEC + 2], const float *src) {
    const float nm = fmaxf(dst[VEC], src[VEC]);
    const float ref = finite_or_zero(nm);
    const float sa = __expf(dst[VEC] - ref), sb = __expf(src[VEC] - ref);
#pragma unroll
    for (int v = 0; v < VEC; ++v) dst[v] = dst[v] * sa + src[v] * sb;
    dst[VEC + 1] = dst[VEC + 1] * sa + src[VEC + 1] * sb;
    dst[VEC] = nm;
  }
  static __device__ __forceinline__ void finish(const float (&st)[VEC + 2], float (&o)[VEC]) {
    const float inv = 1.0f / st[VEC + 1];
#pragma unroll
    for (int v = 0; v < VEC; ++v) o[v] = st[v] * inv;
  }
  static __device__ __forceinline__ void empty_row(float (&o)[VEC]) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) o[v] = 0.0f;
  }
  static __device__ __forceinline__ void emit(const Args &A, out_t *out, int64_t row, int feat,
                                              int f0, const float (&st)[kState]) {
    const int act = ACT == kActRuntime ? A.act : ACT;
    if (act == GA_ACT_NONE) {
      emit_row<GatPolicy>(out, row, feat, f0, st, A.stride_shift);
      return;
    }
    // the activation of the layer (relu, or elu with alpha = 1) on the fp32 row, before
    // it is rounded and stored: the row is not written and read again for it
    typedef RowIO<out_t, VEC, SPREAD> IO;
    float o[VEC];
    finish(st, o);
#pragma unroll
    for (int v = 0; v < VEC; ++v) o[v] = act == GA_ACT_ELU ? elu(o[v]) : relu_keep_nan(o[v]);
    IO::store(out + row * feat + f0, o, IO::lane(A.stride_shift, feat - f0));
  }
  static __device__ __forceinline__ void emit_empty(const Args &A, out_t *out, int64_t row,
                                                    int feat, int f0) {
    emit_empty_row<GatPolicy>(out, row, feat, f0, A.stride_shift);
  }

  template <class Close>
  static __device__ __forceinline__ void walk(const Args &A,
                                              const int32_t *__restrict__ row_of_slot,
                                              int64_t a, int64_t b, int f0, int feat,
                                              float (&st)[VEC + 2], int &cur,
                                              Close &&close_segment) {
    static_assert(!(SPREAD && MODE == kGatFromZ), "the per-head dot product needs consecutive features");
    typedef RowIO<T, VEC, SPREAD> IO;
    const typename IO::lane_t ln = IO::lane(A.stride_shift, feat - f0);
    const int h = SPREAD ? 0 : f0 / A.dph;
    float al[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) al[v] = MODE == kGatFromZ ? A.el[f0 + v] : 0.0f;
    for (int64_t j = a; j < b; j += kUnroll) {
      int r[kUnroll], g[kUnroll];
      float s[kUnroll];
      typename IO::raw_t x[kUnroll];
      load_ids8(row_of_slot, j, b, A.ids_vec, r);
      if (EDGE && !A.nbr) {
#pragma unroll
        for (int t = 0; t < kUnroll; ++t) g[t] = (int)(j + t < b ? j + t : b - 1);
      } else {
        load_ids8(A.nbr, j, b, A.ids_vec, g);
      }
#pragma unroll
      for (int t = 0; t < kUnroll; ++t) {
        x[t] = IO::load(A.z + (int64_t)g[t] * feat + f0, ln);
        if constexpr (MODE == kGatEdge)
          s[t] = A.el[(int64_t)g[t] * A.heads + h];
        else if constexpr (MODE == kGatNode)
          s[t] = leaky(A.el[(int64_t)g[t] * A.heads + h] + A.er[(int64_t)r[t] * A.heads + h],
                       A.slope);
        else
          s[t] = A.er[(int64_t)r[t] * A.heads + h];
      }
      if constexpr (MODE == kGatFromZ) {
        // every live lane of a head runs this together (heads tile the row)
#pragma unroll
        for (int t = 0; t < kUnroll; ++t) {
          float xf[VEC];
          IO::widen(x[t], xf);
          float d = 0.0f;
#pragma unroll
          for (int v = 0; v < VEC; ++v) d = fmaf(xf[v], al[v], d);
          s[t] = leaky(lanes_sum(d, A.head_lanes) + s[t], A.slope);
        }
      }
      const bool one_row = j + kUnroll <= b && r[0] == cur && r[kUnroll - 1] == cur;
      if (one_row) {
        // whole batch inside the open row (rows are sorted): one rescale
        float bm = s[0];
#pragma unroll
        for (int t = 1; t < kUnroll; ++t) bm = fmaxf(bm, s[t]);
        const float nm = fmaxf(st[VEC], bm);
        const float ref = finite_or_zero(nm);
        const float sc = __expf(st[VEC] - ref);
        st[VEC + 1] *= sc;
#pragma unroll
        for (int v = 0; v < VEC; ++v) st[v] *= sc;
        st[VEC] = nm;
#pragma unroll
        for (int t = 0; t < kUnroll; ++t) {
          const float p = __expf(s[t] - ref);
          st[VEC + 1] += p;
          float xf[VEC];
          IO::widen(x[t], xf);
#pragma unroll
          for (int v = 0; v < VEC; ++v) st[v] = fmaf(p, xf[v], st[v]);
        }
      } else {
#pragma unroll
        for (int t = 0; t < kUnroll; ++t) {
          if (j + t < b) {
            if (r[t] != cur) {
              close_segment();
              cur = r[t];
              init(st);
            }
            const float nm = fmaxf(st[VEC], s[t]);
            const float ref = finite_or_zero(nm);
            const float sc = __expf(st[VEC] - ref);
            const float p = __expf(s[t] - ref);
            st[VEC + 1] = st[VEC + 1] * sc + p;
            float xf[VEC];
            IO::widen(x[t], xf);
#pragma unroll
            for (int v = 0; v < VEC; ++v) st[v] = fmaf(p, xf[v], st[v] * sc);
            st[VEC] = nm;
          }
        }
      }
    }
  }
};

// Dot-product attention over an adjacency: slot i of row r weighs the value row
// v[nbr[i]] with softmax_r(<k[nbr[i]], q[qrow[i]]>), per head; beside the weighted sum
// the row's log-sum-exp is written, so that rows which are pieces of one softmax (the
// (destination, relation) pairs of an HGT layer) can be combined afterwards.  State,
// merge and finish are the fused GAT aggregation's; only the logits differ: a second
// gathered row (k) and the slot's query row, which consecutive slots of a pair share.
template <typename T, int VEC>
struct DotAttnPolicy : GatPolicy<T, VEC, kGatEdge, false> {
  typedef GatPolicy<T, VEC, kGatEdge, false> Base;
  struct Args {
    const int32_t *nbr;    // key / value row of a slot
    const int32_t *qrow;   // query row of a slot
    const T *k, *q, *v;    // rows of heads * dph features
    float *lse;            // (n_rows, heads) or null
    const int32_t *lse_index;   // row r's log-sum-exp goes to row lse_index[r] of lse; null: r
    int heads;
    int dph;
    int head_lanes;        // lanes that share a head (dph / VEC)
    bool ids_vec;          // row_of_slot, nbr and qrow are 16-byte aligned
  };
  static __device__ __forceinline__ void emit(const Args &A, T *out, int64_t row, int feat, int f0,
                                              const float (&st)[VEC + 2]) {
    emit_row<DotAttnPolicy>(out, row, feat, f0, st);
    if (A.lse && f0 % A.dph == 0)
      A.lse[(A.lse_index ? (int64_t)A.lse_index[row] : row) * A.heads + f0 / A.dph] =
          st[VEC] + logf(st[VEC + 1]);
  }
  static __device__ __forceinline__ void emit_empty(const Args &A, T *out, int64_t row, int feat,
                                                    int f0) {
    emit_empty_row<DotAttnPolicy>(out, row, feat, f0);
    if (A.lse && f0 % A.dph == 0)
      A.lse[(A.lse_index ? (int64_t)A.lse_index[row] : row) * A.heads + f0 / A.dph] = -INFINITY;
  }

  template <class Close>
  static __device__ __forceinline__ void walk(const Args &A,
                                              const int32_t *__restrict__ row_of_slot,
                                              int64_t a, int64_t b, int f0, int feat,
                                              float (&st)[VEC + 2], int &cur,
                                              Close &&close_segment) {
    typedef RowIO<T, VEC, false> IO;
    const typename IO::lane_t ln = IO::lane(0, feat - f0);
    for (int64_t j = a; j < b; j += kUnroll) {
      int r[kUnroll], g[kUnroll], qr[kUnroll];
      float s[kUnroll];
      typename IO::raw_t x[kUnroll], kx[kUnroll], qx[kUnroll];
      load_ids8(row_of_slot, j, b, A.ids_vec, r);
      load_ids8(A.nbr, j, b, A.ids_vec, g);
      load_ids8(A.qrow, j, b, A.ids_vec, qr);
#pragma unroll
      for (int t = 0; t < kUnroll; ++t) {
        kx[t] = IO::load(A.k + (int64_t)g[t] * feat + f0, ln);
        qx[t] = IO::load(A.q + (int64_t)qr[t] * feat + f0, ln);
        x[t] = IO::load(A.v + (int64_t)g[t] * feat + f0, ln);
      }
      // every live lane of a head runs this together (heads tile the row)
#pragma unroll
      for (int t = 0; t < kUnroll; ++t) {
        float kf[VEC], qf[VEC];
        IO::widen(kx[t], kf);
        IO::widen(qx[t], qf);
        float d = 0.0f;
#pragma unroll
        for (int v = 0; v < VEC; ++v) d = fmaf(kf[v], qf[v], d);
        s[t] = lanes_sum(d, A.head_lanes);
      }
      const bool one_row = j + kUnroll <= b && r[0] == cur && r[kUnroll - 1] == cur;
      if (one_row) {
        // whole batch inside the open row (rows are sorted): one rescale
        float bm = s[0];
#pragma unroll
        for (int t = 1; t < kUnroll; ++t) bm = fmaxf(bm, s[t]);
        const float nm = fmaxf(st[VEC], bm);
        const float ref = finite_or_zero(nm);
        const float sc = __expf(st[VEC] - ref);
        st[VEC + 1] *= sc;
#pragma unroll
        for (int v = 0; v < VEC; ++v) st[v] *= sc;
        st[VEC] = nm;
#pragma unroll
        for (int t = 0; t < kUnroll; ++t) {
          const float p = __expf(s[t] - ref);
          st[VEC + 1] += p;
          float xf[VEC];
          IO::widen(x[t], xf);
#pragma unroll
          for (int v = 0; v < VEC; ++v) st[v] = fmaf(p, xf[v], st[v]);
        }
      } else {
#pragma unroll
        for (int t = 0; t < kUnroll; ++t) {
          if (j + t < b) {
            if (r[t] != cur) {
              close_segment();
              cur = r[t];
              Base::init(st);
            }
            const float nm = fmaxf(st[VEC], s[t]);
            const float ref = finite_or_zero(nm);
            const float sc = __expf(st[VEC] - ref);
            const float p = __expf(s[t] - ref);
            st[VEC + 1] = st[VEC + 1] * sc + p;
            float xf[VEC];
            IO::widen(x[t], xf);
#pragma unroll
            for (int v = 0; v < VEC; ++v) st[v] = fmaf(p, xf[v], st[v] * sc);
            st[VEC] = nm;
          }
        }
      }
    }
  }
};

template <typename T, int VEC>
int launch_dot_attn(const int32_t *pointer, const int32_t *row_of_slot, const int32_t *nbr,
                    const int32_t *qrow, const void *k, const void *q, const void *v, void *out,
                    float *lse, const int32_t *lse_index, int64_t n_rows, int64_t n_edges, int heads,
                    int dim, float *ws, size_t ws_bytes, hipStream_t stream) {
  typedef DotAttnPolicy<T, VEC> P;
  const int head_lanes = dim / VEC;
  if (dim % VEC != 0 || head_lanes > 16 || (head_lanes & (head_lanes - 1)) != 0)
    return GA_EUNSUPPORTED;
  const bool ids_vec = aligned(row_of_slot, 16) && aligned(nbr, 16) && aligned(qrow, 16);
  typename P::Args args{nbr, qrow, (const T *)k, (const T *)q, (const T *)v, lse, lse_index,
                        heads, dim, head_lanes, ids_vec};
  return launch_runs<P>(args, pointer, row_of_slot, out, n_rows, n_edges, heads * dim, ws,
                        stream, ws_bytes);
}

template <typename T, int VEC, int MODE = kGatNode, bool SPREAD = false, int ACT = kActRuntime>
int launch_gat(const int32_t *pointer, const int32_t *row_of_slot,
               const int32_t *nbr, const float *el, const float *er,
               const void *z, void *out, int64_t n_rows, int64_t n_edges,
               int heads, int dim, float slope, float *ws, hipStream_t stream,
               size_t ws_bytes = SIZE_MAX, int act = GA_ACT_NONE, size_t *size_only = nullptr) {
  // the 16-byte lane layouts of the node forms (every benchmarked shape) get a build per
  // activation; everything else reads it from the arguments
  if constexpr (ACT == kActRuntime && !SPREAD && MODE != kGatEdge && VEC > 1) {
    if (act == GA_ACT_NONE)
      return launch_gat<T, VEC, MODE, SPREAD, GA_ACT_NONE>(pointer, row_of_slot, nbr, el, er, z, out,
                                                           n_rows, n_edges, heads, dim, slope, ws,
                                                           stream, ws_bytes, act, size_only);
    if (act == GA_ACT_RELU)
      return launch_gat<T, VEC, MODE, SPREAD, GA_ACT_RELU>(pointer, row_of_slot, nbr, el, er, z, out,
                                                           n_rows, n_edges, heads, dim, slope, ws,
                                                           stream, ws_bytes, act, size_only);
    return launch_gat<T, VEC, MODE, SPREAD, GA_ACT_ELU>(pointer, row_of_slot, nbr, el, er, z, out,
                                                        n_rows, n_edges, heads, dim, slope, ws, stream,
                                                        ws_bytes, act, size_only);
  }
  typedef GatPolicy<T, VEC, MODE, SPREAD, ACT> P;
  const bool ids_vec = aligned(row_of_slot, 16) && (!nbr || aligned(nbr, 16));
  const int head_lanes = dim / VEC;
  if (MODE == kGatFromZ &&
      (dim % VEC != 0 || head_lanes > 16 || (head_lanes & (head_lanes - 1)) != 0))
    return GA_EUNSUPPORTED;
  typename P::Args args{nbr, el, er, (const T *)z, heads, dim, slope, ids_vec, head_lanes, 0, act};
  return launch_runs<P>(args, pointer, row_of_slot, out, n_rows, n_edges,
                        heads * dim, ws, stream, ws_bytes, size_only);
}

// The element type and lane layout ga_gat_aggregate runs for a shape, launched
// with `ws` (capacity `ws_bytes`) as the partial-row scratch.
int gat_aggregate_dispatch(const int32_t *pointer, const int32_t *row_of_slot,
                           const int32_t *nbr, const float *el, const float *er,
                           const void *z, void *out, int64_t n_rows, int64_t n_edges,
                           int heads, int dim, float slope, int dtype, float *ws,
                           size_t ws_bytes, hipStream_t s, int act = GA_ACT_NONE,
                           size_t *size_only = nullptr) {
  const bool vec_ok = aligned(out, 16) && (!z || aligned(z, 16));
  if (dtype == GA_F32) {
    if (vec_ok && dim % 4 == 0)
      return launch_gat<float, 4>(pointer, row_of_slot, nbr, el, er, z, out, n_rows, n_edges,
                                  heads, dim, slope, ws, s, ws_bytes, act, size_only);
    if (heads == 1 && dim >= 3 && dim <= 256)   // rows that 16-byte accesses do not tile
      return launch_gat<float, 4, kGatNode, true>(pointer, row_of_slot, nbr, el, er, z, out,
                                                  n_rows, n_edges, 1, dim, slope, ws, s, ws_bytes, act, size_only);
    return launch_gat<float, 1>(pointer, row_of_slot, nbr, el, er, z, out, n_rows, n_edges,
                                heads, dim, slope, ws, s, ws_bytes, act, size_only);
  }
  if (vec_ok && dim % 8 == 0)
    return launch_gat<bf16_t, 8>(pointer, row_of_slot, nbr, el, er, z, out, n_rows, n_edges,
                                 heads, dim, slope, ws, s, ws_bytes, act, size_only);
  if (heads == 1 && dim >= 3 && dim <= 256)
    return launch_gat<bf16_t, 4, kGatNode, true>(pointer, row_of_slot, nbr, el, er, z, out,
                                                 n_rows, n_edges, 1, dim, slope, ws, s, ws_bytes, act, size_only);
  return launch_gat<bf16_t, 1>(pointer, row_of_slot, nbr, el, er, z, out, n_rows, n_edges,
                               heads, dim, slope, ws, s, ws_bytes, act, size_only);
}

// Argument checks shared by ga_gat_aggregate and ga_gat_aggregate_static
// (everything but the workspace).  GA_OK with *nothing_to_do set for n_rows == 0.
int gat_aggregate_check(const int32_t *pointer, const int32_t *row_of_slot,
                        const int32_t *nbr, const float *el, const float *er,
                        const void *z, const void *out, int64_t n_rows, int64_t n_edges,
                        int64_t heads, int64_t dim, int dtype, bool *nothing_to_do) {
  *nothing_to_do = false;
  if (n_rows < 0 || n_edges < 0 || heads <= 0 || dim <= 0) return GA_EINVAL;
  if (n_rows > 0x7fffffff || n_edges > 0x7fffffff || heads * dim > 0x7fffffff)
    return GA_EINVAL;
  if (dtype != GA_F32 && dtype != GA_BF16) return GA_EINVAL;
  if (n_rows == 0) {
    *nothing_to_do = true;
    return GA_OK;
  }
  if (!pointer || !out) return GA_EINVAL;
  if (n_edges > 0 && (!row_of_slot || !nbr || !el || !er || !z)) return GA_EINVAL;
  const size_t esz = dtype == GA_F32 ? 4 : 2;
  if (!aligned(out, esz) || (z && !aligned(z, esz)) || (el && !aligned(el, 4)) ||
      (er && !aligned(er, 4)))
    return GA_EALIGN;
  return GA_OK;
}

// Scratch of ga_gat_aggregate_static: the partial rows that ga_gat_aggregate
// takes as its workspace, held by the library itself.  Every device the library
// runs on has its own copy of this array at its own address; host code never
// uses the array's name as an address, only the pointer that
// hipGetSymbolAddress returned for the current device (static_scratch_for).
static __device__ __align__(256) unsigned char scratch[GA_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::mutex scratch_mutex;
void *scratch_ptr[kMaxDevices];   // per device, filled on the first call there

int static_scratch_for_current_device(void **ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return GA_EUNSUPPORTED;
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (!scratch_ptr[dev]) {
    void *p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!p) return GA_EINVAL;
    scratch_ptr[dev] = p;
  }
  *ptr = scratch_ptr[dev];
  return GA_OK;
}

}  // namespace
}  // namespace ga

extern "C" {

size_t ga_gat_workspace_bytes(int64_t n_edges, int64_t feat, int64_t heads) {
  if (heads <= 0) return 0;
  // up to three state floats per feature (scalar path: sum, max, denominator)
  return ga::runs_workspace_bytes(n_edges, feat, 3);
}

int ga_gat_aggregate(const int32_t *pointer, const int32_t *row_of_slot,
                     const int32_t *nbr, const float *el, const float *er,
                     const void *z, void *out, int64_t n_rows, int64_t n_edges,
                     int64_t heads, int64_t dim, float slope, int dtype,
                     void *workspace, size_t workspace_bytes,
                     ga_stream_t stream) {
  return ga_gat_aggregate_act(pointer, row_of_slot, nbr, el, er, z, out, n_rows, n_edges, heads,
                              dim, slope, GA_ACT_NONE, dtype, workspace, workspace_bytes, stream);
}

int ga_gat_aggregate_act(const int32_t *pointer, const int32_t *row_of_slot,
                         const int32_t *nbr, const float *el, const float *er,
                         const void *z, void *out, int64_t n_rows, int64_t n_edges,
                         int64_t heads, int64_t dim, float slope, int activation, int dtype,
                         void *workspace, size_t workspace_bytes, ga_stream_t stream) {
  if (activation < GA_ACT_NONE || activation > GA_ACT_ELU) return GA_EINVAL;
  bool nothing = false;
  const int rc = ga::gat_aggregate_check(pointer, row_of_slot, nbr, el, er, z, out, n_rows,
                                         n_edges, heads, dim, dtype, &nothing);
  if (rc != GA_OK || nothing) return rc;
  if (n_edges > 0 &&
      (!workspace || !ga::aligned(workspace, 16) ||
       ga_gat_workspace_bytes(n_edges, heads * dim, heads) > workspace_bytes))
    return GA_EWORKSPACE;
  return ga::gat_aggregate_dispatch(pointer, row_of_slot, nbr, el, er, z, out, n_rows, n_edges,
                                    (int)heads, (int)dim, slope, dtype, (float *)workspace,
                                    workspace_bytes, (hipStream_t)stream, activation);
}

int ga_gat_aggregate_static(const int32_t *pointer, const int32_t *row_of_slot,
                            const int32_t *nbr, const float *el, const float *er,
                            const void *z, void *out, int64_t n_rows, int64_t n_edges,
                            int64_t heads, int64_t dim, float slope, int dtype,
                            ga_stream_t stream) {
  bool nothing = false;
  const int rc = ga::gat_aggregate_check(pointer, row_of_slot, nbr, el, er, z, out, n_rows,
                                         n_edges, heads, dim, dtype, &nothing);
  if (rc != GA_OK || nothing) return rc;
  void *ws = nullptr;
  const int sc = ga::static_scratch_for_current_device(&ws);
  if (sc != GA_OK) return sc;
  // The kernels write every partial row before the fix-up pass reads it, so the
  // previous call's contents need no clearing.
  const int lr = ga::gat_aggregate_dispatch(pointer, row_of_slot, nbr, el, er, z, out, n_rows,
                                            n_edges, (int)heads, (int)dim, slope, dtype,
                                            (float *)ws, (size_t)GA_STATIC_SCRATCH_BYTES,
                                            (hipStream_t)stream);
  return lr == GA_EWORKSPACE ? GA_ESCRATCH : lr;
}

int64_t ga_gat_static_scratch_needed(int64_t n_edges, int64_t heads, int64_t dim, int dtype,
                                     int rows_16_byte_aligned) {
  if (n_edges < 0 || heads <= 0 || dim <= 0 || n_edges > 0x7fffffff ||
      heads * dim > 0x7fffffff || (dtype != GA_F32 && dtype != GA_BF16))
    return GA_EINVAL;
  if (n_edges == 0) return 0;
  // the dispatch itself, asked for the size of the layout it would launch: the two
  // addresses below only carry the alignment and are never dereferenced
  const void *row = (const void *)(uintptr_t)(rows_16_byte_aligned ? 16 : (dtype == GA_F32 ? 4 : 2));
  size_t needed = 0;
  const int rc = ga::gat_aggregate_dispatch(nullptr, nullptr, nullptr, nullptr, nullptr, row,
                                            (void *)row, 1, n_edges, (int)heads, (int)dim, 0.0f,
                                            dtype, nullptr, 0, nullptr, GA_ACT_NONE, &needed);
  return rc == GA_OK ? (int64_t)needed : (int64_t)rc;
}

int ga_edge_softmax_sum(const int32_t *pointer, const int32_t *row_of_slot,
                        const int32_t *eid, const float *logit, const void *m,
                        void *out, int64_t n_rows, int64_t n_edges, int64_t heads,
                        int64_t dim, int dtype, void *workspace,
                        size_t workspace_bytes, ga_stream_t stream) {
  if (n_rows < 0 || n_edges < 0 || heads <= 0 || dim <= 0) return GA_EINVAL;
  if (n_rows > 0x7fffffff || n_edges > 0x7fffffff || heads * dim > 0x7fffffff)
    return GA_EINVAL;
  if (dtype != GA_F32 && dtype != GA_BF16) return GA_EINVAL;
  if (n_rows == 0) return GA_OK;
  if (!pointer || !out) return GA_EINVAL;
  const int64_t feat = heads * dim;
  if (n_edges > 0) {
    if (!row_of_slot || !logit || !m) return GA_EINVAL;
    if (!workspace || !ga::aligned(workspace, 16) ||
        ga_gat_workspace_bytes(n_edges, feat, heads) > workspace_bytes)
      return GA_EWORKSPACE;
  }
  const size_t esz = dtype == GA_F32 ? 4 : 2;
  if (!ga::aligned(out, esz) || (m && !ga::aligned(m, esz)) ||
      (logit && !ga::aligned(logit, 4)))
    return GA_EALIGN;
  const bool vec_ok = ga::aligned(out, 16) && (!m || ga::aligned(m, 16));
  hipStream_t s = (hipStream_t)stream;
  float *ws = (float *)workspace;
  const int h = (int)heads, d = (int)dim;
  if (dtype == GA_F32) {
    if (vec_ok && dim % 4 == 0)
      return ga::launch_gat<float, 4, ga::kGatEdge>(pointer, row_of_slot, eid, logit, nullptr, m,
                                            out, n_rows, n_edges, h, d, 0.0f, ws, s);
    if (heads == 1 && dim >= 3 && dim <= 256)   // rows that 16-byte accesses do not tile
      return ga::launch_gat<float, 4, ga::kGatEdge, true>(pointer, row_of_slot, eid, logit, nullptr,
                                                          m, out, n_rows, n_edges, 1, d, 0.0f, ws, s);
    return ga::launch_gat<float, 1, ga::kGatEdge>(pointer, row_of_slot, eid, logit, nullptr, m, out,
                                          n_rows, n_edges, h, d, 0.0f, ws, s);
  }
  if (vec_ok && dim % 8 == 0)
    return ga::launch_gat<ga::bf16_t, 8, ga::kGatEdge>(pointer, row_of_slot, eid, logit, nullptr, m,
                                               out, n_rows, n_edges, h, d, 0.0f, ws, s);
  if (heads == 1 && dim >= 3 && dim <= 256)
    return ga::launch_gat<ga::bf16_t, 4, ga::kGatEdge, true>(pointer, row_of_slot, eid, logit, nullptr,
                                                             m, out, n_rows, n_edges, 1, d, 0.0f, ws, s);
  return ga::launch_gat<ga::bf16_t, 1, ga::kGatEdge>(pointer, row_of_slot, eid, logit, nullptr, m,
                                             out, n_rows, n_edges, h, d, 0.0f, ws, s);
}

int ga_dot_attention_sum(const int32_t *pointer, const int32_t *row_of_slot,
                         const int32_t *nbr, const int32_t *qrow, const void *k, const void *q,
                         const void *v, void *out, float *lse, const int32_t *lse_index,
                         int64_t n_rows, int64_t n_edges, int64_t heads, int64_t dim, int dtype,
                         void *workspace, size_t workspace_bytes, ga_stream_t stream) {
  if (n_rows < 0 || n_edges < 0 || heads <= 0 || dim <= 0) return GA_EINVAL;
  if (n_rows > 0x7fffffff || n_edges > 0x7fffffff || heads * dim > 0x7fffffff)
    return GA_EINVAL;
  if (dtype != GA_F32 && dtype != GA_BF16) return GA_EINVAL;
  if (n_rows == 0) return GA_OK;
  if (!pointer || !out) return GA_EINVAL;
  const int64_t feat = heads * dim;
  if (n_edges > 0) {
    if (!row_of_slot || !nbr || !qrow || !k || !q || !v) return GA_EINVAL;
    if (!workspace || !ga::aligned(workspace, 16) ||
        ga_gat_workspace_bytes(n_edges, feat, heads) > workspace_bytes)
      return GA_EWORKSPACE;
  }
  if ((lse && !ga::aligned(lse, 4)) || (lse_index && !ga::aligned(lse_index, 4))) return GA_EALIGN;
  if (lse_index && !lse) return GA_EINVAL;
  // rows are read and written in 16-byte pieces that do not straddle a head
  const int vec = dtype == GA_F32 ? 4 : 8;
  if (!ga::aligned(out, 16) || (k && !ga::aligned(k, 16)) || (q && !ga::aligned(q, 16)) ||
      (v && !ga::aligned(v, 16)) || dim % vec != 0)
    return GA_EUNSUPPORTED;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == GA_F32)
    return ga::launch_dot_attn<float, 4>(pointer, row_of_slot, nbr, qrow, k, q, v, out, lse,
                                         lse_index, n_rows, n_edges, (int)heads, (int)dim,
                                         (float *)workspace, workspace_bytes, s);
  return ga::launch_dot_attn<ga::bf16_t, 8>(pointer, row_of_slot, nbr, qrow, k, q, v, out, lse,
                                            lse_index, n_rows, n_edges, (int)heads, (int)dim,
                                            (float *)workspace, workspace_bytes, s);
}

int ga_gat_aggregate_from_z(const int32_t *pointer, const int32_t *row_of_slot,
                            const int32_t *nbr, const float *a_l, const float *er,
                            const void *z, void *out, int64_t n_rows, int64_t n_edges,
                            int64_t heads, int64_t dim, float slope, int dtype,
                            void *workspace, size_t workspace_bytes, ga_stream_t stream) {
  return ga_gat_aggregate_from_z_act(pointer, row_of_slot, nbr, a_l, er, z, out, n_rows, n_edges,
                                     heads, dim, slope, GA_ACT_NONE, dtype, workspace,
                                     workspace_bytes, stream);
}

int ga_gat_aggregate_from_z_act(const int32_t *pointer, const int32_t *row_of_slot,
                                const int32_t *nbr, const float *a_l, const float *er,
                                const void *z, void *out, int64_t n_rows, int64_t n_edges,
                                int64_t heads, int64_t dim, float slope, int activation,
                                int dtype, void *workspace, size_t workspace_bytes,
                                ga_stream_t stream) {
  if (activation < GA_ACT_NONE || activation > GA_ACT_ELU) return GA_EINVAL;
  if (n_rows < 0 || n_edges < 0 || heads <= 0 || dim <= 0) return GA_EINVAL;
  if (n_rows > 0x7fffffff || n_edges > 0x7fffffff || heads * dim > 0x7fffffff)
    return GA_EINVAL;
  if (dtype != GA_F32 && dtype != GA_BF16) return GA_EINVAL;
  if (n_rows == 0) return GA_OK;
  if (!pointer || !out) return GA_EINVAL;
  const int64_t feat = heads * dim;
  if (n_edges > 0) {
    if (!row_of_slot || !nbr || !a_l || !er || !z) return GA_EINVAL;
    if (!workspace || !ga::aligned(workspace, 16) ||
        ga_gat_workspace_bytes(n_edges, feat, heads) > workspace_bytes)
      return GA_EWORKSPACE;
  }
  const size_t esz = dtype == GA_F32 ? 4 : 2;
  if (!ga::aligned(out, esz) || (z && !ga::aligned(z, esz)) ||
      (a_l && !ga::aligned(a_l, 4)) || (er && !ga::aligned(er, 4)))
    return GA_EALIGN;
  const bool vec_ok = ga::aligned(out, 16) && (!z || ga::aligned(z, 16));
  hipStream_t s = (hipStream_t)stream;
  float *ws = (float *)workspace;
  const int h = (int)heads, d = (int)dim;
  if (dtype == GA_F32) {
    if (vec_ok && dim % 4 == 0)
      return ga::launch_gat<float, 4, ga::kGatFromZ>(pointer, row_of_slot, nbr, a_l, er, z, out,
                                                     n_rows, n_edges, h, d, slope, ws, s, SIZE_MAX, activation);
    return ga::launch_gat<float, 1, ga::kGatFromZ>(pointer, row_of_slot, nbr, a_l, er, z, out,
                                                   n_rows, n_edges, h, d, slope, ws, s, SIZE_MAX, activation);
  }
  if (vec_ok && dim % 8 == 0)
    return ga::launch_gat<ga::bf16_t, 8, ga::kGatFromZ>(pointer, row_of_slot, nbr, a_l, er, z,
                                                        out, n_rows, n_edges, h, d, slope, ws, s, SIZE_MAX, activation);
  return ga::launch_gat<ga::bf16_t, 1, ga::kGatFromZ>(pointer, row_of_slot, nbr, a_l, er, z, out,
                                                      n_rows, n_edges, h, d, slope, ws, s, SIZE_MAX, activation);
}

}  // extern "C"
