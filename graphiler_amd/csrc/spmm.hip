// Load-balanced CSR SpMM for gfx950 (copy_u / copy_e / u_mul_e x sum / max / min)
// on the run-based row-reduction schedule of row_runs.h.
#include "row_runs.h"

namespace ga {

int run_shift_for(int64_t n_edges, int64_t feat) {
  // lanes a feature row occupies with 16-byte fp32 accesses
  int64_t lanes = (feat + 3) / 4;
  int lane_shift = ilog2_ceil((uint64_t)(lanes < 1 ? 1 : (lanes > 64 ? 64 : lanes)));
  // aim at >= 16k wavefronts of work, between 32 and 1024 slots per run
  int64_t per_run = (n_edges << lane_shift) / 64 / 16384;
  int shift = per_run < 1 ? 0 : ilog2_floor((uint64_t)per_run);
  if (shift < 5) shift = 5;
  if (shift > 10) shift = 10;
  return shift;
}

namespace {

template <int RED>
__device__ __forceinline__ float red_init() {
  return RED == GA_SUM ? 0.0f : (RED == GA_MAX ? -INFINITY : INFINITY);
}
template <int RED>
__device__ __forceinline__ float red_apply(float acc, float m) {
  if (RED == GA_SUM) return acc + m;
  // strict comparison: the first extremum in slot order wins, NaN never does
  if (RED == GA_MAX) return acc < m ? m : acc;
  return acc > m ? m : acc;
}

// Binary operator between the gathered feature and the edge datum
// (functor.cuh:19-100): 0 = none (copy), else GA_U_MUL_E .. GA_U_DIV_E.
template <int BOP>
__device__ __forceinline__ float bin_apply(float x, float w) {
  if (BOP == GA_U_MUL_E) return x * w;
  if (BOP == GA_U_ADD_E) return x + w;
  if (BOP == GA_U_SUB_E) return x - w;
  if (BOP == GA_U_DIV_E) return x / w;
  return x;
}

// Row-reduction policy of the SpMM: the state is the VEC running reductions.
// SPREAD: the lane's features lie a lane-group width apart (rows that 16-byte
// accesses do not tile); all of them must share the edge datum, i.e. one head.
// EPI: a finished row is multiplied by its entry of Args::row_scale (when given) and
// passes through Args::act before it is stored -- a GCN layer's destination norm and
// relu (examples/GCN/GCN.py:26) without a pass of their own; rows without edges too
// (0 * scale, so a non-finite scale shows as it does in the separate multiplication).
// The factor travels in one more float of state, fetched beside the gathers of the
// row's slots: read when the row is stored, it would put a load's latency in front of
// every store of the walk.
// ACT (EPI only): the activation, fixed at compile time -- the store sits inside the
// walk over the slots, once per unrolled position, and a choice made there at run time
// triples the loop's code.
template <typename T, int VEC, int RED, int BOP, bool SPREAD = false, bool EPI = false,
          int ACT = GA_ACT_NONE>
struct SpmmPolicy {
  static constexpr bool HASW = BOP != 0;
  typedef T out_t;
  static constexpr int kVec = VEC;
  static constexpr int kState = VEC + (EPI ? 1 : 0);
  static constexpr bool kSpread = SPREAD;
  struct Args {
    const int32_t *gidx;  // row of `u` gathered per slot (neighbour id, or edge
                          // id for copy_e); nullptr: the slot index itself
    const int32_t *eid;   // edge id per slot for `w`; nullptr: the slot index
    const T *u;
    const float *w;
    int heads;
    int dph;
    bool ids_vec;   // row_of_slot, gidx and eid (where given) are 16-byte aligned
    int stride_shift;   // SPREAD: log2 of the lanes per group, set by the launcher
    const float *row_scale;   // EPI: factor per output row, or nullptr
  };
  static __device__ __forceinline__ void init(float (&st)[kState]) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) st[v] = red_init<RED>();
    if constexpr (EPI) st[VEC] = 1.0f;
  }
  // o <- act(o * f); f is 1 (an exact product) without Args::row_scale
  static __device__ __forceinline__ void epilogue(float f, float (&o)[VEC]) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      const float x = o[v] * f;
      o[v] = ACT == GA_ACT_NONE ? x : (ACT == GA_ACT_ELU ? elu(x) : relu_keep_nan(x));
    }
  }
  static __device__ __forceinline__ void merge(float (&dst)[kState], const float *src) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) dst[v] = red_apply<RED>(dst[v], src[v]);
    if constexpr (EPI) dst[VEC] = src[VEC];   // every piece of a row carries the row's factor
  }
  static __device__ __forceinline__ void finish(const float (&st)[kState], float (&o)[VEC]) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) o[v] = st[v];
  }
  static __device__ __forceinline__ void empty_row(float (&o)[VEC]) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) o[v] = red_init<RED>();
  }
  static __device__ __forceinline__ void emit(const Args &A, out_t *out, int64_t row, int feat,
                                              int f0, const float (&st)[kState]) {
    if constexpr (EPI) {
      typedef RowIO<T, VEC, SPREAD> IO;
      float o[VEC];
      finish(st, o);
      epilogue(st[VEC], o);
      IO::store(out + row * feat + f0, o, IO::lane(A.stride_shift, feat - f0));
    } else {
      emit_row<SpmmPolicy>(out, row, feat, f0, st, A.stride_shift);
    }
  }
  static __device__ __forceinline__ void emit_empty(const Args &A, out_t *out, int64_t row,
                                                    int feat, int f0) {
    if constexpr (EPI) {
      typedef RowIO<T, VEC, SPREAD> IO;
      float o[VEC];
      empty_row(o);
      epilogue(A.row_scale ? A.row_scale[row] : 1.0f, o);
      IO::store(out + row * feat + f0, o, IO::lane(A.stride_shift, feat - f0));
    } else {
      emit_empty_row<SpmmPolicy>(out, row, feat, f0, A.stride_shift);
    }
  }

  template <class Close>
  static __device__ __forceinline__ void walk(const Args &A,
                                              const int32_t *__restrict__ row_of_slot,
                                              int64_t a, int64_t b, int f0, int feat,
                                              float (&st)[kState], int &cur,
                                              Close &&close_segment) {
    typedef RowIO<T, VEC, SPREAD> IO;
    const typename IO::lane_t ln = IO::lane(A.stride_shift, feat - f0);
    const int h = HASW && !SPREAD ? f0 / A.dph : 0;
    for (int64_t j = a; j < b; j += kUnroll) {
      int r[kUnroll], g[kUnroll], e[kUnroll];
      float ww[kUnroll];
      typename IO::raw_t x[kUnroll];
      load_ids8(row_of_slot, j, b, A.ids_vec, r);
      if (A.gidx) {
        load_ids8(A.gidx, j, b, A.ids_vec, g);
      } else {
#pragma unroll
        for (int t = 0; t < kUnroll; ++t) g[t] = (int)(j + t < b ? j + t : b - 1);
      }
      if (HASW) {
        if (A.eid) {
          load_ids8(A.eid, j, b, A.ids_vec, e);
        } else {
#pragma unroll
          for (int t = 0; t < kUnroll; ++t) e[t] = (int)(j + t < b ? j + t : b - 1);
        }
#pragma unroll
        for (int t = 0; t < kUnroll; ++t) ww[t] = A.w[(int64_t)e[t] * A.heads + h];
      }
#pragma unroll
      for (int t = 0; t < kUnroll; ++t) x[t] = IO::load(A.u + (int64_t)g[t] * feat + f0, ln);
      float rs[kUnroll];
      if constexpr (EPI) {
#pragma unroll
        for (int t = 0; t < kUnroll; ++t) rs[t] = A.row_scale ? A.row_scale[r[t]] : 1.0f;
      }
#pragma unroll
      for (int t = 0; t < kUnroll; ++t) {
        if (j + t < b) {
          if (r[t] != cur) {
            close_segment();
            cur = r[t];
            init(st);
          }
          float xf[VEC];
          IO::widen(x[t], xf);
#pragma unroll
          for (int v = 0; v < VEC; ++v)
            st[v] = red_apply<RED>(st[v], bin_apply<BOP>(xf[v], ww[t]));
          if constexpr (EPI) st[VEC] = rs[t];
        }
      }
    }
  }
};

template <typename T, int VEC, int RED, int BOP, bool SPREAD, bool EPI = false,
          int ACT = GA_ACT_NONE>
int launch_spmm(const int32_t *pointer, const int32_t *row_of_slot,
                const int32_t *gidx, const int32_t *eid, const void *u,
                const float *w, void *out, int64_t n_rows, int64_t n_edges,
                int feat, int heads, float *partial, hipStream_t stream,
                const float *row_scale = nullptr, size_t partial_bytes = SIZE_MAX) {
  typedef SpmmPolicy<T, VEC, RED, BOP, SPREAD, EPI, ACT> P;
  const bool ids_vec = aligned(row_of_slot, 16) && (!gidx || aligned(gidx, 16)) &&
                       (!eid || aligned(eid, 16));
  typename P::Args args{gidx, eid, (const T *)u, w, heads, feat / heads, ids_vec, 0, row_scale};
  return launch_runs<P>(args, pointer, row_of_slot, out, n_rows, n_edges, feat,
                        partial, stream, partial_bytes);
}

// max / min with the position of the extremum (the reference's generic kernel,
// spmm.cuh:30-71 with functor.cuh:148-213): beside each running extremum the
// state keeps the SLOT that produced it, so "first extremum in slot order wins"
// survives every merge (a later partial replaces an earlier one only when
// strictly better) and the ids are looked up once, when the row is written:
// arg_u = neighbour id of that slot (operators that read u), arg_e = its edge id
// (operators that read edge data).  Rows whose extremum was never replaced
// (no edges, or only NaN / infinities of the wrong sign) report 0, as the
// reference's zero-initialised locals do.
template <typename T, int VEC, int RED, int BOP>
struct SpmmArgPolicy {
  static constexpr bool HASW = BOP != 0;
  typedef T out_t;
  static constexpr int kVec = VEC;
  static constexpr int kState = 2 * VEC;
  static constexpr bool kSpread = false;
  struct Args {
    const int32_t *gidx;  // row of `u` gathered per slot; nullptr: the slot index
    const int32_t *eid;   // edge id per slot; nullptr: the slot index
    const int32_t *nbr;   // neighbour id per slot (for arg_u)
    const T *u;
    const float *w;
    int32_t *arg_u;       // nullptr: not wanted
    int32_t *arg_e;
    int heads;
    int dph;
  };
  static __device__ __forceinline__ void init(float (&st)[2 * VEC]) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      st[v] = red_init<RED>();
      st[VEC + v] = __int_as_float(-1);
    }
  }
  static __device__ __forceinline__ bool better(float acc, float m) {
    return RED == GA_MAX ? acc < m : acc > m;
  }
  static __device__ __forceinline__ void merge(float (&dst)[2 * VEC], const float *src) {
#pragma unroll
    for (int v = 0; v < VEC; ++v)
      if (better(dst[v], src[v])) {
        dst[v] = src[v];
        dst[VEC + v] = src[VEC + v];
      }
  }
  static __device__ __forceinline__ void finish(const float (&st)[2 * VEC], float (&o)[VEC]) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) o[v] = st[v];
  }
  static __device__ __forceinline__ void empty_row(float (&o)[VEC]) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) o[v] = red_init<RED>();
  }
  static __device__ __forceinline__ void emit(const Args &A, out_t *out, int64_t row, int feat,
                                              int f0, const float (&st)[2 * VEC]) {
    emit_row<SpmmArgPolicy>(out, row, feat, f0, st);
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      if (f0 + v >= feat) break;
      const int slot = __float_as_int(st[VEC + v]);
      if (A.arg_u) A.arg_u[row * feat + f0 + v] = slot < 0 ? 0 : A.nbr[slot];
      if (A.arg_e) A.arg_e[row * feat + f0 + v] = slot < 0 ? 0 : (A.eid ? A.eid[slot] : slot);
    }
  }
  static __device__ __forceinline__ void emit_empty(const Args &A, out_t *out, int64_t row,
                                                    int feat, int f0) {
    emit_empty_row<SpmmArgPolicy>(out, row, feat, f0);
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      if (f0 + v >= feat) break;
      if (A.arg_u) A.arg_u[row * feat + f0 + v] = 0;
      if (A.arg_e) A.arg_e[row * feat + f0 + v] = 0;
    }
  }

  template <class Close>
  static __device__ __forceinline__ void walk(const Args &A,
                                              const int32_t *__restrict__ row_of_slot,
                                              int64_t a, int64_t b, int f0, int feat,
                                              float (&st)[2 * VEC], int &cur,
                                              Close &&close_segment) {
    typedef Frag<T, VEC> IO;
    const int h = HASW ? f0 / A.dph : 0;
    for (int64_t j = a; j < b; j += kUnroll) {
      int r[kUnroll];
      int64_t g[kUnroll];
      float ww[kUnroll];
      typename IO::raw_t x[kUnroll];
#pragma unroll
      for (int t = 0; t < kUnroll; ++t) {
        const int64_t jj = j + t < b ? j + t : b - 1;
        r[t] = row_of_slot[jj];
        g[t] = A.gidx ? (int64_t)A.gidx[jj] : jj;
        if (HASW) {
          const int64_t e = A.eid ? (int64_t)A.eid[jj] : jj;
          ww[t] = A.w[e * A.heads + h];
        }
      }
#pragma unroll
      for (int t = 0; t < kUnroll; ++t) x[t] = IO::load(A.u + g[t] * feat + f0);
#pragma unroll
      for (int t = 0; t < kUnroll; ++t) {
        if (j + t < b) {
          if (r[t] != cur) {
            close_segment();
            cur = r[t];
            init(st);
          }
          float xf[VEC];
          IO::widen(x[t], xf);
#pragma unroll
          for (int v = 0; v < VEC; ++v) {
            const float m = bin_apply<BOP>(xf[v], ww[t]);
            if (better(st[v], m)) {
              st[v] = m;
              st[VEC + v] = __int_as_float((int)(j + t));
            }
          }
        }
      }
    }
  }
};

template <typename T, int VEC>
int launch_spmm_arg(int reduce, int bop, const int32_t *pointer,
                    const int32_t *row_of_slot, const int32_t *gidx,
                    const int32_t *eid, const int32_t *nbr, const void *u,
                    const float *w, void *out, int32_t *arg_u, int32_t *arg_e,
                    int64_t n_rows, int64_t n_edges, int feat, int heads,
                    float *partial, hipStream_t stream) {
#define GA_SPMM_ARG(RED, B)                                                        \
  do {                                                                             \
    typedef SpmmArgPolicy<T, VEC, RED, B> P;                                       \
    typename P::Args args{gidx, eid, nbr, (const T *)u, w, arg_u, arg_e, heads,    \
                          feat / heads};                                           \
    return launch_runs<P>(args, pointer, row_of_slot, out, n_rows, n_edges, feat,  \
                          partial, stream);                                        \
  } while (0)
#define GA_SPMM_ARG_RED(RED)                                                       \
  switch (bop) {                                                                   \
    case GA_U_MUL_E: GA_SPMM_ARG(RED, GA_U_MUL_E);                                 \
    case GA_U_ADD_E: GA_SPMM_ARG(RED, GA_U_ADD_E);                                 \
    case GA_U_SUB_E: GA_SPMM_ARG(RED, GA_U_SUB_E);                                 \
    case GA_U_DIV_E: GA_SPMM_ARG(RED, GA_U_DIV_E);                                 \
    default: GA_SPMM_ARG(RED, 0);                                                  \
  }
  if (reduce == GA_MAX) GA_SPMM_ARG_RED(GA_MAX)
  GA_SPMM_ARG_RED(GA_MIN)
#undef GA_SPMM_ARG_RED
#undef GA_SPMM_ARG
}

template <typename T, int VEC, int RED, bool SPREAD>
int pick_w(int bop, const int32_t *pointer, const int32_t *row_of_slot,
           const int32_t *gidx, const int32_t *eid, const void *u,
           const float *w, void *out, int64_t n_rows, int64_t n_edges, int feat,
           int heads, float *partial, hipStream_t stream) {
#define GA_SPMM_BOP(B)                                                             \
  return launch_spmm<T, VEC, RED, B, SPREAD>(pointer, row_of_slot, gidx, eid, u, w, out, \
                                             n_rows, n_edges, feat, heads, partial, stream)
  switch (bop) {
    case GA_U_MUL_E: GA_SPMM_BOP(GA_U_MUL_E);
    case GA_U_ADD_E: GA_SPMM_BOP(GA_U_ADD_E);
    case GA_U_SUB_E: GA_SPMM_BOP(GA_U_SUB_E);
    case GA_U_DIV_E: GA_SPMM_BOP(GA_U_DIV_E);
    default: GA_SPMM_BOP(0);
  }
#undef GA_SPMM_BOP
}

template <typename T, int VEC, bool SPREAD = false>
int pick_red(int reduce, int bop, const int32_t *pointer,
             const int32_t *row_of_slot, const int32_t *gidx,
             const int32_t *eid, const void *u, const float *w, void *out,
             int64_t n_rows, int64_t n_edges, int feat, int heads,
             float *partial, hipStream_t stream) {
  switch (reduce) {
    case GA_SUM:
      return pick_w<T, VEC, GA_SUM, SPREAD>(bop, pointer, row_of_slot, gidx, eid, u, w,
                                    out, n_rows, n_edges, feat, heads, partial,
                                    stream);
    case GA_MAX:
      return pick_w<T, VEC, GA_MAX, SPREAD>(bop, pointer, row_of_slot, gidx, eid, u, w,
                                    out, n_rows, n_edges, feat, heads, partial,
                                    stream);
    default:
      return pick_w<T, VEC, GA_MIN, SPREAD>(bop, pointer, row_of_slot, gidx, eid, u, w,
                                    out, n_rows, n_edges, feat, heads, partial,
                                    stream);
  }
}

__global__ __launch_bounds__(kBlock) void row_ids_kernel(
    const int32_t *__restrict__ pointer, int64_t n_rows, int64_t n_edges,
    int32_t *__restrict__ row_of_slot) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= n_edges) return;
  // largest v with pointer[v] <= i  (rows without edges are skipped over)
  int64_t lo = 0, hi = n_rows;  // invariant: pointer[lo] <= i < pointer[hi]
  while (hi - lo > 1) {
    const int64_t mid = (lo + hi) >> 1;
    if ((int64_t)pointer[mid] <= i) lo = mid; else hi = mid;
  }
  row_of_slot[i] = (int32_t)lo;
}

}  // namespace
}  // namespace ga

extern "C" {

int ga_csr_row_ids(const int32_t *pointer, int64_t n_rows, int64_t n_edges,
                   int32_t *row_of_slot, ga_stream_t stream) {
  if (n_rows < 0 || n_edges < 0 || n_rows > 0x7fffffff || n_edges > 0x7fffffff)
    return GA_EINVAL;
  if (n_edges == 0) return GA_OK;
  if (!pointer || !row_of_slot || n_rows == 0) return GA_EINVAL;
  const int64_t blocks = (n_edges + ga::kBlock - 1) / ga::kBlock;
  hipLaunchKernelGGL(ga::row_ids_kernel, dim3((unsigned)blocks),
                     dim3(ga::kBlock), 0, (hipStream_t)stream, pointer, n_rows,
                     n_edges, row_of_slot);
  return ga::launch_status();
}

size_t ga_spmm_workspace_bytes(int64_t n_edges, int64_t feat) {
  return ga::runs_workspace_bytes(n_edges, feat, 1);
}

int ga_spmm_csr(const int32_t *pointer, const int32_t *row_of_slot,
                const int32_t *nbr, const int32_t *eid, const void *u,
                const float *w, void *out, int64_t n_rows, int64_t n_edges,
                int64_t feat, int64_t heads, int op, int reduce, int dtype,
                void *workspace, size_t workspace_bytes, ga_stream_t stream) {
  if (n_rows < 0 || n_edges < 0 || feat <= 0 || heads <= 0 || feat % heads)
    return GA_EINVAL;
  if (n_rows > 0x7fffffff || n_edges > 0x7fffffff || feat > 0x7fffffff)
    return GA_EINVAL;
  if (op < GA_COPY_U || op > GA_U_DIV_E || reduce < GA_SUM || reduce > GA_MIN)
    return GA_EINVAL;
  if (dtype != GA_F32 && dtype != GA_BF16) return GA_EINVAL;
  if (n_rows == 0) return GA_OK;
  if (!pointer || !out) return GA_EINVAL;
  if (n_edges > 0) {
    if (!row_of_slot || !u) return GA_EINVAL;
    if (op != GA_COPY_E && !nbr) return GA_EINVAL;
    if (op >= GA_U_MUL_E && !w) return GA_EINVAL;
    if (ga_spmm_workspace_bytes(n_edges, feat) > workspace_bytes || !workspace)
      return GA_EWORKSPACE;
    if (!ga::aligned(workspace, 16)) return GA_EWORKSPACE;
  }
  const size_t esz = dtype == GA_F32 ? 4 : 2;
  if (!ga::aligned(out, esz) || (u && !ga::aligned(u, esz)) ||
      (w && !ga::aligned(w, 4)))
    return GA_EALIGN;

  const bool hasw = op >= GA_U_MUL_E;
  const int bop = hasw ? op : 0;
  const int32_t *gidx = op == GA_COPY_E ? eid : nbr;
  const int64_t dph = feat / heads;
  const bool vec_ok = ga::aligned(out, 16) && (!u || ga::aligned(u, 16));
  hipStream_t s = (hipStream_t)stream;
  float *partial = (float *)workspace;
  // rows that 16-byte accesses do not tile: four features per lane, a lane-group
  // width apart, when all of a row shares the edge datum (one head, or none read)
  const bool spread_ok = (!hasw || heads == 1) && feat >= 3 && feat <= 256;
  if (dtype == GA_F32) {
    if (vec_ok && feat % 4 == 0 && (!hasw || dph % 4 == 0))
      return ga::pick_red<float, 4>(reduce, bop, pointer, row_of_slot, gidx,
                                    eid, u, w, out, n_rows, n_edges, (int)feat,
                                    (int)heads, partial, s);
    if (spread_ok)
      return ga::pick_red<float, 4, true>(reduce, bop, pointer, row_of_slot, gidx,
                                          eid, u, w, out, n_rows, n_edges, (int)feat,
                                          (int)heads, partial, s);
    return ga::pick_red<float, 1>(reduce, bop, pointer, row_of_slot, gidx, eid,
                                  u, w, out, n_rows, n_edges, (int)feat,
                                  (int)heads, partial, s);
  }
  if (vec_ok && feat % 8 == 0 && (!hasw || dph % 8 == 0))
    return ga::pick_red<ga::bf16_t, 8>(reduce, bop, pointer, row_of_slot, gidx,
                                       eid, u, w, out, n_rows, n_edges,
                                       (int)feat, (int)heads, partial, s);
  if (spread_ok)
    return ga::pick_red<ga::bf16_t, 4, true>(reduce, bop, pointer, row_of_slot, gidx,
                                             eid, u, w, out, n_rows, n_edges, (int)feat,
                                             (int)heads, partial, s);
  return ga::pick_red<ga::bf16_t, 1>(reduce, bop, pointer, row_of_slot, gidx,
                                     eid, u, w, out, n_rows, n_edges, (int)feat,
                                     (int)heads, partial, s);
}

size_t ga_spmm_scaled_workspace_bytes(int64_t n_edges, int64_t feat) {
  // a float of state per lane beside its features: at most twice the plain sum's
  return ga::runs_workspace_bytes(n_edges, feat, 2);
}

int ga_spmm_csr_scaled(const int32_t *pointer, const int32_t *row_of_slot,
                       const int32_t *nbr, const int32_t *eid, const void *u, void *out,
                       const float *row_scale, int activation, int64_t n_rows,
                       int64_t n_edges, int64_t feat, int op, int dtype, void *workspace,
                       size_t workspace_bytes, ga_stream_t stream) {
  if (n_rows < 0 || n_edges < 0 || feat <= 0) return GA_EINVAL;
  if (n_rows > 0x7fffffff || n_edges > 0x7fffffff || feat > 0x7fffffff) return GA_EINVAL;
  if (op != GA_COPY_U && op != GA_COPY_E) return GA_EINVAL;
  if (activation < GA_ACT_NONE || activation > GA_ACT_ELU) return GA_EINVAL;
  if (dtype != GA_F32 && dtype != GA_BF16) return GA_EINVAL;
  if (n_rows == 0) return GA_OK;
  if (!pointer || !out) return GA_EINVAL;
  if (n_edges > 0) {
    if (!row_of_slot || !u) return GA_EINVAL;
    if (op == GA_COPY_U && !nbr) return GA_EINVAL;
    if (ga_spmm_scaled_workspace_bytes(n_edges, feat) > workspace_bytes || !workspace)
      return GA_EWORKSPACE;
    if (!ga::aligned(workspace, 16)) return GA_EWORKSPACE;
  }
  const size_t esz = dtype == GA_F32 ? 4 : 2;
  if (!ga::aligned(out, esz) || (u && !ga::aligned(u, esz)) ||
      (row_scale && !ga::aligned(row_scale, 4)))
    return GA_EALIGN;
  const int32_t *gidx = op == GA_COPY_E ? eid : nbr;
  const bool vec_ok = ga::aligned(out, 16) && (!u || ga::aligned(u, 16));
  hipStream_t s = (hipStream_t)stream;
  float *partial = (float *)workspace;
  const bool spread_ok = feat >= 3 && feat <= 256;
#define GA_SPMM_EPI_ACT(T, VEC, SPREAD, ACT)                                             \
  return ga::launch_spmm<T, VEC, GA_SUM, 0, SPREAD, true, ACT>(                         \
      pointer, row_of_slot, gidx, eid, u, nullptr, out, n_rows, n_edges, (int)feat, 1, \
      partial, s, row_scale, workspace_bytes)
#define GA_SPMM_EPI(T, VEC, SPREAD)                                        \
  do {                                                                     \
    if (activation == GA_ACT_RELU) GA_SPMM_EPI_ACT(T, VEC, SPREAD, GA_ACT_RELU); \
    if (activation == GA_ACT_ELU) GA_SPMM_EPI_ACT(T, VEC, SPREAD, GA_ACT_ELU);   \
    GA_SPMM_EPI_ACT(T, VEC, SPREAD, GA_ACT_NONE);                          \
  } while (0)
  if (dtype == GA_F32) {
    if (vec_ok && feat % 4 == 0) GA_SPMM_EPI(float, 4, false);
    if (spread_ok) GA_SPMM_EPI(float, 4, true);
    GA_SPMM_EPI(float, 1, false);
  }
  if (vec_ok && feat % 8 == 0) GA_SPMM_EPI(ga::bf16_t, 8, false);
  if (spread_ok) GA_SPMM_EPI(ga::bf16_t, 4, true);
  GA_SPMM_EPI(ga::bf16_t, 1, false);
#undef GA_SPMM_EPI
#undef GA_SPMM_EPI_ACT
}

size_t ga_spmm_arg_workspace_bytes(int64_t n_edges, int64_t feat) {
  return ga::runs_workspace_bytes(n_edges, feat, 2);
}

int ga_spmm_csr_arg(const int32_t *pointer, const int32_t *row_of_slot,
                    const int32_t *nbr, const int32_t *eid, const void *u,
                    const float *w, void *out, int32_t *arg_u, int32_t *arg_e,
                    int64_t n_rows, int64_t n_edges, int64_t feat, int64_t heads,
                    int op, int reduce, int dtype, void *workspace,
                    size_t workspace_bytes, ga_stream_t stream) {
  if (n_rows < 0 || n_edges < 0 || feat <= 0 || heads <= 0 || feat % heads)
    return GA_EINVAL;
  if (n_rows > 0x7fffffff || n_edges > 0x7fffffff || feat > 0x7fffffff)
    return GA_EINVAL;
  if (op < GA_COPY_U || op > GA_U_DIV_E) return GA_EINVAL;
  if (reduce != GA_MAX && reduce != GA_MIN) return GA_EINVAL;   // sum has no position
  if (dtype != GA_F32 && dtype != GA_BF16) return GA_EINVAL;
  // arg_u exists for operators that read u, arg_e for those that read edge data
  if (op == GA_COPY_E && arg_u) return GA_EINVAL;
  if (op == GA_COPY_U && arg_e) return GA_EINVAL;
  if (n_rows == 0) return GA_OK;
  if (!pointer || !out) return GA_EINVAL;
  if (n_edges > 0) {
    if (!row_of_slot || !u) return GA_EINVAL;
    if (op != GA_COPY_E && !nbr) return GA_EINVAL;
    if (op >= GA_U_MUL_E && !w) return GA_EINVAL;
    if (ga_spmm_arg_workspace_bytes(n_edges, feat) > workspace_bytes || !workspace)
      return GA_EWORKSPACE;
    if (!ga::aligned(workspace, 16)) return GA_EWORKSPACE;
  }
  const size_t esz = dtype == GA_F32 ? 4 : 2;
  if (!ga::aligned(out, esz) || (u && !ga::aligned(u, esz)) ||
      (w && !ga::aligned(w, 4)) || (arg_u && !ga::aligned(arg_u, 4)) ||
      (arg_e && !ga::aligned(arg_e, 4)))
    return GA_EALIGN;

  const bool hasw = op >= GA_U_MUL_E;
  const int bop = hasw ? op : 0;
  const int32_t *gidx = op == GA_COPY_E ? eid : nbr;
  const int64_t dph = feat / heads;
  const bool vec_ok = ga::aligned(out, 16) && (!u || ga::aligned(u, 16));
  hipStream_t s = (hipStream_t)stream;
  float *partial = (float *)workspace;
  if (dtype == GA_F32) {
    if (vec_ok && feat % 4 == 0 && (!hasw || dph % 4 == 0))
      return ga::launch_spmm_arg<float, 4>(reduce, bop, pointer, row_of_slot, gidx, eid,
                                           nbr, u, w, out, arg_u, arg_e, n_rows, n_edges,
                                           (int)feat, (int)heads, partial, s);
    return ga::launch_spmm_arg<float, 1>(reduce, bop, pointer, row_of_slot, gidx, eid, nbr,
                                         u, w, out, arg_u, arg_e, n_rows, n_edges,
                                         (int)feat, (int)heads, partial, s);
  }
  if (vec_ok && feat % 8 == 0 && (!hasw || dph % 8 == 0))
    return ga::launch_spmm_arg<ga::bf16_t, 8>(reduce, bop, pointer, row_of_slot, gidx, eid,
                                              nbr, u, w, out, arg_u, arg_e, n_rows, n_edges,
                                              (int)feat, (int)heads, partial, s);
  return ga::launch_spmm_arg<ga::bf16_t, 1>(reduce, bop, pointer, row_of_slot, gidx, eid,
                                            nbr, u, w, out, arg_u, arg_e, n_rows, n_edges,
                                            (int)feat, (int)heads, partial, s);
}

}  // extern "C"
