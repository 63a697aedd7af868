// Load-balanced row reduction over a grouped adjacency (shared by the SpMM and
// the fused GAT aggregation).
//
// Schedule.  The slots [0, E) are cut into equal runs of 2^run_shift slots.  A
// group of `tpr` adjacent lanes (tpr * VEC features = one feature-row tile;
// a lane holds VEC consecutive features, 16 bytes, or -- Policy::kSpread -- VEC
// features tpr apart, see RowIO) owns one run and walks it in slot order with
// eight gathers in flight per lane; a workgroup of 256 lanes owns G = 256 / tpr
// consecutive runs.  Rows that lie inside one run are written straight to the
// output.  A row shared by neighbouring runs leaves partial states, which the
// workgroup chains together in LDS; only a row that crosses the workgroup's
// slot range leaves (at most two) partial states in the global workspace, and
// a small second kernel combines those in workgroup order.  Work per lane group
// is therefore identical whatever the degree distribution, no atomics are used
// and the order of every combination depends on the graph and sizes only.
//
// A Policy supplies the per-lane state and arithmetic:
//   kState                      floats of state per lane
//   init(st)                    empty state
//   absorb(st, ...)             done inside Policy::walk, which processes one
//                               batch of slots
//   merge(dst, src)             dst <- dst (+) src, dst precedes src in slot order
//   finish(st, o)               state -> VEC output features
//   empty_row(o)                output of a row without edges
//   emit(args, out, row, feat, f0, st) / emit_empty(args, out, row, feat, f0)
//                               write a finished / an edgeless row's tile; the
//                               usual ones are emit_row / emit_empty_row below,
//                               a policy with further outputs writes them here
//   kSpread                     lane layout (see above); such a policy's Args carry
//                               `stride_shift`, which the launcher sets to log2(tpr)
#pragma once

#include "common.h"

namespace ga {

constexpr int kUnroll = 8;

static_assert(kUnroll == 8, "load_ids8 reads two int4");

// Eight consecutive int32 of a slot-indexed column starting at slot j (a
// multiple of 8: runs start at multiples of 32).  Two 16-byte loads when the
// column is 16-byte aligned and the batch is whole; otherwise element loads
// clamped to the run's last slot.
__device__ __forceinline__ void load_ids8(const int32_t *__restrict__ p, int64_t j, int64_t b,
                                          bool vec, int (&out)[kUnroll]) {
  if (vec && j + kUnroll <= b) {
    const int4 lo = *reinterpret_cast<const int4 *>(p + j);
    const int4 hi = *reinterpret_cast<const int4 *>(p + j + 4);
    out[0] = lo.x; out[1] = lo.y; out[2] = lo.z; out[3] = lo.w;
    out[4] = hi.x; out[5] = hi.y; out[6] = hi.z; out[7] = hi.w;
  } else {
#pragma unroll
    for (int t = 0; t < kUnroll; ++t) out[t] = p[j + t < b ? j + t : b - 1];
  }
}

struct RunGeom {
  int64_t n_edges;
  int64_t n_runs;
  int64_t n_rows;
  int feat;
  int run_shift;
  int tpr_shift;
  int lanes_total;  // ceil(feat / VEC): state slots per partial row
  int64_t n_wg;     // workgroups of the main kernel that walk runs; the blocks
                    // after them write the rows without edges
};

// Per-run bookkeeping shared through LDS.
struct RunFlags {
  int has_a;    // first segment began before this run
  int a_open;   // ... and it also continues past the run's end
  int has_b;    // last segment began inside this run and continues past its end
  int row_a;
  int row_b;
};

template <class Policy>
__device__ __forceinline__ void emit_row(typename Policy::out_t *out, int64_t row, int feat,
                                         int f0, const float (&st)[Policy::kState],
                                         int stride_shift = 0) {
  typedef RowIO<typename Policy::out_t, Policy::kVec, Policy::kSpread> IO;
  float o[Policy::kVec];
  Policy::finish(st, o);
  IO::store(out + row * feat + f0, o, IO::lane(stride_shift, feat - f0));
}
template <class Policy>
__device__ __forceinline__ void emit_empty_row(typename Policy::out_t *out, int64_t row,
                                               int feat, int f0, int stride_shift = 0) {
  typedef RowIO<typename Policy::out_t, Policy::kVec, Policy::kSpread> IO;
  float o[Policy::kVec];
  Policy::empty_row(o);
  IO::store(out + row * feat + f0, o, IO::lane(stride_shift, feat - f0));
}

// First feature of lane `lane` of a group in feature tile `tile`.
template <class Policy>
__device__ __forceinline__ int lane_first_feature(int tile, int lane, int tpr_shift) {
  return Policy::kSpread ? ((tile * Policy::kVec) << tpr_shift) + lane
                         : ((tile << tpr_shift) + lane) * Policy::kVec;
}

template <class Policy>
__global__ __launch_bounds__(kBlock) void runs_kernel(
    typename Policy::Args args, const int32_t *__restrict__ pointer,
    const int32_t *__restrict__ row_of_slot, typename Policy::out_t *__restrict__ out,
    float *__restrict__ partial, RunGeom geo) {
  constexpr int SF = Policy::kState;
  if ((int64_t)blockIdx.x >= geo.n_wg) {
    // Trailing blocks: one lane group per row, rows without edges get the empty
    // value.  They share the launch with the gathers, so this small amount of
    // streaming work hides behind them instead of costing a pass of its own.
    const int tpr_ = 1 << geo.tpr_shift;
    const int f0_ = lane_first_feature<Policy>((int)blockIdx.y, threadIdx.x & (tpr_ - 1), geo.tpr_shift);
    const int64_t row = (((int64_t)blockIdx.x - geo.n_wg) * kBlock + threadIdx.x) >> geo.tpr_shift;
    if (f0_ < geo.feat && row < geo.n_rows && pointer[row] == pointer[row + 1])
      Policy::emit_empty(args, out, row, geo.feat, f0_);
    return;
  }
  // LDS: [run in block][A|B][lane in group][SF]
  extern __shared__ float lds_state[];
  __shared__ RunFlags flags[kBlock];

  const int tpr = 1 << geo.tpr_shift;
  const int G = kBlock >> geo.tpr_shift;
  const int grp = threadIdx.x >> geo.tpr_shift;
  const int lane = threadIdx.x & (tpr - 1);
  const int64_t k = (int64_t)blockIdx.x * G + grp;
  const int flane = (int)blockIdx.y * tpr + lane;   // feature lane index
  const int f0 = lane_first_feature<Policy>((int)blockIdx.y, lane, geo.tpr_shift);
  const bool live = k < geo.n_runs && f0 < geo.feat;

  float *my_a = lds_state + ((grp * 2 + 0) * tpr + lane) * SF;
  float *my_b = lds_state + ((grp * 2 + 1) * tpr + lane) * SF;

  float st[SF];
  Policy::init(st);
  bool has_a = false, a_open = false, has_b = false;
  int row_a = 0, row_b = 0;

  if (live) {
    const int64_t a = k << geo.run_shift;
    const int64_t b = min(a + ((int64_t)1 << geo.run_shift), geo.n_edges);
    int cur = row_of_slot[a];
    const bool began_before = a > 0 && row_of_slot[a - 1] == cur;
    bool first_seg = true;

    // closes the open segment: complete rows go to `out`, a first segment that
    // began before the run becomes this run's A state
    auto close_segment = [&]() {
      if (first_seg && began_before) {
        has_a = true;
        row_a = cur;
#pragma unroll
        for (int i = 0; i < SF; ++i) my_a[i] = st[i];
      } else {
        Policy::emit(args, out, cur, geo.feat, f0, st);
      }
      first_seg = false;
    };

    Policy::walk(args, row_of_slot, a, b, f0, geo.feat, st, cur, close_segment);

    const bool continues = b < geo.n_edges && row_of_slot[b] == cur;
    if (first_seg && began_before) {
      has_a = true;
      a_open = continues;
      row_a = cur;
#pragma unroll
      for (int i = 0; i < SF; ++i) my_a[i] = st[i];
    } else if (continues) {
      has_b = true;
      row_b = cur;
#pragma unroll
      for (int i = 0; i < SF; ++i) my_b[i] = st[i];
    } else {
      Policy::emit(args, out, cur, geo.feat, f0, st);
    }
  }
  if (lane == 0) {
    flags[grp].has_a = has_a;
    flags[grp].a_open = a_open;
    flags[grp].has_b = has_b;
    flags[grp].row_a = row_a;
    flags[grp].row_b = row_b;
  }
  __syncthreads();
  if (!live) return;

  auto state_of = [&](int g, int slot) -> const float * {
    return lds_state + ((g * 2 + slot) * tpr + lane) * SF;
  };
  // chain ending at run `i` (its A state included): walk back over runs the
  // row passes straight through, then combine in ascending run order
  auto chain_into = [&](int i, float (&acc)[SF]) -> bool {
    int j = i - 1;
    while (j >= 0 && flags[j].has_a && flags[j].a_open) --j;
    const bool starts_inside = j >= 0;   // then run j holds the chain's B state
    if (starts_inside) {
      const float *p = state_of(j, 1);
#pragma unroll
      for (int q = 0; q < SF; ++q) acc[q] = p[q];
    } else {
      Policy::init(acc);
    }
    for (int g = j + 1; g <= i; ++g) Policy::merge(acc, state_of(g, 0));
    return starts_inside;
  };
  float *const gp = partial + (int64_t)blockIdx.x * 2 * geo.lanes_total * SF;
  const int64_t runs_left = geo.n_runs - (int64_t)blockIdx.x * G;
  const int last = (int)(runs_left < G ? runs_left : G) - 1;

  if (has_a && !a_open) {            // a row ends in my run
    float acc[SF];
    if (chain_into(grp, acc)) {
      Policy::emit(args, out, row_a, geo.feat, f0, acc);
    } else {                         // began before this workgroup: slot 0
      float *p = gp + (int64_t)flane * SF;
#pragma unroll
      for (int q = 0; q < SF; ++q) p[q] = acc[q];
    }
  }
  if (grp == last) {                 // what leaves the workgroup at its end
    if (has_b) {
      float *p = gp + ((int64_t)geo.lanes_total + flane) * SF;
#pragma unroll
      for (int q = 0; q < SF; ++q) p[q] = my_b[q];
    } else if (has_a && a_open) {
      float acc[SF];
      const bool inside = chain_into(grp, acc);
      float *p = gp + ((int64_t)(inside ? geo.lanes_total : 0) + flane) * SF;
#pragma unroll
      for (int q = 0; q < SF; ++q) p[q] = acc[q];
    }
  }
}

// Blocks [0, fix_blocks): one lane group per main-kernel workgroup q; the group
// whose slot range holds the END of a row that began in an earlier workgroup
// combines that row's global partial states in workgroup order.  A chain of more
// than max(kLongChain, lane groups per block) states is combined by the whole
// block instead: every lane group folds a contiguous piece of the chain, in order,
// and the owning group combines the pieces in order -- so a row of any length costs
// chain / groups sequential steps, not chain.  Remaining blocks (only for a graph
// without edges, where the main kernel does not run): one lane group per row, every
// row gets Policy::empty_row.
constexpr int kLongChain = 64;

// acc <- acc (+) states w0 .. w1-1 of a chain (stride floats apart, `src` at w0), four
// fetched at a time so that the loads overlap instead of queueing up one latency
// after the other.
template <class Policy>
__device__ __forceinline__ void fold_chain(float (&acc)[Policy::kState], const float *src,
                                           int64_t stride, int64_t w0, int64_t w1) {
  constexpr int SF = Policy::kState;
  int64_t w = w0;
  for (; w + 4 <= w1; w += 4, src += 4 * stride) {
    float nxt[4][SF];
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int i = 0; i < SF; ++i) nxt[u][i] = src[u * stride + i];
#pragma unroll
    for (int u = 0; u < 4; ++u) Policy::merge(acc, nxt[u]);
  }
  for (; w < w1; ++w, src += stride) Policy::merge(acc, src);
}

template <class Policy>
__global__ __launch_bounds__(kBlock) void runs_fixup_kernel(
    typename Policy::Args args, const int32_t *__restrict__ pointer,
    const int32_t *__restrict__ row_of_slot,
    const float *__restrict__ partial, typename Policy::out_t *__restrict__ out,
    RunGeom geo, int64_t n_wg, int fix_blocks) {
  constexpr int SF = Policy::kState;
  extern __shared__ float piece_state[];      // [thread][SF]: pieces of a long chain
  __shared__ int64_t long_first[kBlock];      // per lane group: first workgroup of its long chain, or -1
  const int tpr = 1 << geo.tpr_shift;
  const int G = kBlock >> geo.tpr_shift;
  const int lane = threadIdx.x & (tpr - 1);
  const int grp = threadIdx.x >> geo.tpr_shift;
  const int flane = (int)blockIdx.y * tpr + lane;
  const int f0 = lane_first_feature<Policy>((int)blockIdx.y, lane, geo.tpr_shift);
  const bool lane_live = f0 < geo.feat;
  if ((int)blockIdx.x >= fix_blocks) {
    const int64_t row =
        ((int64_t)(blockIdx.x - fix_blocks) * kBlock + threadIdx.x) >> geo.tpr_shift;
    if (!lane_live || row >= geo.n_rows || pointer[row] != pointer[row + 1]) return;
    Policy::emit_empty(args, out, row, geo.feat, f0);
    return;
  }
  const int64_t q = (int64_t)blockIdx.x * G + grp;
  const int wg_shift = geo.run_shift + (8 - geo.tpr_shift);  // log2(G * run)
  const int64_t stride = (int64_t)2 * geo.lanes_total * SF;  // floats between workgroups' states
  bool mine = false;     // a row that began in an earlier workgroup ends in workgroup q
  int row = 0;
  int64_t q_lo = 0;
  if (q < n_wg) {
    const int64_t a = q << wg_shift;
    const int64_t b = min(a + ((int64_t)1 << wg_shift), geo.n_edges);
    row = row_of_slot[a];
    const int64_t s = pointer[row], e = pointer[row + 1];
    mine = s < a && e <= b;
    q_lo = s >> wg_shift;
  }
  // the chain: slot 1 of workgroup q_lo, then slot 0 of workgroups q_lo + 1 .. q
  // with many narrow lane groups per block the cooperative form starts later: its
  // barriers and the scan over the groups cost more than a chain of that length
  const bool is_long = mine && q - q_lo > max(kLongChain, G);
  if (lane == 0) long_first[grp] = is_long ? q_lo : -1;
  if (mine && !is_long && lane_live) {
    float acc[SF];
    const float *p = partial + ((q_lo * 2 + 1) * geo.lanes_total + flane) * SF;
#pragma unroll
    for (int i = 0; i < SF; ++i) acc[i] = p[i];
    fold_chain<Policy>(acc, partial + (((q_lo + 1) * 2) * geo.lanes_total + flane) * SF, stride,
                       q_lo + 1, q + 1);
    Policy::emit(args, out, row, geo.feat, f0, acc);
  }
  if (!__syncthreads_or(is_long)) return;     // the usual case: no long chain in this block
  // pieces: the first min(G, 64) lane groups take one each
  const int p_shift = min(8 - geo.tpr_shift, 6);
  for (int gg = 0; gg < G; ++gg) {
    const int64_t c_lo = long_first[gg];      // the same for the whole block
    if (c_lo < 0) continue;
    const int64_t first = c_lo + 1;           // slot-0 states of workgroups first .. first + len - 1
    const int64_t len = (int64_t)blockIdx.x * G + gg - c_lo;
    const int64_t w0 = first + ((len * grp) >> p_shift), w1 = first + ((len * (grp + 1)) >> p_shift);
    if (lane_live && (grp >> p_shift) == 0 && w0 < w1) {
      float acc[SF];
      const float *src = partial + ((w0 * 2) * geo.lanes_total + flane) * SF;
#pragma unroll
      for (int i = 0; i < SF; ++i) acc[i] = src[i];
      fold_chain<Policy>(acc, src + stride, stride, w0 + 1, w1);
#pragma unroll
      for (int i = 0; i < SF; ++i) piece_state[threadIdx.x * SF + i] = acc[i];
    }
    __syncthreads();
    if (grp == gg && lane_live) {             // the chain's own group: pieces in order
      float acc[SF];
      const float *p = partial + ((c_lo * 2 + 1) * geo.lanes_total + flane) * SF;
#pragma unroll
      for (int i = 0; i < SF; ++i) acc[i] = p[i];
      for (int j = 0; j < (1 << p_shift); ++j)
        if (((len * j) >> p_shift) < ((len * (j + 1)) >> p_shift))
          Policy::merge(acc, piece_state + ((j << geo.tpr_shift) + lane) * SF);
      Policy::emit(args, out, row, geo.feat, f0, acc);
    }
    __syncthreads();
  }
}

// Workspace bound that holds for every element type, vector width and lane layout:
// at most ceil(n_runs / 4) workgroups (tpr <= 64), two partial rows each.  A partial
// row has a state per lane of every feature tile, dead lanes included; the widest
// case is the spread layout of four features per lane, whose tiles are counted here.
inline size_t runs_workspace_bytes(int64_t n_edges, int64_t feat,
                                   int state_floats_per_feature) {
  if (n_edges <= 0 || feat <= 0) return 0;
  const int run_shift = run_shift_for(n_edges, feat);
  const int64_t n_runs = (n_edges + ((int64_t)1 << run_shift) - 1) >> run_shift;
  const int64_t n_wg = (n_runs + 3) / 4;
  const int64_t lanes = (feat + 3) / 4;
  const int64_t tpr = (int64_t)1 << ilog2_ceil((uint64_t)(lanes > kWave ? kWave : lanes));
  const int64_t slots = (lanes + tpr - 1) / tpr * tpr * 4;
  return (size_t)n_wg * 2 * (size_t)slots * state_floats_per_feature * sizeof(float);
}

// `partial_bytes`: capacity of `partial`.  The launch needs two partial rows per
// workgroup of the layout actually chosen (never more than runs_workspace_bytes)
// and returns GA_EWORKSPACE, having launched nothing, when that does not fit.
// With `size_only` the call only stores that byte count there (host arithmetic,
// no pointer is read, nothing is launched).
template <class Policy>
int launch_runs(typename Policy::Args args, const int32_t *pointer,
                const int32_t *row_of_slot, void *out, int64_t n_rows,
                int64_t n_edges, int feat, float *partial, hipStream_t stream,
                size_t partial_bytes = SIZE_MAX, size_t *size_only = nullptr) {
  constexpr int VEC = Policy::kVec;
  constexpr int SF = Policy::kState;
  RunGeom geo;
  const int lanes = (feat + VEC - 1) / VEC;
  geo.tpr_shift = ilog2_ceil((uint64_t)(lanes > kWave ? kWave : lanes));
  const int tpr = 1 << geo.tpr_shift;
  const int ftiles = (lanes + tpr - 1) / tpr;
  geo.run_shift = run_shift_for(n_edges, feat);
  geo.n_runs = (n_edges + ((int64_t)1 << geo.run_shift) - 1) >> geo.run_shift;
  geo.n_edges = n_edges;
  geo.n_rows = n_rows;
  geo.feat = feat;
  geo.lanes_total = Policy::kSpread ? ftiles * tpr : lanes;
  if constexpr (Policy::kSpread) args.stride_shift = geo.tpr_shift;
  const int G = kBlock >> geo.tpr_shift;
  const int64_t n_wg = (geo.n_runs + G - 1) / G;
  const int64_t row_blocks = (n_rows + G - 1) / G;
  geo.n_wg = n_wg;
  typedef typename Policy::out_t out_t;
  if (n_wg + row_blocks > 0x7fffffff) return GA_EUNSUPPORTED;
  const size_t needed = (size_t)n_wg * 2 * (size_t)geo.lanes_total * SF * sizeof(float);
  if (size_only) {          // sizing query: report the bytes of this layout, launch nothing
    *size_only = needed;
    return GA_OK;
  }
  if (needed > partial_bytes) return GA_EWORKSPACE;
  if (n_wg > 0) {
    const size_t lds = (size_t)kBlock * 2 * SF * sizeof(float);
    hipLaunchKernelGGL((runs_kernel<Policy>), dim3((unsigned)(n_wg + row_blocks), ftiles),
                       dim3(kBlock), lds, stream, args, pointer, row_of_slot,
                       (out_t *)out, partial, geo);
  }
  const int64_t fix_blocks = (n_wg + G - 1) / G;
  const int64_t fill_blocks = n_wg > 0 ? 0 : row_blocks;
  if (fix_blocks + fill_blocks > 0x7fffffff) return GA_EUNSUPPORTED;
  if (fix_blocks + fill_blocks > 0)
    hipLaunchKernelGGL((runs_fixup_kernel<Policy>),
                       dim3((unsigned)(fix_blocks + fill_blocks), ftiles),
                       dim3(kBlock), (size_t)kBlock * SF * sizeof(float), stream, args, pointer,
                       row_of_slot, partial, (out_t *)out, geo, n_wg, (int)fix_blocks);
  return launch_status();
}

}  // namespace ga
