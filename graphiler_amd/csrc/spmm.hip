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

// ---- sums of rows of at most eight features: one or two lanes per slot --------
// With one or two lanes per row a lane group of the run schedule walks a run of its
// own, so a wave instruction reads 32 or 64 separate pieces of the slot-indexed columns
// and nothing of the walk coalesces (copy_u with one feature on 11.6 M edges: 129 us
// for 93 MB).  Here L = 1 or 2 adjacent lanes own one SLOT (a lane holds up to four of
// the row's features, L apart): the wavefront reads 64 / L consecutive slots of the
// columns with one access each, gathers their rows, and adds up the slots of each row
// with a segmented scan over the lanes -- rows are sorted, so lanes with equal row ids
// at distance d have that id in between: DPP shifts inside rows of 16 lanes, then the
// totals at the end of a row of lanes go to the lanes of the next one that continue
// its segment.  A wavefront owns up to 16 consecutive chunks; the segment that runs
// into the next chunk is carried in registers.  The first and the last segment of a
// wavefront's range may be pieces of a longer row: they take the route of the run
// schedule -- the four wavefronts of a workgroup chain their pieces through LDS, and
// what crosses the workgroup's slot range leaves the same two partial states per
// workgroup that runs_kernel leaves, so the second kernel is runs_fixup_kernel of the
// L-lanes-per-row layout, unchanged.  Additions of a row happen in the scan's tree
// order, fixed by the slot positions.
constexpr int kSlotUnroll = 4;   // chunks whose loads are in flight together

// One step of the segmented scan inside rows of 16 lanes: a lane whose neighbour OFF
// lanes down (in its row of lanes) holds the same key adds that neighbour's sums.  Lanes
// without such a neighbour see the key -3, which no slot has.
template <int OFF>
__device__ __forceinline__ void slots_scan16(int key, float (&acc)[4], int live) {
  const int pk = __builtin_amdgcn_update_dpp(-3, key, 0x110 + OFF, 0xF, 0xF, false);   // row_shr:OFF
  const bool hit = pk == key;
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    if (v < live) {                          // uniform: the most features a lane holds
      const float pv = __int_as_float(__builtin_amdgcn_update_dpp(
          0, __float_as_int(acc[v]), 0x110 + OFF, 0xF, 0xF, false));
      if (hit) acc[v] += pv;
    }
  }
}
// The lanes of row ROW whose key is that of the last slot of the row before add that
// slot's (already complete) sums: lane 16 ROW - L + (lane mod L) holds them.
template <int ROW, int L>
__device__ __forceinline__ void slots_row_carry(int key, float (&acc)[4], int live, int lane) {
  const int ck = __builtin_amdgcn_readlane(key, 16 * ROW - 1);
  const bool hit = (lane >> 4) == ROW && key == ck;
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    if (v < live) {
      float cv = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(acc[v]), 16 * ROW - 1));
      if (L == 2) {
        const float c0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(acc[v]), 16 * ROW - 2));
        cv = (lane & 1) ? cv : c0;
      }
      if (hit) acc[v] += cv;
    }
  }
}
// v of lane `from + (lane mod L)` (from: uniform, a multiple of L) in every lane
template <int L>
__device__ __forceinline__ float slots_from(float v, int from, int lane) {
  float r = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), from));
  if (L == 2) {
    const float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), from + 1));
    r = (lane & 1) ? r1 : r;
  }
  return r;
}

template <class P, int BOP, int LS>
__global__ __launch_bounds__(kBlock) void slots_kernel(
    typename P::Args args, const int32_t *__restrict__ pointer,
    const int32_t *__restrict__ row_of_slot, typename P::out_t *__restrict__ out,
    float *__restrict__ partial, RunGeom geo) {
  typedef typename P::out_t T;
  typedef RowIO<T, 4, true> IO;
  constexpr int SF = P::kState;          // 4 sums (+ the row factor)
  constexpr bool EPI = SF > 4;
  constexpr bool HASW = BOP != 0;
  constexpr int kWaves = kBlock / kWave;
  constexpr int L = 1 << LS;             // lanes per slot
  constexpr int kChunk = kWave >> LS;    // slots per chunk
  const int sub = threadIdx.x & (L - 1); // the lane's first feature
  if ((int64_t)blockIdx.x >= geo.n_wg) {   // rows without edges, L lanes per row
    const int64_t row = (((int64_t)blockIdx.x - geo.n_wg) * kBlock + threadIdx.x) >> LS;
    if (row < geo.n_rows && pointer[row] == pointer[row + 1])
      P::emit_empty(args, out, row, geo.feat, sub);
    return;
  }
  __shared__ float piece[kWaves][2][L][SF];   // [wavefront][A | B][lane of the slot][state]
  __shared__ RunFlags flags[kWaves];
  const int lane = threadIdx.x & (kWave - 1);
  const int slot_lane = lane >> LS;
  const int wave = threadIdx.x / kWave;
  const int feat = geo.feat;
  const typename IO::lane_t ln = IO::lane(LS, feat - sub);
  const int live = (feat + L - 1) >> LS;   // features of the slot's first lane (the most)
  const int wg_shift = geo.run_shift + 8 - LS;
  const int64_t wave_slots = (int64_t)1 << (wg_shift - 2);
  const int64_t wa = ((int64_t)blockIdx.x << wg_shift) + wave * wave_slots;
  const int64_t wb = min(wa + wave_slots, geo.n_edges);
  if (lane == 0) {
    flags[wave].has_a = flags[wave].a_open = flags[wave].has_b = 0;
    flags[wave].row_a = flags[wave].row_b = 0;
  }
  if (wa < wb) {
    const int first_key = row_of_slot[wa];
    const bool first_open = wa > 0 && row_of_slot[wa - 1] == first_key;
    int carry_key = -1;                    // row of the segment that runs on from the last chunk
    float carry[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    float carry_scale = 1.0f;
    // the slot-indexed columns of kSlotUnroll chunks; those of the next round are
    // requested before the current round's sums, so they arrive meanwhile
    struct Ids {
      int r[kSlotUnroll], rn[kSlotUnroll];
      int64_t g[kSlotUnroll], e[kSlotUnroll];
    };
    auto load_ids = [&](int64_t j0, Ids &I) {
#pragma unroll
      for (int c = 0; c < kSlotUnroll; ++c) {
        const int64_t j = j0 + c * kChunk + slot_lane;
        const int64_t jc = j < wb ? j : wb - 1;
        I.r[c] = row_of_slot[jc];
        I.rn[c] = jc + 1 < geo.n_edges ? row_of_slot[jc + 1] : -1;
        I.g[c] = args.gidx ? (int64_t)args.gidx[jc] : jc;
        if (HASW) I.e[c] = args.eid ? (int64_t)args.eid[jc] : jc;
      }
    };
    Ids cur;
    load_ids(wa, cur);
    for (int64_t j0 = wa; j0 < wb; j0 += kSlotUnroll * kChunk) {
      float val[kSlotUnroll][4], rs[kSlotUnroll];
      typename IO::raw_t x[kSlotUnroll];
#pragma unroll
      for (int c = 0; c < kSlotUnroll; ++c) {
        x[c] = IO::load(args.u + cur.g[c] * feat + sub, ln);
        if (EPI) rs[c] = args.row_scale ? args.row_scale[cur.r[c]] : 1.0f;
        if (HASW) {
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            // the weight of feature sub + v L; dead features: any valid weight
            const int h = min((sub + (v << LS)) / args.dph, args.heads - 1);
            val[c][v] = args.w[cur.e[c] * args.heads + h];
          }
        }
      }
      int r[kSlotUnroll], rn[kSlotUnroll];
#pragma unroll
      for (int c = 0; c < kSlotUnroll; ++c) {
        r[c] = cur.r[c];
        rn[c] = cur.rn[c];
      }
      if (j0 + kSlotUnroll * kChunk < wb) load_ids(j0 + kSlotUnroll * kChunk, cur);
#pragma unroll
      for (int c = 0; c < kSlotUnroll; ++c) {
        const int64_t c0 = j0 + c * kChunk;   // uniform
        if (c0 >= wb) break;
        const bool valid = c0 + slot_lane < wb;
        float xf[4];
        IO::widen(x[c], xf);
        int key = valid ? r[c] : -2;         // lanes past the range: a row id no slot has
        float acc[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const float m = HASW ? bin_apply<BOP>(xf[v], val[c][v]) : xf[v];
          acc[v] = valid ? m : 0.0f;
        }
        if (slot_lane == 0 && key == carry_key) {
#pragma unroll
          for (int v = 0; v < 4; ++v) acc[v] = carry[v] + acc[v];
        }
        // inclusive segmented sum over the slots of the chunk
        if (L == 1) slots_scan16<1>(key, acc, live);
        slots_scan16<2>(key, acc, live);
        slots_scan16<4>(key, acc, live);
        slots_scan16<8>(key, acc, live);
        slots_row_carry<1, L>(key, acc, live, lane);
        slots_row_carry<2, L>(key, acc, live, lane);
        slots_row_carry<3, L>(key, acc, live, lane);
        const bool is_end = valid && rn[c] != key;
        if (is_end) {
          float st[SF];
#pragma unroll
          for (int v = 0; v < 4; ++v) st[v] = acc[v];
          if (EPI) st[4] = rs[c];
          if (key == first_key && first_open) {   // the piece of a row that began before this range
#pragma unroll
            for (int i = 0; i < SF; ++i) piece[wave][0][sub][i] = st[i];
            flags[wave].has_a = 1;
            flags[wave].row_a = key;
          } else {
            P::emit(args, out, key, feat, sub, st);
          }
        }
        // the segment of the last slot runs on into the next chunk (or past the range)
        const int last = (int)min((int64_t)kChunk - 1, wb - 1 - c0) << LS;   // its first lane, uniform
        const bool open = !__builtin_amdgcn_readlane((int)is_end, last);
        carry_key = open ? __builtin_amdgcn_readlane(key, last) : -1;
#pragma unroll
        for (int v = 0; v < 4; ++v) carry[v] = slots_from<L>(acc[v], last, lane);
        if (EPI) carry_scale = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(rs[c]), last));
      }
    }
    if (carry_key != -1 && lane < L) {       // the range ends inside a row
      const bool through = carry_key == first_key && first_open;   // ... that also began before it
      float *dst = piece[wave][through ? 0 : 1][sub];
#pragma unroll
      for (int v = 0; v < 4; ++v) dst[v] = carry[v];
      if (EPI) dst[4] = carry_scale;
      if (through) {
        flags[wave].has_a = flags[wave].a_open = 1;
        flags[wave].row_a = carry_key;
      } else {
        flags[wave].has_b = 1;
        flags[wave].row_b = carry_key;
      }
    }
  }
  __syncthreads();
  if (lane >= L || wa >= wb) return;
  // the pieces of the workgroup's wavefronts, chained as runs_kernel chains its runs
  auto chain_into = [&](int i, float (&acc)[SF]) -> bool {
    int j = i - 1;
    while (j >= 0 && flags[j].has_a && flags[j].a_open) --j;
    const bool starts_inside = j >= 0;
    if (starts_inside) {
#pragma unroll
      for (int q = 0; q < SF; ++q) acc[q] = piece[j][1][sub][q];
    } else {
      P::init(acc);
    }
    for (int g = j + 1; g <= i; ++g) P::merge(acc, piece[g][0][sub]);
    return starts_inside;
  };
  float *const gp = partial + ((int64_t)blockIdx.x * 2 * L + sub) * SF;   // slot 1: L * SF further
  const int64_t slots_left = geo.n_edges - ((int64_t)blockIdx.x << wg_shift);
  const int last_wave = (int)min((int64_t)kWaves, (slots_left + wave_slots - 1) / wave_slots) - 1;
  const bool has_a = flags[wave].has_a, a_open = flags[wave].a_open, has_b = flags[wave].has_b;
  if (has_a && !a_open) {
    float acc[SF];
    if (chain_into(wave, acc)) {
      P::emit(args, out, flags[wave].row_a, feat, sub, acc);
    } else {
#pragma unroll
      for (int q = 0; q < SF; ++q) gp[q] = acc[q];
    }
  }
  if (wave == last_wave) {
    if (has_b) {
#pragma unroll
      for (int q = 0; q < SF; ++q) gp[L * SF + q] = piece[wave][1][sub][q];
    } else if (has_a && a_open) {
      float acc[SF];
      const bool inside = chain_into(wave, acc);
      float *p = gp + (inside ? L * SF : 0);
#pragma unroll
      for (int q = 0; q < SF; ++q) p[q] = acc[q];
    }
  }
}

// Slots per workgroup: a power of two from 256 to 4096, for about 2048 workgroups
// (measured on 11.6 M edges, one feature, us by slots per workgroup: 256: 189, 512:
// 129, 1024: 97, 2048: 93, 4096: 95, 8192: 98, 16384: 120; on 1 M edges 1024 slots, 977
// workgroups: 16 against 20 with 256 slots); never fewer slots than four runs of the
// run schedule, whose workspace bound the caller sized.
// Where the lanes-per-slot kernel is the faster one: rows of up to four features
// everywhere (11.6 M edges, us: copy_u with one feature 129 -> 93, three 165 -> 104;
// 108 k edges: three features 22 -> 14); five to seven features, with two lanes per slot
// and so twice the chunks, on small graphs only (108 k edges 21 -> 14; 1 M edges 23 -> 26;
// eight features tile 16-byte accesses and are as fast on the run schedule).
inline bool slots_preferred(int64_t n_edges, int64_t feat) {
  return feat <= 4 || (feat <= 7 && n_edges <= 300000);
}

template <typename T, int BOP, int LS, bool EPI = false, int ACT = GA_ACT_NONE>
int launch_spmm_slots(const int32_t *pointer, const int32_t *row_of_slot, const int32_t *gidx,
                      const int32_t *eid, const void *u, const float *w, void *out,
                      int64_t n_rows, int64_t n_edges, int feat, int heads, float *partial,
                      hipStream_t stream, const float *row_scale = nullptr,
                      size_t partial_bytes = SIZE_MAX) {
  typedef SpmmPolicy<T, 4, GA_SUM, BOP, true, EPI, ACT> P;
  constexpr int SF = P::kState;
  constexpr int L = 1 << LS;
  typename P::Args args{gidx, eid, (const T *)u, w, heads, feat / heads, false, LS, row_scale};
  RunGeom geo;
  int wg_shift = ilog2_ceil((uint64_t)((n_edges + 2047) / 2048));
  const int floor_shift = std::max(8, run_shift_for(n_edges, feat) + 2);
  wg_shift = std::min(std::max(wg_shift, floor_shift), std::max(12, floor_shift));
  geo.tpr_shift = LS;
  geo.run_shift = wg_shift - 8 + LS;       // the second kernel's slots per workgroup: run << (8 - LS)
  geo.lanes_total = L;
  geo.feat = feat;
  geo.n_edges = n_edges;
  geo.n_rows = n_rows;
  const int64_t n_wg = (n_edges + ((int64_t)1 << wg_shift) - 1) >> wg_shift;
  geo.n_runs = n_wg * (kBlock >> LS);
  geo.n_wg = n_wg;
  const int G = kBlock >> LS;              // rows per block of the trailing blocks and of the second kernel
  const int64_t row_blocks = (n_rows + G - 1) / G;
  if (n_wg + row_blocks > 0x7fffffff) return GA_EUNSUPPORTED;
  if ((size_t)n_wg * 2 * L * SF * sizeof(float) > partial_bytes) return GA_EWORKSPACE;
  hipLaunchKernelGGL((slots_kernel<P, BOP, LS>), dim3((unsigned)(n_wg + row_blocks)), dim3(kBlock),
                     0, stream, args, pointer, row_of_slot, (T *)out, partial, geo);
  const int64_t fix_blocks = (n_wg + G - 1) / G;
  hipLaunchKernelGGL((runs_fixup_kernel<P>), dim3((unsigned)fix_blocks), dim3(kBlock),
                     (size_t)kBlock * SF * sizeof(float), stream, args, pointer, row_of_slot,
                     partial, (T *)out, geo, n_wg, (int)fix_blocks);
  return launch_status();
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
  // sums of rows of up to eight features: one or two lanes per slot
  if (reduce == GA_SUM && n_edges > 0 && ga::slots_preferred(n_edges, feat)) {
#define GA_SPMM_SLOTS(T, B)                                                                   \
  do {                                                                                        \
    if (feat <= 4)                                                                            \
      return ga::launch_spmm_slots<T, B, 0>(pointer, row_of_slot, gidx, eid, u, w, out,       \
                                            n_rows, n_edges, (int)feat, (int)heads, partial,  \
                                            s, nullptr, workspace_bytes);                     \
    return ga::launch_spmm_slots<T, B, 1>(pointer, row_of_slot, gidx, eid, u, w, out, n_rows, \
                                          n_edges, (int)feat, (int)heads, partial, s,         \
                                          nullptr, workspace_bytes);                          \
  } while (0)
#define GA_SPMM_SLOTS_T(T)                                  \
  switch (bop) {                                            \
    case GA_U_MUL_E: GA_SPMM_SLOTS(T, GA_U_MUL_E);          \
    case GA_U_ADD_E: GA_SPMM_SLOTS(T, GA_U_ADD_E);          \
    case GA_U_SUB_E: GA_SPMM_SLOTS(T, GA_U_SUB_E);          \
    case GA_U_DIV_E: GA_SPMM_SLOTS(T, GA_U_DIV_E);          \
    default: GA_SPMM_SLOTS(T, 0);                           \
  }
    if (dtype == GA_F32) GA_SPMM_SLOTS_T(float)
    GA_SPMM_SLOTS_T(ga::bf16_t)
#undef GA_SPMM_SLOTS_T
#undef GA_SPMM_SLOTS
  }
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
  if (n_edges > 0 && ga::slots_preferred(n_edges, feat)) {   // one or two lanes per slot
#define GA_SPMM_SLOTS_EPI(T, ACT)                                                                 \
  do {                                                                                            \
    if (feat <= 4)                                                                                \
      return ga::launch_spmm_slots<T, 0, 0, true, ACT>(pointer, row_of_slot, gidx, eid, u,        \
                                                       nullptr, out, n_rows, n_edges, (int)feat,  \
                                                       1, partial, s, row_scale, workspace_bytes); \
    return ga::launch_spmm_slots<T, 0, 1, true, ACT>(pointer, row_of_slot, gidx, eid, u, nullptr, \
                                                     out, n_rows, n_edges, (int)feat, 1, partial, \
                                                     s, row_scale, workspace_bytes);              \
  } while (0)
#define GA_SPMM_SLOTS_EPI_T(T)                                        \
  do {                                                                \
    if (activation == GA_ACT_RELU) GA_SPMM_SLOTS_EPI(T, GA_ACT_RELU); \
    if (activation == GA_ACT_ELU) GA_SPMM_SLOTS_EPI(T, GA_ACT_ELU);   \
    GA_SPMM_SLOTS_EPI(T, GA_ACT_NONE);                                \
  } while (0)
    if (dtype == GA_F32) GA_SPMM_SLOTS_EPI_T(float);
    GA_SPMM_SLOTS_EPI_T(ga::bf16_t);
#undef GA_SPMM_SLOTS_EPI_T
#undef GA_SPMM_SLOTS_EPI
  }
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
