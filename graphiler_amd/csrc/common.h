// Shared device/host helpers for the gfx950 graph-primitive kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/graphiler_amd.h"

namespace ga {

constexpr int kWave = 64;      // CDNA wavefront width
constexpr int kBlock = 256;    // threads per workgroup used by the row kernels

typedef uint16_t bf16_t;  // raw bf16 storage

__device__ __forceinline__ float bf16_lo(uint32_t packed) {
  return __uint_as_float(packed << 16);
}
__device__ __forceinline__ float bf16_hi(uint32_t packed) {
  return __uint_as_float(packed & 0xffff0000u);
}
// fp32 -> bf16, round to nearest even, NaN kept quiet (same rounding as
// PyTorch's float -> bfloat16 conversion).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  return f32_to_bf16_bits(lo) | (f32_to_bf16_bits(hi) << 16);
}

// Sums over lane groups with DPP moves (all VALU, no LDS), result in every lane
// of the group: swaps inside quads, then the half-row mirror (8 lanes:
// 8j..8j+7) and the row mirror (16 lanes: 16j..16j+15).
__device__ __forceinline__ float row8_sum(float v) {
  v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
  v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
  v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x141, 0xF, 0xF, true));  // row_half_mirror
  return v;
}
__device__ __forceinline__ float row16_sum(float v) {
  v = row8_sum(v);
  v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x140, 0xF, 0xF, true));  // row_mirror
  return v;
}

// Row fragment I/O: VEC consecutive features of element type T, widened to
// fp32 registers.  VEC > 1 uses one 16-byte access.
template <typename T, int VEC>
struct Frag;

template <>
struct Frag<float, 4> {
  typedef float4 raw_t;
  static __device__ __forceinline__ raw_t load(const float *p) {
    return *reinterpret_cast<const float4 *>(p);
  }
  static __device__ __forceinline__ void widen(const raw_t &r, float (&f)[4]) {
    f[0] = r.x; f[1] = r.y; f[2] = r.z; f[3] = r.w;
  }
  static __device__ __forceinline__ void store(float *p, const float (&f)[4]) {
    *reinterpret_cast<float4 *>(p) = make_float4(f[0], f[1], f[2], f[3]);
  }
};

template <>
struct Frag<float, 1> {
  typedef float raw_t;
  static __device__ __forceinline__ raw_t load(const float *p) { return *p; }
  static __device__ __forceinline__ void widen(const raw_t &r, float (&f)[1]) {
    f[0] = r;
  }
  static __device__ __forceinline__ void store(float *p, const float (&f)[1]) {
    *p = f[0];
  }
};

template <>
struct Frag<bf16_t, 8> {
  typedef uint4 raw_t;
  static __device__ __forceinline__ raw_t load(const bf16_t *p) {
    return *reinterpret_cast<const uint4 *>(p);
  }
  static __device__ __forceinline__ void widen(const raw_t &r, float (&f)[8]) {
    f[0] = bf16_lo(r.x); f[1] = bf16_hi(r.x);
    f[2] = bf16_lo(r.y); f[3] = bf16_hi(r.y);
    f[4] = bf16_lo(r.z); f[5] = bf16_hi(r.z);
    f[6] = bf16_lo(r.w); f[7] = bf16_hi(r.w);
  }
  static __device__ __forceinline__ void store(bf16_t *p, const float (&f)[8]) {
    uint4 r;
    r.x = pack_bf16(f[0], f[1]);
    r.y = pack_bf16(f[2], f[3]);
    r.z = pack_bf16(f[4], f[5]);
    r.w = pack_bf16(f[6], f[7]);
    *reinterpret_cast<uint4 *>(p) = r;
  }
};

template <>
struct Frag<bf16_t, 1> {
  typedef bf16_t raw_t;
  static __device__ __forceinline__ raw_t load(const bf16_t *p) { return *p; }
  static __device__ __forceinline__ void widen(const raw_t &r, float (&f)[1]) {
    f[0] = bf16_lo(r);
  }
  static __device__ __forceinline__ void store(bf16_t *p, const float (&f)[1]) {
    *p = (bf16_t)f32_to_bf16_bits(f[0]);
  }
};

// Row access of the row-reduction kernels.  RowIO<T, VEC, false> is Frag: the lane's
// VEC features are consecutive and move with one 16-byte access.  RowIO<T, VEC, true>
// is for rows that such accesses do not tile (feature count not a multiple of the
// vector, or unaligned storage): the lane's features lie one lane-group width apart
// (f0, f0 + stride, f0 + 2 stride, ...), so the lanes of a group read consecutive
// elements with each of their VEC element loads.  Features past the end of the row
// are read from the lane's first feature instead and never stored.
__device__ __forceinline__ float elem_to_f32(float x) { return x; }
__device__ __forceinline__ float elem_to_f32(bf16_t x) { return bf16_lo(x); }
__device__ __forceinline__ void f32_to_elem(float f, float &o) { o = f; }
__device__ __forceinline__ void f32_to_elem(float f, bf16_t &o) { o = (bf16_t)f32_to_bf16_bits(f); }

template <typename T, int VEC, bool SPREAD>
struct RowIO;

template <typename T, int VEC>
struct RowIO<T, VEC, false> {
  typedef typename Frag<T, VEC>::raw_t raw_t;
  struct lane_t {};
  static __device__ __forceinline__ lane_t lane(int, int) { return lane_t(); }
  static __device__ __forceinline__ raw_t load(const T *p, const lane_t &) {
    return Frag<T, VEC>::load(p);
  }
  static __device__ __forceinline__ void widen(const raw_t &r, float (&f)[VEC]) {
    Frag<T, VEC>::widen(r, f);
  }
  static __device__ __forceinline__ void store(T *p, const float (&f)[VEC], const lane_t &) {
    Frag<T, VEC>::store(p, f);
  }
};

template <typename T, int VEC>
struct RowIO<T, VEC, true> {
  struct raw_t { T e[VEC]; };
  struct lane_t {
    int off[VEC];   // element offset of feature v from the lane's first feature
    int live;       // features of this lane that lie inside the row
  };
  // stride = 1 << stride_shift features between a lane's features; `left` = features
  // from the lane's first one to the end of the row (> 0 for a live lane)
  static __device__ __forceinline__ lane_t lane(int stride_shift, int left) {
    lane_t l;
    const int n = (left + (1 << stride_shift) - 1) >> stride_shift;
    l.live = n < VEC ? n : VEC;
#pragma unroll
    for (int v = 0; v < VEC; ++v) l.off[v] = v < l.live ? v << stride_shift : 0;
    return l;
  }
  static __device__ __forceinline__ raw_t load(const T *p, const lane_t &l) {
    raw_t r;
#pragma unroll
    for (int v = 0; v < VEC; ++v) r.e[v] = p[l.off[v]];
    return r;
  }
  static __device__ __forceinline__ void widen(const raw_t &r, float (&f)[VEC]) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) f[v] = elem_to_f32(r.e[v]);
  }
  static __device__ __forceinline__ void store(T *p, const float (&f)[VEC], const lane_t &l) {
#pragma unroll
    for (int v = 0; v < VEC; ++v)
      if (v < l.live) f32_to_elem(f[v], p[l.off[v]]);
  }
};

// Loads through a buffer descriptor: address = descriptor base + 32-bit lane offset
// + 32-bit scalar offset, formed by the load unit.  The lane offsets are fixed for
// the whole kernel and the scalar offset advances with the slice, so a load costs no
// address arithmetic (plain pointers cost a 64-bit vector add per load here).  The
// scalar offset takes no part in the descriptor's range check, so the code keeps
// every address valid itself.
typedef __amdgpu_buffer_rsrc_t rsrc_t;
__device__ __forceinline__ rsrc_t make_rsrc(const void *base, uint64_t bytes) {
  const uint32_t n = bytes > 0xffffffffull ? 0xffffffffu : (uint32_t)bytes;
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)n, 0x00020000);
}
template <int VK> struct BufLoad;
template <> struct BufLoad<4> {
  static __device__ __forceinline__ float4 at(rsrc_t r, uint32_t lane_off, uint32_t scalar_off) {
    return __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(r, lane_off, scalar_off, 0));
  }
};
template <> struct BufLoad<2> {
  static __device__ __forceinline__ float2 at(rsrc_t r, uint32_t lane_off, uint32_t scalar_off) {
    return __builtin_bit_cast(float2, __builtin_amdgcn_raw_buffer_load_b64(r, lane_off, scalar_off, 0));
  }
};
template <> struct BufLoad<1> {
  static __device__ __forceinline__ float at(rsrc_t r, uint32_t lane_off, uint32_t scalar_off) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, lane_off, scalar_off, 0));
  }
};

// ---- activations applied to fp32 rows before they are rounded and stored ----

// elu with alpha = 1 (torch.nn.functional.elu computes expm1 for x <= 0).  exp(x) - 1
// loses its leading digits near zero, so a short series takes over above -1/8: its
// first dropped term is x^7 / 5040, below 2^-24 |x| there; below -1/8 the result is at
// least 0.117 in magnitude and the rounding of exp (about 1e-7) is under 1e-6 of it.
__device__ __forceinline__ float elu(float x) {
  const float e = __expf(x) - 1.0f;
  const float p = x * (1.0f + x * (0.5f + x * (1.0f / 6 + x * (1.0f / 24 + x * (1.0f / 120 + x * (1.0f / 720))))));
  const float neg = x > -0.125f ? p : e;
  return x > 0.0f ? x : neg;          // NaN: the comparisons fail, neg = e = NaN
}
__device__ __forceinline__ float relu_keep_nan(float x) {
  return x > 0.0f ? x : (x != x ? x : 0.0f);
}

// ---- host side -----------------------------------------------------------

inline int ilog2_floor(uint64_t x) {
  int s = 0;
  while (x > 1) { x >>= 1; ++s; }
  return s;
}
inline int ilog2_ceil(uint64_t x) {
  int s = ilog2_floor(x);
  return ((uint64_t)1 << s) < x ? s + 1 : s;
}
inline bool aligned(const void *p, size_t a) {
  return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0;
}
inline int launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? GA_OK : (int)e;
}

// log2 of the slots per run of the load-balanced row reductions.  Every lane
// group walks exactly one run, so the value trades scheduling slack and
// workspace (two partial rows per run) against per-run overhead.  It depends
// on the edge count and the feature width only, so the workspace query and the
// launch agree.
int run_shift_for(int64_t n_edges, int64_t feat);

}  // namespace ga
