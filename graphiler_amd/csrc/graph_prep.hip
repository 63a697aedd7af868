// Graph preparation on the device: stable grouping of an edge list by one
// endpoint (or of items by type) into pointer / neighbour / edge-id columns,
// the layout python/graphiler/utils/setup.py:116-146 builds on the host with a
// Python prefix-sum loop and DGL's in_edges / out_edges.
//
// Order contract (what the operators rely on): slots of one key are contiguous,
// keys ascend, and inside a key the edge ids ascend, i.e. a STABLE sort of the
// edge ids by key.  Steps, all on the caller's stream:
//   1. narrow the int64 keys to int32 and check their range,
//   2. stable LSD radix sort of (key, edge id) pairs over the bits the keys
//      use (rocPRIM device radix sort: a library sort, like a library GEMM),
//   3. pointer[v] = first slot whose key is >= v, by binary search in the sorted
//      keys (no counting with atomics: a hub node of a power-law graph would
//      serialise tens of thousands of them on one address),
//   4. gather the other endpoint through the sorted edge ids.
#include "common.h"

#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>

namespace ga {
namespace {

__global__ __launch_bounds__(kBlock) void prep_keys_kernel(
    const int64_t *__restrict__ key, int64_t n_keys, int64_t n_items,
    int32_t *__restrict__ key32, int32_t *__restrict__ ids,
    int32_t *__restrict__ status) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= n_items) return;
  int64_t k = key[i];
  if (k < 0 || k >= n_keys) {
    *status = 1;          // every writer stores the same value
    k = 0;                // keeps the remaining steps inside their arrays
  }
  key32[i] = (int32_t)k;
  ids[i] = (int32_t)i;
}

// pointer[v] = number of items with key < v, v in [0, n_keys]
__global__ __launch_bounds__(kBlock) void pointer_kernel(
    const int32_t *__restrict__ key_sorted, int64_t n_keys, int64_t n_items,
    int32_t *__restrict__ pointer) {
  const int64_t v = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (v > n_keys) return;
  int64_t lo = 0, hi = n_items;          // first index with key_sorted[index] >= v
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if ((int64_t)key_sorted[mid] < v) lo = mid + 1; else hi = mid;
  }
  pointer[v] = (int32_t)lo;
}

__global__ __launch_bounds__(kBlock) void gather_other_kernel(
    const int64_t *__restrict__ other, const int32_t *__restrict__ ids,
    int64_t n_items, int32_t *__restrict__ nbr) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= n_items) return;
  nbr[i] = (int32_t)other[ids[i]];
}

__global__ __launch_bounds__(kBlock) void fill_zero_kernel(int32_t *p, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i < n) p[i] = 0;
}

inline size_t round_up(size_t v) { return (v + 255) & ~(size_t)255; }

struct PrepLayout {
  size_t key32, key_sorted, ids, temp, total;
  size_t temp_bytes;
};

int end_bit_for(int64_t n_keys) {
  int bits = 1;
  while (bits < 31 && ((int64_t)1 << bits) < n_keys) ++bits;
  return bits;
}

// Sizes only; nothing is launched (rocPRIM's calls with a null temporary
// buffer just report what they need).
int prep_layout(int64_t n_keys, int64_t n_items, PrepLayout &L) {
  size_t sort_bytes = 0;
  int32_t *k = nullptr;
  if (n_items > 0) {
    hipError_t e = rocprim::radix_sort_pairs(nullptr, sort_bytes, k, k, k, k,
                                             (size_t)n_items, 0, end_bit_for(n_keys));
    if (e != hipSuccess) return (int)e;
  }
  L.temp_bytes = sort_bytes;
  size_t off = 0;
  L.key32 = off;       off += round_up((size_t)n_items * 4);
  L.key_sorted = off;  off += round_up((size_t)n_items * 4);
  L.ids = off;         off += round_up((size_t)n_items * 4);
  L.temp = off;        off += round_up(L.temp_bytes);
  L.total = off;
  return GA_OK;
}

}  // namespace
}  // namespace ga

extern "C" {

size_t ga_group_edges_workspace_bytes(int64_t n_keys, int64_t n_items) {
  if (n_keys < 0 || n_items < 0 || n_keys > 0x7ffffffe || n_items > 0x7fffffff) return 0;
  ga::PrepLayout L;
  if (ga::prep_layout(n_keys, n_items, L) != GA_OK) return 0;
  return L.total;
}

int ga_group_edges(const int64_t *key, const int64_t *other, int64_t n_keys,
                   int64_t n_items, int32_t *pointer, int32_t *nbr, int32_t *eid,
                   int32_t *status, void *workspace, size_t workspace_bytes,
                   ga_stream_t stream) {
  using namespace ga;
  if (n_keys < 0 || n_items < 0 || n_keys > 0x7ffffffe || n_items > 0x7fffffff)
    return GA_EINVAL;
  if (!pointer || !status) return GA_EINVAL;
  if (n_items > 0 && (!key || !eid || n_keys == 0)) return GA_EINVAL;
  if (nbr && !other) return GA_EINVAL;
  PrepLayout L;
  const int rc = prep_layout(n_keys, n_items, L);
  if (rc != GA_OK) return rc;
  if (!workspace || workspace_bytes < L.total || !aligned(workspace, 256)) return GA_EWORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  char *ws = (char *)workspace;
  int32_t *key32 = (int32_t *)(ws + L.key32);
  int32_t *key_sorted = (int32_t *)(ws + L.key_sorted);
  int32_t *ids = (int32_t *)(ws + L.ids);
  void *temp = ws + L.temp;

  // the status word starts at 0; a fill kernel rather than a memset node keeps
  // the sequence capturable
  hipLaunchKernelGGL(fill_zero_kernel, dim3(1), dim3(kBlock), 0, s, status, (int64_t)1);
  if (n_items > 0) {
    const int64_t blocks = (n_items + kBlock - 1) / kBlock;
    hipLaunchKernelGGL(prep_keys_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, s, key,
                       n_keys, n_items, key32, ids, status);
    size_t tb = L.temp_bytes;
    hipError_t e = rocprim::radix_sort_pairs(temp, tb, key32, key_sorted, ids, eid,
                                             (size_t)n_items, 0, end_bit_for(n_keys), s);
    if (e != hipSuccess) return (int)e;
  }
  const int64_t pblocks = (n_keys + 1 + kBlock - 1) / kBlock;
  hipLaunchKernelGGL(pointer_kernel, dim3((unsigned)pblocks), dim3(kBlock), 0, s, key_sorted,
                     n_keys, n_items, pointer);
  if (n_items > 0 && nbr) {
    const int64_t blocks = (n_items + kBlock - 1) / kBlock;
    hipLaunchKernelGGL(gather_other_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, s, other,
                       eid, n_items, nbr);
  }
  return launch_status();
}

}  // extern "C"
