// Sort keys of the LRU order: least recently used first, ties by lowest slot,
// i.e. the order of torch.argsort(page_access_time, stable=True) in
// dram_attention/lru_triton_kernel.py:175-177 of the reference.
#pragma once

#include "select.hpp"

namespace da {

template <typename TimeT>
__device__ __forceinline__ uint32_t time_order_key(TimeT v);
template <>
__device__ __forceinline__ uint32_t time_order_key<float>(float v) { return float_order_key(v); }
template <>
__device__ __forceinline__ uint32_t time_order_key<int32_t>(int32_t v) {
  return (uint32_t)v ^ 0x80000000u;
}

// "largest key" = smallest access time, ties by lowest slot: the order of
// torch.argsort(page_access_time, stable=True).
template <typename TimeT>
struct LeastRecentKey {
  const TimeT *time;
  __device__ __forceinline__ uint32_t operator()(int i) const {
    return ~time_order_key<TimeT>(time[i]);
  }
  __device__ __forceinline__ void load4(int i, uint32_t *k) const {
    TimeT v[4];
    if (((uintptr_t)time & 15) == 0) {
      *(u32x4 *)v = *(const u32x4 *)(time + i);
    } else {
#pragma unroll
      for (int x = 0; x < 4; ++x) v[x] = time[i + x];
    }
#pragma unroll
    for (int x = 0; x < 4; ++x) k[x] = ~time_order_key<TimeT>(v[x]);
  }
};

}  // namespace da
