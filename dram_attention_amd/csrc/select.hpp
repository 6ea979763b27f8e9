// Block-wide ordered selection in LDS: the k largest of n 32-bit keys, ties by
// lowest index, returned sorted (key descending, index ascending).
//
// Used twice: page top-k (keys = order-preserving image of the fp32 scores;
// replaces the full torch.argsort of dram_attention/topk_selector.py:61) and
// LRU victim choice (keys = inverted access times, so "largest" = least
// recently used; replaces the full stable argsort of
// dram_attention/lru_triton_kernel.py:170, of which only a prefix is consumed).
//
// Method: MSB-first radix select, 8 bits per pass, on the 32-bit key to find
// the k-th largest key T; one compaction pass gathers every key > T plus the
// lowest-index keys == T into LDS as 64-bit (key, ~index) words; a bitonic
// network sorts those.  Histograms are replicated 32x so that clustered keys
// (bf16-rounded scores share their top digits) do not serialise LDS atomics.
#pragma once

#include "common.hpp"

namespace da {

constexpr int kSelThreads = 1024;
constexpr int kSelWaves = kSelThreads / 64;
constexpr int kHistCopies = 32;
constexpr int kSelMaxK = 8192;  // survivors sorted in LDS: 8 bytes each

struct SelectShared {
  // the histogram phase and the survivor array never overlap in time
  union {
    uint32_t hist[256 * kHistCopies];  // 32 KiB
    uint64_t sel[kSelMaxK];            // 64 KiB
  };
  uint32_t total[256];
  uint32_t chunk_eq[kSelWaves];   // per-wave counts for the block scans
  uint32_t chunk_gt[kSelWaves];
  uint32_t digit;      // digit chosen by the current pass
  uint32_t remaining;  // how many keys are still wanted from the chosen bin
  uint32_t n_gt;       // running count of survivors with key > T
  uint32_t eq_base;    // equal keys seen in earlier rounds of the compaction
};

__device__ __forceinline__ int next_pow2(int v) {
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}

// KeyFn: uint32_t operator()(int i) for 0 <= i < n.  Every thread of the
// 1024-thread block must call this with the same n and k (1 <= k <= n,
// k <= kSelMaxK).  On return sm.sel[0..k) holds the winners, best first, as
// (key << 32) | (0xffffffff - index); all threads have passed a barrier.
template <typename KeyFn>
__device__ void select_sorted(const KeyFn &key_of, int n, int k, SelectShared &sm) {
  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = t >> 6;

  for (int i = t; i < 256 * kHistCopies; i += kSelThreads) sm.hist[i] = 0;
  if (t == 0) {
    sm.remaining = (uint32_t)k;
    sm.n_gt = 0;
    sm.eq_base = 0;
  }
  __syncthreads();

  uint32_t prefix = 0;  // the digits of T fixed so far (high bits)
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
    for (int i = t; i < n; i += kSelThreads) {
      const uint32_t key = key_of(i);
      const bool live = pass == 0 || (key >> (shift + 8)) == prefix;
      if (live) atomicAdd(&sm.hist[((key >> shift) & 255u) * kHistCopies + (lane & 31)], 1u);
    }
    __syncthreads();
    if (t < 256) {
      uint32_t s = 0;
#pragma unroll
      for (int c = 0; c < kHistCopies; ++c) {
        const int cc = (c + t) & (kHistCopies - 1);  // rotate: one bank per lane
        s += sm.hist[t * kHistCopies + cc];
        sm.hist[t * kHistCopies + cc] = 0;
      }
      sm.total[t] = s;
    }
    __syncthreads();
    if (wave == 0) {
      // lane l owns bins 255-4l .. 252-4l, i.e. the bins in descending order
      const int b0 = 255 - 4 * lane;
      const uint32_t c0 = sm.total[b0], c1 = sm.total[b0 - 1], c2 = sm.total[b0 - 2],
                     c3 = sm.total[b0 - 3];
      const uint32_t mine = c0 + c1 + c2 + c3;
      uint32_t incl = mine;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const uint32_t up = __shfl_up(incl, d, 64);
        if (lane >= d) incl += up;
      }
      const uint32_t excl = incl - mine;
      const uint32_t want = sm.remaining;
      if (excl < want && want <= incl) {
        uint32_t above = excl;
        int bin = b0;
        if (above + c0 < want) {
          above += c0;
          bin = b0 - 1;
          if (above + c1 < want) {
            above += c1;
            bin = b0 - 2;
            if (above + c2 < want) {
              above += c2;
              bin = b0 - 3;
            }
          }
        }
        sm.digit = (uint32_t)bin;
        sm.remaining = want - above;  // still needed from inside `bin`
      }
    }
    __syncthreads();
    prefix = (prefix << 8) | sm.digit;
  }
  const uint32_t thresh = prefix;        // the k-th largest key
  const uint32_t n_eq = sm.remaining;    // how many keys == thresh to keep
  const uint32_t n_gt_total = (uint32_t)k - n_eq;
  __syncthreads();  // hist is dead from here on; sel may be written

  // Compaction in index order, 1024 indices per round.  Keys > T take any
  // free place among the first n_gt_total; keys == T are kept while their
  // running rank (by index) is below n_eq and go behind the larger keys.
  for (int base = 0; base < n; base += kSelThreads) {
    const int i = base + t;
    uint32_t key = 0;
    bool gt = false, eq = false;
    if (i < n) {
      key = key_of(i);
      gt = key > thresh;
      eq = key == thresh;
    }
    const uint64_t m_gt = __ballot(gt), m_eq = __ballot(eq);
    const uint64_t below = lane == 0 ? 0ull : (~0ull >> (64 - lane));
    if (lane == 0) {
      sm.chunk_gt[wave] = (uint32_t)__popcll(m_gt);
      sm.chunk_eq[wave] = (uint32_t)__popcll(m_eq);
    }
    __syncthreads();
    uint32_t gt_before = sm.n_gt, eq_before = sm.eq_base, gt_round = 0, eq_round = 0;
#pragma unroll
    for (int w = 0; w < kSelWaves; ++w) {
      const uint32_t g = sm.chunk_gt[w], e = sm.chunk_eq[w];
      if (w < wave) {
        gt_before += g;
        eq_before += e;
      }
      gt_round += g;
      eq_round += e;
    }
    const uint64_t word = ((uint64_t)key << 32) | (uint64_t)(0xffffffffu - (uint32_t)i);
    if (gt) sm.sel[gt_before + (uint32_t)__popcll(m_gt & below)] = word;
    if (eq) {
      const uint32_t rank = eq_before + (uint32_t)__popcll(m_eq & below);
      if (rank < n_eq) sm.sel[n_gt_total + rank] = word;
    }
    __syncthreads();
    if (t == 0) {
      sm.n_gt += gt_round;
      sm.eq_base += eq_round;
    }
    __syncthreads();
  }

  // Bitonic sort, descending, on the padded power-of-two prefix of sel.
  const int n2 = next_pow2(k);
  for (int i = k + t; i < n2; i += kSelThreads) sm.sel[i] = 0;  // below every real word
  __syncthreads();
  for (int size = 2; size <= n2; size <<= 1) {
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      for (int p = t; p < (n2 >> 1); p += kSelThreads) {
        const int lo = ((p / stride) * stride * 2) + (p % stride);
        const int hi = lo + stride;
        const bool desc = (lo & size) == 0;
        const uint64_t a = sm.sel[lo], b = sm.sel[hi];
        if ((a < b) == desc) {
          sm.sel[lo] = b;
          sm.sel[hi] = a;
        }
      }
      __syncthreads();
    }
  }
}

__device__ __forceinline__ uint32_t sel_index(uint64_t word) {
  return 0xffffffffu - (uint32_t)word;
}

}  // namespace da
