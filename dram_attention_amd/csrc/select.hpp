// Block-wide ordered selection in LDS: the k largest of n 32-bit keys, ties by
// lowest index, returned as indices sorted by (key descending, index ascending).
//
// Used twice: page top-k (keys = order-preserving image of the fp32 scores;
// replaces the full torch.argsort of dram_attention/topk_selector.py:61) and
// LRU victim choice (keys = inverted access times, so "largest" = least
// recently used; replaces the full stable argsort of
// dram_attention/lru_triton_kernel.py:170, of which only a prefix is consumed).
//
// Method (one 1024-thread workgroup; barriers and LDS round trips are the cost
// that matters, so every phase is built to need few of them):
//   1. a thread owns a CONTIGUOUS run of up to 16 indices and keeps those keys
//      in registers (16-byte loads); thread order is index order;
//   2. MSB-first radix select, 8 bits per pass, finds the k-th largest key T.
//      Histograms are replicated 32x so that clustered keys (rounded scores
//      share their top digits) do not serialise the LDS atomics; if all keys
//      agree in their low 16 bits (bf16-rounded scores) two passes suffice;
//   3. one block-wide scan of per-thread counts places every key > T and the
//      lowest-index keys == T into LDS as 64-bit (key, ~index) words;
//   4. the k survivors are ordered by rank counting (k <= 512: thread (e, slice)
//      counts the words of its slice that beat word e; 32-bit words when key and
//      index fit) or by a bitonic network (larger k).
// Rows longer than 16384 keys are processed in segments of 16384 and re-read
// from memory in every pass.
#pragma once

#include "common.hpp"

namespace da {

constexpr int kSelThreads = 1024;
constexpr int kSelWaves = kSelThreads / 64;
constexpr int kHistCopies = 32;
constexpr int kSelMaxK = 8192;     // survivors held in LDS: 8 bytes each
constexpr int kSelRegKeys = 16;    // keys cached per thread
constexpr int kSelRankSortMax = 512;

struct alignas(16) SelectShared {
  // the histogram phase and the survivor array never overlap in time
  union {
    uint32_t hist[256 * kHistCopies];  // 32 KiB
    uint64_t sel[kSelMaxK];            // 64 KiB
  };
  uint32_t idx_out[kSelMaxK];          // the result: winning indices, best first
  alignas(16) uint32_t w32[kSelRankSortMax + 4];   // compact sort words
  uint32_t rank[kSelRankSortMax];
  uint32_t total[256];
  uint32_t wave_gt[kSelWaves], wave_eq[kSelWaves];
  uint32_t digit;        // digit chosen by the current pass
  uint32_t remaining;    // how many keys are still wanted from the chosen bin
  uint32_t low_or, low_and;  // OR / AND over the low 16 bits of all keys
};

__device__ __forceinline__ int next_pow2(int v) {
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}

template <int kCtrl, int kRowMask>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, kCtrl, kRowMask, 0xf, false);
}
// Inclusive prefix sum over the 64 lanes of a wave, all on DPP operands.
__device__ __forceinline__ uint32_t wave_scan_inclusive(uint32_t v) {
  v += dpp_u32<0x111, 0xf>(v);  // row_shr:1
  v += dpp_u32<0x112, 0xf>(v);  // row_shr:2
  v += dpp_u32<0x114, 0xf>(v);  // row_shr:4
  v += dpp_u32<0x118, 0xf>(v);  // row_shr:8  -> scan inside each 16-lane row
  v += dpp_u32<0x142, 0xa>(v);  // row_bcast:15 into rows 1 and 3
  v += dpp_u32<0x143, 0xc>(v);  // row_bcast:31 into rows 2 and 3
  return v;
}

// KeyFn provides
//   uint32_t operator()(int i)            key of index i (0 <= i < n)
//   void load4(int i, uint32_t *k)        keys of i..i+3 (i % 4 == 0, i+3 < n)
// Every thread of the 1024-thread block must call this with the same n and k
// (1 <= k <= n, k <= kSelMaxK).  Returns a pointer into sm to the k winning
// indices, best first; all threads have passed a barrier.
//
// Slots past the end of the row are padded with key 0 (the smallest key) at
// the highest indices: they can never displace a real key, so no phase needs a
// validity test.  C = keys per thread per segment (4, 8 or 16).
template <int C, typename KeyFn>
__device__ const uint32_t *select_sorted_impl(const KeyFn &key_of, int n, int k,
                                              SelectShared &sm) {
  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = t >> 6;

  // geometry: thread t owns indices [s*seg_n + t*C, +C) of segment s
  constexpr int seg_n = C * kSelThreads;
  const int n_seg = (n + seg_n - 1) / seg_n;

  uint32_t kreg[C];
  auto load_segment = [&](int s) {
    const int i0 = s * seg_n + t * C;
    const int valid = n - i0;
#pragma unroll
    for (int u = 0; u < C; u += 4) {
      if (u + 4 <= valid) {
        key_of.load4(i0 + u, &kreg[u]);
      } else {
#pragma unroll
        for (int x = 0; x < 4; ++x) kreg[u + x] = u + x < valid ? key_of(i0 + u + x) : 0u;
      }
    }
  };

  uint32_t low_or = 0, low_and = 0xffffu;
  for (int s = n_seg - 1; s >= 0; --s) {  // ends with segment 0 in registers
    load_segment(s);
    const int real = n - (s * seg_n + t * C);
#pragma unroll
    for (int u = 0; u < C; ++u) {
      if (u < real) {  // padding must not spoil the low-bits test
        low_or |= kreg[u];
        low_and &= kreg[u];
      }
    }
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) {
    low_or |= __shfl_xor(low_or, d, 64);
    low_and &= __shfl_xor(low_and, d, 64);
  }
  for (int i = t; i < 256 * kHistCopies; i += kSelThreads) sm.hist[i] = 0;
  if (t < kSelRankSortMax) sm.rank[t] = 0;
  if (t == 0) {
    sm.remaining = (uint32_t)k;
    sm.low_or = 0;
    sm.low_and = 0xffffu;
  }
  __syncthreads();
  if (lane == 0) {
    atomicOr(&sm.low_or, low_or & 0xffffu);
    atomicAnd(&sm.low_and, low_and & 0xffffu);
  }

  uint32_t prefix = 0;  // the digits of T fixed so far (high bits)
  int passes = 4;
  for (int pass = 0; pass < passes; ++pass) {
    const int shift = 24 - 8 * pass;
    for (int s = 0; s < n_seg; ++s) {
      if (n_seg > 1) load_segment(s);
#pragma unroll
      for (int u = 0; u < C; ++u) {
        const uint32_t key = kreg[u];
        if (pass == 0 || (key >> (shift + 8)) == prefix)
          atomicAdd(&sm.hist[((key >> shift) & 255u) * kHistCopies + (lane & (kHistCopies - 1))], 1u);
      }
    }
    __syncthreads();
    // all keys share their low 16 bits (rounded scores, small step counts):
    // the two low digits cannot separate anything
    if (pass == 0 && sm.low_or == sm.low_and) passes = 2;
    if (t < 256) {
      uint32_t s = 0;
#pragma unroll
      for (int cp = 0; cp < kHistCopies; ++cp) {
        const int cc = (cp + t) & (kHistCopies - 1);  // rotate: one bank per lane
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
      const uint32_t incl = wave_scan_inclusive(mine);
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
  const bool low_const = passes == 2;
  const uint32_t thresh = low_const ? (prefix << 16) | sm.low_or : prefix;  // k-th largest key
  const uint32_t n_eq = sm.remaining;                                       // keys == T to keep
  const uint32_t n_gt_total = (uint32_t)k - n_eq;
  // (the last barrier of the loop also retired every read of hist: sel may be written)

  // Compaction in index order = thread order.  Keys > T fill the first
  // n_gt_total places, keys == T follow while their rank is below n_eq.
  uint32_t gt_base = 0, eq_base = 0;
  for (int s = 0; s < n_seg; ++s) {
    if (n_seg > 1) load_segment(s);
    uint32_t gt_c = 0, eq_c = 0;
#pragma unroll
    for (int u = 0; u < C; ++u) {
      gt_c += kreg[u] > thresh ? 1u : 0u;
      eq_c += kreg[u] == thresh ? 1u : 0u;
    }
    const uint32_t gt_incl = wave_scan_inclusive(gt_c), eq_incl = wave_scan_inclusive(eq_c);
    if (lane == 63) {
      sm.wave_gt[wave] = gt_incl;
      sm.wave_eq[wave] = eq_incl;
    }
    __syncthreads();
    uint32_t gt_off = gt_base + gt_incl - gt_c, eq_off = eq_base + eq_incl - eq_c;
#pragma unroll
    for (int w = 0; w < kSelWaves; ++w) {
      const uint32_t g = sm.wave_gt[w], e = sm.wave_eq[w];
      if (w < wave) {
        gt_off += g;
        eq_off += e;
      }
      gt_base += g;
      eq_base += e;
    }
    const int i0 = s * seg_n + t * C;
#pragma unroll
    for (int u = 0; u < C; ++u) {
      const uint32_t key = kreg[u];
      const uint64_t word = ((uint64_t)key << 32) | (uint64_t)(0xffffffffu - (uint32_t)(i0 + u));
      if (key > thresh) sm.sel[gt_off++] = word;
      if (key == thresh) {
        if (eq_off < n_eq) sm.sel[n_gt_total + eq_off] = word;
        ++eq_off;
      }
    }
    __syncthreads();
  }

  if (k <= kSelRankSortMax) {
    // Rank counting: thread (e, slice) counts the words of its slice that beat
    // word e; all words are distinct, so the summed counts are a permutation.
    const int kpad = next_pow2(k);
    const int slices = kSelThreads / kpad;
    const int e = t % kpad, slice = t / kpad;
    const int per = (((k + slices - 1) / slices) + 3) & ~3;
    const int lo = slice * per;
    const int hi = lo + per < k ? lo + per : k;
    const uint64_t mine = e < k ? sm.sel[e] : 0ull;
    uint32_t beat = 0;
    if (low_const && n <= 65536) {
      // key bits 31..16 and a 16-bit index say it all: 32-bit words
      if (t < kSelRankSortMax + 4)
        sm.w32[t] = t < k ? ((uint32_t)(sm.sel[t] >> 32) & 0xffff0000u) | ((uint32_t)sm.sel[t] & 0xffffu)
                          : 0u;
      __syncthreads();
      const uint32_t mine32 = ((uint32_t)(mine >> 32) & 0xffff0000u) | ((uint32_t)mine & 0xffffu);
      for (int j = lo; j < hi; j += 4) {
        const uint4 v = *(const uint4 *)&sm.w32[j];  // padding words are 0: they beat nothing
        beat += (v.x > mine32) + (v.y > mine32) + (v.z > mine32) + (v.w > mine32);
      }
    } else {
      for (int j = lo; j < hi; ++j) beat += sm.sel[j] > mine ? 1u : 0u;
    }
    if (e < k && beat) atomicAdd(&sm.rank[e], beat);
    __syncthreads();
    if (slice == 0 && e < k) sm.idx_out[sm.rank[e]] = 0xffffffffu - (uint32_t)mine;
    __syncthreads();
    return sm.idx_out;
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
  for (int j = t; j < k; j += kSelThreads) sm.idx_out[j] = 0xffffffffu - (uint32_t)sm.sel[j];
  __syncthreads();
  return sm.idx_out;
}

template <typename KeyFn>
__device__ __forceinline__ const uint32_t *select_sorted(const KeyFn &key_of, int n, int k,
                                                         SelectShared &sm) {
  if (n <= 4 * kSelThreads) return select_sorted_impl<4>(key_of, n, k, sm);
  if (n <= 8 * kSelThreads) return select_sorted_impl<8>(key_of, n, k, sm);
  return select_sorted_impl<16>(key_of, n, k, sm);
}

}  // namespace da
