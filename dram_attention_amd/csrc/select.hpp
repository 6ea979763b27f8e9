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
//      Histograms are replicated 16x so that clustered keys (rounded scores
//      share their top digits) do not serialise the LDS atomics; a digit in which
//      no two keys differ needs no pass (scores rounded to bf16 differ in their
//      high half only, time stamps of a decoding run in two digits at most);
//   3. one block-wide scan of per-thread counts places every key > T and the
//      lowest-index keys == T into LDS as 64-bit (key, ~index) words;
//   4. the k survivors are ordered by rank counting (k <= 256: thread (e, slice)
//      counts the words of its slice that beat word e; 32-bit words when key and
//      index fit) or, for larger k, by a stable LSD radix sort on the key alone
//      (the compaction leaves equal keys in index order already): 8-bit digits,
//      ranks inside a wave from eight ballots per word, digits that no two keys
//      differ in skipped.
// k == n (a complete ordering) skips phases 2 and 3.
// Rows longer than 16384 keys are processed in segments of 16384 and re-read
// from memory in every pass.
#pragma once

#include "common.hpp"

namespace da {

constexpr int kSelThreads = 1024;
constexpr int kSelWaves = kSelThreads / 64;
constexpr int kHistCopies = 16;
constexpr int kSelMaxK = 8192;     // survivors held in LDS: 8 bytes each
constexpr int kSelRegKeys = 16;    // keys cached per thread
constexpr int kSelRankSortMax = 256;  // longest list ordered by rank counting (measured: the
                                      // radix sort is 1.8 us slower at 256, 2.3 us faster at 512)

struct alignas(16) SelectShared {
  // the histogram phase and the survivor array never overlap in time
  union {
    uint32_t hist[256 * kHistCopies];  // 16 KiB
    uint64_t sel[kSelMaxK];            // 64 KiB
  };
  uint32_t idx_out[kSelMaxK];          // the result: winning indices, best first
  alignas(16) uint32_t w32[kSelRankSortMax + 4];   // compact sort words
  uint32_t rank[kSelRankSortMax];
  uint32_t total[256];
  uint32_t wave_pack[kSelWaves];  // per wave: (keys > T) << 16 | (keys == T)
  uint32_t wave_or[kSelWaves], wave_nor[kSelWaves];  // per wave: OR over the (normalised) keys / their complements
  uint32_t digit;        // digit chosen by the current pass
  uint32_t remaining;    // how many keys are still wanted from the chosen bin
  uint32_t sort_or, sort_and;  // OR / AND over the keys of the survivors (radix sort)
  uint32_t wave_tot[4];
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

// OR over the 64 lanes of a wave, valid in lane 63 (the same DPP steps as the scan).
__device__ __forceinline__ uint32_t wave_or_to_last_lane(uint32_t v) {
  v |= dpp_u32<0x111, 0xf>(v);
  v |= dpp_u32<0x112, 0xf>(v);
  v |= dpp_u32<0x114, 0xf>(v);
  v |= dpp_u32<0x118, 0xf>(v);
  v |= dpp_u32<0x142, 0xa>(v);
  v |= dpp_u32<0x143, 0xc>(v);
  return v;
}

// Exclusive prefix of this wave over the per-wave counts cnt[0..kSelWaves) in LDS,
// and their total: lanes 0..15 take one count each, one more scan, and every wave
// reads its own entry of the result (instead of a loop over the waves).  All 64
// lanes of the calling wave must be active.
__device__ __forceinline__ uint32_t waves_prefix(const uint32_t *cnt, uint32_t &total) {
  const int lane = threadIdx.x & 63;
  const uint32_t mine = lane < kSelWaves ? cnt[lane] : 0u;
  const uint32_t upto = wave_scan_inclusive(mine);
  const int my_wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  total = (uint32_t)__builtin_amdgcn_readlane((int)upto, kSelWaves - 1);
  return (uint32_t)__builtin_amdgcn_readlane((int)(upto - mine), my_wave);
}

// Stable LSD radix sort of the words sel[0..k) by their key half (bits 63..32),
// descending, in place; words of equal key keep their order.  The index space
// is striped over the block: wave w, round u, lane l holds position
// w*64*E + u*64 + l (E = rounds = ceil(k / 1024) <= 8), so going through a wave's
// rounds in turn visits its positions in ascending order.  Per pass and word:
// eight ballots give the lanes that hold the same digit (its peers); the word's
// rank is (what earlier rounds of this wave counted for the digit) + (peers in
// lower lanes), kept in a counter row that only this wave touches, so no atomics
// and no barrier inside the ranking.  A 256-thread scan over (digit, wave) turns
// the counters into offsets, and the words, held in registers meanwhile, go back
// to sel at their new places.  Uses idx_out as scratch: (16 waves x 256 digits)
// counters and 256 digit bases.
__device__ __forceinline__ void radix_sort_survivors(SelectShared &sm, int k) {
  constexpr int kMaxRounds = kSelMaxK / kSelThreads;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int rounds = (k + kSelThreads - 1) / kSelThreads;
  const int first = wave * 64 * rounds + lane;
  uint32_t *cnt = sm.idx_out;                 // [kSelWaves][256]
  uint32_t *base = cnt + kSelWaves * 256;     // [256]
  uint32_t *row = cnt + wave * 256;

  uint64_t word[kMaxRounds] = {};
  uint32_t k_or = 0, k_and = 0xffffffffu;
#pragma unroll
  for (int u = 0; u < kMaxRounds; ++u) {
    const int p = first + u * 64;
    if (u < rounds && p < k) {
      const uint32_t key = (uint32_t)(sm.sel[p] >> 32);
      k_or |= key;
      k_and &= key;
    }
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) {
    k_or |= __shfl_xor(k_or, d, 64);
    k_and &= __shfl_xor(k_and, d, 64);
  }
  if (lane == 0) {
    atomicOr(&sm.sort_or, k_or);
    atomicAnd(&sm.sort_and, k_and);
  }
  __syncthreads();
  const uint32_t differ = sm.sort_or ^ sm.sort_and;  // bits in which two keys differ

  for (int shift = 0; shift < 32; shift += 8) {
    if (((differ >> shift) & 255u) == 0) continue;  // same for every thread
    for (int i = t; i < kSelWaves * 256; i += kSelThreads) cnt[i] = 0;
#pragma unroll
    for (int u = 0; u < kMaxRounds; ++u) {
      const int p = first + u * 64;
      if (u < rounds && p < k) word[u] = sm.sel[p];
    }
    __syncthreads();
    uint32_t place[kMaxRounds];
#pragma unroll
    for (int u = 0; u < kMaxRounds; ++u) {
      if (u < rounds) {  // whole waves take this branch together
        const bool valid = first + u * 64 < k;
        const uint32_t digit = 255u - ((uint32_t)(word[u] >> (32 + shift)) & 255u);
        uint64_t peers = __ballot(valid);
#pragma unroll
        for (int b = 0; b < 8; ++b) {
          const bool bit = (digit >> b) & 1u;
          const uint64_t with = __ballot(bit);
          peers &= bit ? with : ~with;
        }
        const uint32_t below = __builtin_amdgcn_mbcnt_hi(
            (uint32_t)(peers >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)peers, 0u));
        if (valid) {
          // every peer reads the counter before the lowest of them raises it: one
          // wave, one instruction after the other
          const uint32_t seen = row[digit];
          place[u] = seen + below;
          if (below == 0) row[digit] = seen + (uint32_t)__popcll(peers);
        }
        // the next round's reads of the row come after this round's store (no
        // instruction: it only forbids the compiler to move LDS accesses across)
        __builtin_amdgcn_wave_barrier();
      }
    }
    __syncthreads();
    if (t < 256) {  // digit t: counters of the waves -> offsets inside the digit
      uint32_t run = 0;
#pragma unroll
      for (int w = 0; w < kSelWaves; ++w) {
        const uint32_t c = cnt[w * 256 + t];
        cnt[w * 256 + t] = run;
        run += c;
      }
      const uint32_t incl = wave_scan_inclusive(run);
      base[t] = incl - run;
      if (lane == 63) sm.wave_tot[wave] = incl;
    }
    __syncthreads();
    const uint32_t t0 = sm.wave_tot[0], t1 = t0 + sm.wave_tot[1], t2 = t1 + sm.wave_tot[2];
#pragma unroll
    for (int u = 0; u < kMaxRounds; ++u) {
      if (u < rounds && first + u * 64 < k) {
        const uint32_t digit = 255u - ((uint32_t)(word[u] >> (32 + shift)) & 255u);
        const uint32_t ahead = digit < 64 ? 0u : digit < 128 ? t0 : digit < 192 ? t1 : t2;
        sm.sel[ahead + base[digit] + row[digit] + place[u]] = word[u];
      }
    }
    __syncthreads();
  }
}

// Where the result goes.  IntoLds: the winners' indices are left in sm.idx_out (best
// first) behind a barrier, and select_sorted returns that array.  Direct<F>: every
// winner is handed to f(rank, index) by one thread as soon as its rank is known,
// without the trip through idx_out and its barrier (the return value is unused).
struct IntoLds {
  static constexpr bool kDirect = false;
  __device__ __forceinline__ void operator()(uint32_t, uint32_t) const {}
};
template <typename F>
struct Direct {
  F f;
  static constexpr bool kDirect = true;
  __device__ __forceinline__ void operator()(uint32_t rank, uint32_t index) const { f(rank, index); }
};
template <typename F>
__device__ __forceinline__ Direct<F> direct(F f) { return Direct<F>{f}; }

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
template <int C, typename KeyFn, typename Emit>
__device__ const uint32_t *select_sorted_impl(const KeyFn &key_of, int n, int k,
                                              SelectShared &sm, const Emit &emit) {
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

  const bool take_all = k == n;  // a complete ordering: nothing to select
  // Which bits do two keys differ in?  OR over the keys and OR over their complements;
  // a bit set in both is a 1 in one key and a 0 in another.  The low half is
  // complemented first where the key's top bit is clear: the order-preserving image
  // of a float rounded to 16 bits ends in 0x0000 when its top bit is set and in
  // 0xffff when it is clear (and the complemented image likewise), so that such keys
  // differ in their high half only, whatever their signs.
  uint32_t acc_or = 0, acc_nor = 0;
  for (int s = n_seg - 1; s >= 0; --s) {  // ends with segment 0 in registers
    load_segment(s);
    const int real = n - (s * seg_n + t * C);
#pragma unroll
    for (int u = 0; u < C; ++u) {
      if (u < real) {  // padding must not count
        const uint32_t norm = kreg[u] ^ (~(uint32_t)((int32_t)kreg[u] >> 31) & 0xffffu);
        acc_or |= norm;
        acc_nor |= ~norm;
      }
    }
  }
  acc_or = wave_or_to_last_lane(acc_or);
  acc_nor = wave_or_to_last_lane(acc_nor);
  if (lane == 63) {
    sm.wave_or[wave] = acc_or;
    sm.wave_nor[wave] = acc_nor;
  }
  for (int i = t; i < 256 * kHistCopies; i += kSelThreads) sm.hist[i] = 0;
  if (t < kSelRankSortMax) sm.rank[t] = 0;
  if (t == 0) {
    sm.remaining = (uint32_t)k;
    sm.sort_or = 0;
    sm.sort_and = 0xffffffffu;
  }
  __syncthreads();
  // every wave folds the 16 partial results for itself: no atomics, no second barrier
  const uint32_t key_or = (uint32_t)__builtin_amdgcn_readlane(
      (int)wave_or_to_last_lane(lane < kSelWaves ? sm.wave_or[lane] : 0u), 63);
  const uint32_t key_nor = (uint32_t)__builtin_amdgcn_readlane(
      (int)wave_or_to_last_lane(lane < kSelWaves ? sm.wave_nor[lane] : 0u), 63);
  const uint32_t differ = key_or & key_nor;

  // When the bits in which keys differ span at most 12 positions (scores rounded to
  // bf16 within 16 binades, time stamps of a run), ONE pass over that window finds
  // the threshold: 1024 bins x 4 copies, 2048 x 2 or 4096 x 1 in the same 16 KiB, the
  // window's raw bits as the digit (outside the window all keys agree, up to the
  // complement of the low half that follows the top bit).
  const int d_lsb = differ ? __builtin_ctz(differ) : 0;
  const int d_width = differ ? 32 - __builtin_clz(differ) - d_lsb : 0;
  const bool one_pass = !take_all && differ != 0 && d_width <= 12;
  uint32_t thresh;  // k-th largest key
  if (one_pass) {
    const int wbits = d_width <= 10 ? 10 : d_width;
    const int wshift = d_lsb + wbits <= 32 ? d_lsb : 32 - wbits;
    const uint32_t wmask = (1u << wbits) - 1u;
    const int copy_bits = 12 - wbits;  // 4 copies, 2, or 1
    for (int s = 0; s < n_seg; ++s) {
      if (n_seg > 1) load_segment(s);
#pragma unroll
      for (int u = 0; u < C; ++u)
        atomicAdd(&sm.hist[(((kreg[u] >> wshift) & wmask) << copy_bits) + (lane & ((1 << copy_bits) - 1))], 1u);
    }
    __syncthreads();
    // thread t takes the t-th group of four words from the top: one bin (four
    // copies), two bins (two copies each) or four bins, in descending order
    const int group = kSelThreads - 1 - t;
    const uint4 w = *(const uint4 *)&sm.hist[4 * group];
    uint32_t c[4];  // counts of the group's bins, highest bin first; unused ones 0
    if (wbits == 10) {
      c[0] = w.x + w.y + w.z + w.w;
      c[1] = c[2] = c[3] = 0;
    } else if (wbits == 11) {
      c[0] = w.z + w.w;
      c[1] = w.x + w.y;
      c[2] = c[3] = 0;
    } else {
      c[0] = w.w;
      c[1] = w.z;
      c[2] = w.y;
      c[3] = w.x;
    }
    const uint32_t mine = c[0] + c[1] + c[2] + c[3];
    const uint32_t incl = wave_scan_inclusive(mine);
    if (lane == 63) sm.wave_pack[wave] = incl;
    __syncthreads();
    uint32_t all;
    const uint32_t excl = waves_prefix(sm.wave_pack, all) + incl - mine;
    const uint32_t want = (uint32_t)k;
    if (excl < want && want <= excl + mine) {  // true in exactly one thread
      uint32_t above = excl;
      int j = 0;  // which bin of the group, from the top
#pragma unroll
      for (int x = 0; x < 3; ++x) {
        if (j == x && above + c[x] < want) {
          above += c[x];
          j = x + 1;
        }
      }
      sm.digit = (uint32_t)(((group + 1) << (wbits - 10)) - 1 - j);
      sm.remaining = want - above;  // still needed from inside that bin
    }
    __syncthreads();
    thresh = (key_or & ~(wmask << wshift)) | (sm.digit << wshift);
    // low-half bits outside the window: undo the complement where the top bit is clear
    if (!(thresh >> 31)) thresh ^= 0xffffu & ~(wmask << wshift);
  } else {
  uint32_t prefix = 0;  // the digits of T fixed so far (high bits)
  const int passes = take_all ? 0 : 4;
  bool counted = false;  // has a histogram pass run yet
  for (int pass = 0; pass < passes; ++pass) {
    const int shift = 24 - 8 * pass;
    if (((differ >> shift) & 255u) == 0) {
      // every key has the same digit here: it is the threshold's too (in the low
      // half, undo the complement applied to keys whose top bit is clear)
      uint32_t digit = (key_or >> shift) & 255u;
      if (shift < 16 && !((prefix >> (23 - shift)) & 1u)) digit ^= 255u;
      prefix = (prefix << 8) | digit;
      continue;
    }
    for (int s = 0; s < n_seg; ++s) {
      if (n_seg > 1) load_segment(s);
#pragma unroll
      for (int u = 0; u < C; ++u) {
        const uint32_t key = kreg[u];
        if (!counted || (key >> (shift + 8)) == prefix)
          atomicAdd(&sm.hist[((key >> shift) & 255u) * kHistCopies + (lane & (kHistCopies - 1))], 1u);
      }
    }
    counted = true;
    __syncthreads();
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
  thresh = prefix;
  }
  // Do the bits in which keys differ fit a window of 16?  (Rounded scores: the high
  // half; time stamps of a run: a few low or middle bits.)  Then those bits order
  // the keys: two keys that differ in their top bit put the window into the high
  // half, where the complement of the low half plays no part.
  const int key_lsb = differ ? __builtin_ctz(differ) : 16;
  const bool narrow = (differ >> key_lsb) < 65536u && n <= 65536;
  const uint32_t n_eq = sm.remaining;  // keys == T to keep (k itself when nothing was selected)
  const uint32_t n_gt_total = (uint32_t)k - n_eq;
  // (the last barrier of the loop also retired every read of hist: sel may be written)

  // Compaction in index order = thread order.  Keys > T fill the first
  // n_gt_total places, keys == T follow while their rank is below n_eq.
  uint32_t gt_base = 0, eq_base = 0;
  if (take_all) {  // every key stays, at its own index (n = k <= kSelMaxK: one segment)
    const int i0 = t * C;
#pragma unroll
    for (int u = 0; u < C; ++u)
      if (i0 + u < n)
        sm.sel[i0 + u] = ((uint64_t)kreg[u] << 32) | (uint64_t)(0xffffffffu - (uint32_t)(i0 + u));
    __syncthreads();
  }
  for (int s = 0; s < (take_all ? 0 : n_seg); ++s) {
    if (n_seg > 1) load_segment(s);
    uint32_t gt_c = 0, eq_c = 0;
#pragma unroll
    for (int u = 0; u < C; ++u) {
      gt_c += kreg[u] > thresh ? 1u : 0u;
      eq_c += kreg[u] == thresh ? 1u : 0u;
    }
    // both counts in one word (a segment has at most 16384 keys: 15 bits each)
    const uint32_t incl = wave_scan_inclusive((gt_c << 16) | eq_c);
    if (lane == 63) sm.wave_pack[wave] = incl;
    __syncthreads();
    uint32_t all;
    const uint32_t before = waves_prefix(sm.wave_pack, all);
    uint32_t gt_off = gt_base + (before >> 16) + (incl >> 16) - gt_c;
    uint32_t eq_off = eq_base + (before & 0xffffu) + (incl & 0xffffu) - eq_c;
    gt_base += all >> 16;
    eq_base += all & 0xffffu;
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
    if (narrow) {
      // the 16 key bits that can differ and a 16-bit index say it all: 32-bit words
      if (t < kSelRankSortMax + 4)
        sm.w32[t] = t < k ? (((uint32_t)(sm.sel[t] >> 32) >> key_lsb) << 16) | ((uint32_t)sm.sel[t] & 0xffffu)
                          : 0u;
      __syncthreads();
      const uint32_t mine32 = (((uint32_t)(mine >> 32) >> key_lsb) << 16) | ((uint32_t)mine & 0xffffu);
#pragma unroll 16
      for (int j = lo; j < hi; j += 4) {
        const uint4 v = *(const uint4 *)&sm.w32[j];  // padding words are 0: they beat nothing
        beat += (v.x > mine32) + (v.y > mine32) + (v.z > mine32) + (v.w > mine32);
      }
    } else {
      for (int j = lo; j < hi; ++j) beat += sm.sel[j] > mine ? 1u : 0u;
    }
    if (e < k && beat) atomicAdd(&sm.rank[e], beat);
    __syncthreads();
    if (slice == 0 && e < k) {
      if constexpr (Emit::kDirect)
        emit(sm.rank[e], 0xffffffffu - (uint32_t)mine);
      else
        sm.idx_out[sm.rank[e]] = 0xffffffffu - (uint32_t)mine;
    }
    if constexpr (!Emit::kDirect) __syncthreads();
    return sm.idx_out;
  }

  radix_sort_survivors(sm, k);
  for (int j = t; j < k; j += kSelThreads) {
    if constexpr (Emit::kDirect)
      emit((uint32_t)j, 0xffffffffu - (uint32_t)sm.sel[j]);
    else
      sm.idx_out[j] = 0xffffffffu - (uint32_t)sm.sel[j];
  }
  if constexpr (!Emit::kDirect) __syncthreads();
  return sm.idx_out;
}

template <typename KeyFn, typename Emit = IntoLds>
__device__ __forceinline__ const uint32_t *select_sorted(const KeyFn &key_of, int n, int k,
                                                         SelectShared &sm, const Emit &emit = Emit()) {
  if (n <= 4 * kSelThreads) return select_sorted_impl<4>(key_of, n, k, sm, emit);
  if (n <= 8 * kSelThreads) return select_sorted_impl<8>(key_of, n, k, sm, emit);
  return select_sorted_impl<16>(key_of, n, k, sm, emit);
}

}  // namespace da
