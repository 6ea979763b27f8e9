// Split-K decode attention for one query token over
//   [prefix segment] ++ [local cache rows 0..c_len) ++ [the new token],
// with the in-place append of the new key/value and a log-sum-exp merge of all
// partial results.  Counterpart of the two flash_attn_with_kvcache calls and
// _combine_attention in dram_attention/dram_attention.py:191-238 of the
// reference.
//
// Bound: HBM.  Algorithmic bytes = (p_len + c_len + 1) * Hkv * 2 * D * e.
//
// Work split: grid = (token chunks, kv heads, query-row groups).  A 256-thread
// block streams one chunk of one kv head for up to kRows query heads of that
// head's GQA group, so keys/values are read once per group.  kLanes = D*e/16
// adjacent lanes cover a key (or value) row with 16-byte loads; a wave handles
// 64/kLanes tokens per step and every lane group keeps its own online-softmax
// state (running max, sum, and its 16-byte slice of the output row) in
// registers.  States are merged by shuffles inside the wave, through LDS
// across the four waves, and written as one fp32 partial per (chunk, q head);
// a second kernel merges the partials of all chunks.
//
// Paged prefix with overlap: when the prefix is the slot array of an LRU page
// cache whose missed pages are still being streamed in on another stream, the
// work is issued in two phases.  Phase 1 covers the local segment and every
// slot that was NOT re-assigned in this step (slot_epoch != current epoch);
// phase 2, issued once the page stream has finished, covers the re-assigned
// slots through the miss list and then merges everything.  Both phases are the
// same kernel; a chunk id says which segment a block works on.
#include "common.hpp"
#ifdef DA_TUNE
#include <stdlib.h>
#endif

namespace da {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kMinusHuge = -1.0e30f;  // finite stand-in for -inf as a running max
// The softmax reference m of a lane group is not kept equal to the running
// maximum: it is only raised when a score exceeds it by more than this many
// powers of two.  Softmax is shift invariant, so the result is the same; the
// weights stay below 2^slack, and the register-wide rescale becomes rare.
constexpr float kRescaleSlack = 8.0f;
constexpr int kAttnThreads = 256;
constexpr int kAttnWaves = kAttnThreads / 64;
#ifndef DA_ATTN_UNROLL
#define DA_ATTN_UNROLL 4
#endif
constexpr int kAttnUnroll = DA_ATTN_UNROLL;  // tokens in flight per lane group (even)

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// 16 bytes of q against 16 bytes of k, fp32 accumulate.
template <typename T>
__device__ __forceinline__ float dot16(const u32x4 &q, const u32x4 &k);
template <>
__device__ __forceinline__ float dot16<F32>(const u32x4 &q, const u32x4 &k) {
  float a = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) a = fmaf(as_f32(q[i]), as_f32(k[i]), a);
  return a;
}
template <>
__device__ __forceinline__ float dot16<BF16>(const u32x4 &q, const u32x4 &k) {
  float a = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
    a = __builtin_amdgcn_fdot2_f32_bf16(as_bf16x2(q[i]), as_bf16x2(k[i]), a, false);
  return a;
}
template <>
__device__ __forceinline__ float dot16<F16>(const u32x4 &q, const u32x4 &k) {
  float a = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) a = __builtin_amdgcn_fdot2(as_f16x2(q[i]), as_f16x2(k[i]), a, false);
  return a;
}

// acc[r][:] += p0[r] * v0[:] + p1[r] * v1[:] for the lane's 16-byte value slices
// of two tokens.  16-bit types interleave the two slices so that one packed dot
// product per output channel takes both tokens; the probabilities are rounded
// to the value type for it (as flash-attn does before its P*V product).
template <typename T, int kRows>
struct PvPair;
template <int kRows>
struct PvPair<F32, kRows> {
  static __device__ __forceinline__ void run(const u32x4 &v0, const u32x4 &v1, const float *p0,
                                             const float *p1, float (*acc)[4]) {
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        acc[r][i] = fmaf(p1[r], as_f32(v1[i]), fmaf(p0[r], as_f32(v0[i]), acc[r][i]));
    }
  }
};
template <int kRows>
struct PvPair<BF16, kRows> {
  static __device__ __forceinline__ void run(const u32x4 &v0, const u32x4 &v1, const float *p0,
                                             const float *p1, float (*acc)[8]) {
    uint32_t lo[4], hi[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      lo[i] = __builtin_amdgcn_perm(v1[i], v0[i], 0x05040100u);  // (v0 ch 2i,   v1 ch 2i)
      hi[i] = __builtin_amdgcn_perm(v1[i], v0[i], 0x07060302u);  // (v0 ch 2i+1, v1 ch 2i+1)
    }
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      const bf16x2 pp = as_bf16x2(pack_bf16(p0[r], p1[r]));
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc[r][2 * i] = __builtin_amdgcn_fdot2_f32_bf16(as_bf16x2(lo[i]), pp, acc[r][2 * i], false);
        acc[r][2 * i + 1] =
            __builtin_amdgcn_fdot2_f32_bf16(as_bf16x2(hi[i]), pp, acc[r][2 * i + 1], false);
      }
    }
  }
};
template <int kRows>
struct PvPair<F16, kRows> {
  static __device__ __forceinline__ void run(const u32x4 &v0, const u32x4 &v1, const float *p0,
                                             const float *p1, float (*acc)[8]) {
    uint32_t lo[4], hi[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      lo[i] = __builtin_amdgcn_perm(v1[i], v0[i], 0x05040100u);
      hi[i] = __builtin_amdgcn_perm(v1[i], v0[i], 0x07060302u);
    }
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      const f16x2 pp = as_f16x2(pack_f16(p0[r], p1[r]));
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc[r][2 * i] = __builtin_amdgcn_fdot2(as_f16x2(lo[i]), pp, acc[r][2 * i], false);
        acc[r][2 * i + 1] = __builtin_amdgcn_fdot2(as_f16x2(hi[i]), pp, acc[r][2 * i + 1], false);
      }
    }
  }
};

struct AttnArgs {
  const char *q;
  int64_t q_head_stride;  // elements
  int rep;                // query heads per kv head
  const char *pk, *pv;    // prefix segment
  int64_t p_tok_stride, p_head_stride, p_len;
  char *ck, *cv;  // local cache
  int64_t c_tok_stride, c_head_stride, c_capacity, c_len;
  const int32_t *c_len_dev;
  const char *new_k, *new_v;
  int64_t new_head_stride;
  float scale_log2;  // softmax scale * log2(e)
  int chunk;         // tokens per block (prefix and local segments)
  int tail_chunk;    // tokens per block of the tail segment
  // chunk ids: [0, n_pchunks) prefix, [n_pchunks, +n_lchunks) local, then n_tchunks tail
  int n_pchunks, n_lchunks, n_tchunks;
  int chunk_base;  // chunk id of blockIdx.x == 0 in this launch
  int pre_chunk;   // chunk id that holds the merged result of the prefix and local chunks
  int gather_chunk0;   // first chunk id of the partials a gather-with-attention pass wrote
  int gather_blocks;   // its blocks per kv head (0: the tail kernel covers the re-assigned slots)
  int n_q_heads;
  float *part_ml;   // (chunks, Hq, 2): running max (log2 domain), sum
  float *part_acc;  // (chunks, Hq, D)
  // paged prefix with overlap (all null / 0 otherwise)
  int page_size;
  int page_shift;  // log2(page_size), or -1 if it is not a power of two
  const int32_t *slot_epoch;  // (Hkv, p_len / page_size): epoch of a slot's last re-assignment
  int64_t slot_epoch_head_stride;
  const int32_t *epoch;       // the current epoch (one int32)
  const int32_t *miss_slot;   // (Hkv, miss_capacity) slots re-assigned in this epoch
  const int32_t *miss_count;  // (Hkv)
  int miss_capacity;
};

struct LocalLen {
  int64_t c_len;  // rows already in the local cache (clamped to its capacity)
  bool has_new;   // the new token is appended and attended
};
__device__ __forceinline__ LocalLen local_len(const AttnArgs &a) {
  int64_t c_len = a.c_len;
  if (a.c_len_dev) c_len += *a.c_len_dev;  // host value = offset to the device counter
  if (c_len < 0) c_len = 0;
  const bool has_new = a.new_k != nullptr && c_len < a.c_capacity;
  if (c_len > a.c_capacity) c_len = a.c_capacity;
  return {c_len, has_new};
}

// kTail = false: chunks of the prefix and local segments; kTail = true: chunks
// of the tail segment (the slots listed in the miss list).
template <typename T, int kLanes, int kRows, bool kTail>
__device__ __forceinline__ void attention_split_block(const AttnArgs &a, const int block_x) {
  constexpr int V = T::kVec;
  constexpr int kGroups = 64 / kLanes;  // tokens per wave step
  constexpr int kStepTokens = kAttnWaves * kGroups;
  constexpr int D = kLanes * V;
  constexpr int kUnrollHere = kRows >= 8 ? 2 : kAttnUnroll;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int c = lane % kLanes;
  const int g = lane / kLanes;
  const int h = blockIdx.y;
  const int row_group = blockIdx.z;
  const int row0 = row_group * kRows;  // first query row of the GQA group handled here
  const int chunk_id = a.chunk_base + block_x;

  // Which segment, which token range.
  const int kind = kTail ? 2 : (chunk_id < a.n_pchunks ? 0 : 1);
  const LocalLen ll = local_len(a);
  const int64_t c_len = ll.c_len;
  int64_t seg_len, t_begin;
  if (kind == 0) {
    seg_len = a.p_len;
    t_begin = (int64_t)chunk_id * a.chunk;
  } else if (kind == 1) {
    seg_len = c_len + (ll.has_new ? 1 : 0);
    t_begin = (int64_t)(chunk_id - a.n_pchunks) * a.chunk;
  } else {
    seg_len = (int64_t)a.miss_count[h] * a.page_size;
    t_begin = (int64_t)(chunk_id - a.n_pchunks - a.n_lchunks) * a.tail_chunk;
  }
  if (t_begin >= seg_len) return;  // the merge kernel skips this chunk as well
  const int chunk = kind == 2 ? a.tail_chunk : a.chunk;
  const int64_t t_end = t_begin + chunk < seg_len ? t_begin + chunk : seg_len;

  const char *kbase, *vbase;
  int64_t tok_stride_b;
  if (kind == 1) {
    kbase = a.ck + h * a.c_head_stride * T::kBytes + c * 16;
    vbase = a.cv + h * a.c_head_stride * T::kBytes + c * 16;
    tok_stride_b = a.c_tok_stride * T::kBytes;
  } else {
    kbase = a.pk + h * a.p_head_stride * T::kBytes + c * 16;
    vbase = a.pv + h * a.p_head_stride * T::kBytes + c * 16;
    tok_stride_b = a.p_tok_stride * T::kBytes;
  }
  const char *newk = nullptr, *newv = nullptr;
  if (kind == 1 && ll.has_new) {
    newk = a.new_k + h * a.new_head_stride * T::kBytes + c * 16;
    newv = a.new_v + h * a.new_head_stride * T::kBytes + c * 16;
  }
  const bool skip_fresh = kind == 0 && a.slot_epoch != nullptr;
  const int32_t epoch_now = skip_fresh ? *a.epoch : 0;
  const int32_t *slot_epoch = skip_fresh ? a.slot_epoch + h * a.slot_epoch_head_stride : nullptr;
  const int32_t *miss_slot = kind == 2 ? a.miss_slot + (int64_t)h * a.miss_capacity : nullptr;
  // When a block step never straddles a page and the chunk has at most 64
  // pages, one load per wave fetches the chunk's epochs and a ballot turns them
  // into a bit mask: the token loop then needs no memory access for the test.
  const bool uniform_pages = skip_fresh && a.page_shift >= 0 &&
                             a.page_size % kStepTokens == 0 && a.chunk % a.page_size == 0 &&
                             (a.chunk >> a.page_shift) <= 64;
  uint64_t fresh_mask = 0;
  if (uniform_pages) {
    const int64_t first_page = t_begin >> a.page_shift;
    const int64_t n_pages_here = (t_end - t_begin + a.page_size - 1) >> a.page_shift;
    const bool fresh = lane < n_pages_here && slot_epoch[first_page + lane] == epoch_now;
    fresh_mask = __ballot(fresh);
  }

  u32x4 qv[kRows];
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const int rr = row0 + r < a.rep ? row0 + r : a.rep - 1;
    qv[r] = load16(a.q + ((int64_t)(h * a.rep + rr) * a.q_head_stride) * T::kBytes + c * 16);
  }

  float m[kRows], l[kRows], acc[kRows][V];
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    m[r] = kMinusHuge;
    l[r] = 0.f;
#pragma unroll
    for (int i = 0; i < V; ++i) acc[r][i] = 0.f;
  }

  const int64_t my_off = wave * kGroups + g;
  for (int64_t base = t_begin; base < t_end; base += (int64_t)kStepTokens * kUnrollHere) {
    // `base` is the same for the whole block, so the wave-wide vote below sees
    // every lane; lanes past the chunk end compute on a clamped row, masked.
    const int64_t t0 = base + my_off;
    u32x4 kk[kUnrollHere], vv[kUnrollHere];
    bool valid[kUnrollHere];
#pragma unroll
    for (int u = 0; u < kUnrollHere; ++u) {
      const int64_t tok = t0 + (int64_t)u * kStepTokens;
      valid[u] = tok < t_end;
      int64_t tk = valid[u] ? tok : t_begin;  // clamp the address, mask the score
      if (skip_fresh) {
        // A slot that is being rewritten right now is left to the tail pass; its
        // rows are still loaded (no dependent address) and discarded below.
        bool fresh;
        if (uniform_pages)
          fresh = (fresh_mask >> ((base - t_begin + (int64_t)u * kStepTokens) >> a.page_shift)) & 1;
        else
          fresh = slot_epoch[a.page_shift >= 0 ? tk >> a.page_shift : tk / a.page_size] == epoch_now;
        if (fresh) valid[u] = false;
      } else if (kTail) {
        const int64_t entry = a.page_shift >= 0 ? tk >> a.page_shift : tk / a.page_size;
        const int64_t within = tk - entry * a.page_size;
        const int32_t slot = miss_slot[entry];
        if (slot < 0) valid[u] = false;  // entry superseded later in the same step
        tk = (int64_t)(slot < 0 ? 0 : slot) * a.page_size + within;
      }
      const bool is_new = newk != nullptr && tk == c_len;
      const char *kp = is_new ? newk : kbase + tk * tok_stride_b;
      const char *vp = is_new ? newv : vbase + tk * tok_stride_b;
      kk[u] = load16(kp);
      vv[u] = load16(vp);
      if (is_new && valid[u] && row_group == 0) {
        // the append: this lane group owns the new token's row
        store16(a.ck + (h * a.c_head_stride + c_len * a.c_tok_stride) * T::kBytes + c * 16, kk[u]);
        store16(a.cv + (h * a.c_head_stride + c_len * a.c_tok_stride) * T::kBytes + c * 16, vv[u]);
      }
    }
#pragma unroll
    for (int u = 0; u < kUnrollHere; u += 2) {
      float s0[kRows], s1[kRows];
      bool grow = false;
#pragma unroll
      for (int r = 0; r < kRows; ++r) {
        s0[r] = group_sum<kLanes>(dot16<T>(qv[r], kk[u])) * a.scale_log2;
        s1[r] = group_sum<kLanes>(dot16<T>(qv[r], kk[u + 1])) * a.scale_log2;
        if (!valid[u]) s0[r] = -INFINITY;
        if (!valid[u + 1]) s1[r] = -INFINITY;
        grow |= fmaxf(s0[r], s1[r]) > m[r] + kRescaleSlack;
      }
      if (__any(grow)) {  // rare: the reference only moves when a score clears it by the slack
#pragma unroll
        for (int r = 0; r < kRows; ++r) {
          const float mn = fmaxf(m[r], fmaxf(s0[r], s1[r]));
          const float alpha = fast_exp2(m[r] - mn);
          m[r] = mn;
          l[r] *= alpha;
#pragma unroll
          for (int i = 0; i < V; ++i) acc[r][i] *= alpha;
        }
      }
      // a masked row may be memory another stream is writing (torn values, NaN):
      // its weight is 0, and its values are zeroed so that 0 * NaN cannot arise
      if (!valid[u]) vv[u] = u32x4{0, 0, 0, 0};
      if (!valid[u + 1]) vv[u + 1] = u32x4{0, 0, 0, 0};
      float p0[kRows], p1[kRows];
#pragma unroll
      for (int r = 0; r < kRows; ++r) {
        p0[r] = fast_exp2(s0[r] - m[r]);
        p1[r] = fast_exp2(s1[r] - m[r]);
        l[r] += p0[r] + p1[r];
      }
      PvPair<T, kRows>::run(vv[u], vv[u + 1], p0, p1, acc);
    }
  }

  // Merge the lane groups of the wave (butterfly over the group index).
#pragma unroll
  for (int off = kLanes; off < 64; off <<= 1) {
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      const float mo = __shfl_xor(m[r], off, 64);
      const float lo = __shfl_xor(l[r], off, 64);
      const float mn = fmaxf(m[r], mo);
      const float wa = fast_exp2(m[r] - mn), wb = fast_exp2(mo - mn);
      l[r] = l[r] * wa + lo * wb;
#pragma unroll
      for (int i = 0; i < V; ++i) {
        const float ao = __shfl_xor(acc[r][i], off, 64);
        acc[r][i] = acc[r][i] * wa + ao * wb;
      }
      m[r] = mn;
    }
  }

  // Merge the waves through LDS; wave w's state sits in sm_*[w].
  __shared__ float sm_m[kAttnWaves][kRows];
  __shared__ float sm_l[kAttnWaves][kRows];
  __shared__ float sm_acc[kAttnWaves][kRows][D];
  if (g == 0) {
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      if (c == 0) {
        sm_m[wave][r] = m[r];
        sm_l[wave][r] = l[r];
      }
#pragma unroll
      for (int i = 0; i < V; ++i) sm_acc[wave][r][c * V + i] = acc[r][i];
    }
  }
  __syncthreads();
  for (int item = threadIdx.x; item < kRows * D; item += kAttnThreads) {
    const int r = item / D, d = item % D;
    if (row0 + r >= a.rep) continue;
    float mn = sm_m[0][r];
#pragma unroll
    for (int w = 1; w < kAttnWaves; ++w) mn = fmaxf(mn, sm_m[w][r]);
    float lt = 0.f, at = 0.f;
#pragma unroll
    for (int w = 0; w < kAttnWaves; ++w) {
      const float wgt = fast_exp2(sm_m[w][r] - mn);
      lt += sm_l[w][r] * wgt;
      at += sm_acc[w][r][d] * wgt;
    }
    const int64_t hq = (int64_t)h * a.rep + row0 + r;
    const int64_t slot = (int64_t)chunk_id * a.n_q_heads + hq;
    a.part_acc[slot * D + d] = at;
    if (d == 0) {
      a.part_ml[slot * 2] = mn;
      a.part_ml[slot * 2 + 1] = lt;
    }
  }
}

template <typename T, int kLanes, int kRows, bool kTail>
__global__ void __launch_bounds__(kAttnThreads)
decode_attention_split_kernel(const AttnArgs a) {
  attention_split_block<T, kLanes, kRows, kTail>(a, blockIdx.x);
}

// ---------------------------------------------------------------------------
// Page stream with attention riding on it.  A block copies the pages of one kv
// head's miss list (entries block_x, += n_blocks) from the host page store
// into their slots, 16 bytes per lane, and the registers the page passes
// through also feed the attention of this step's query over that page: the
// re-assigned slots then need no second pass after the stream has finished.
// A page holds page_size tokens, each token its K row followed by its V row,
// so 2*kLanes adjacent lanes hold one token: the lower kLanes its key (they
// produce the score), the upper kLanes its value (they keep the softmax state
// and the weighted sum).  The next page's loads are issued before the current
// page is stored and attended, so the host link never waits for arithmetic.
// Every block with an entry to copy leaves one partial (all query rows of the
// kv head) at chunk id gather_chunk0 + block_x.
struct GatherAttendArgs {
  const char *dram;
  int64_t dram_head_stride, dram_page_stride;
  char *hbm;
  int64_t hbm_head_stride, hbm_slot_stride;
  int page_vecs;  // 16-byte lanes per page
  const int32_t *miss_page, *miss_slot, *miss_count;
  int K;
  const char *q;
  int64_t q_head_stride;
  int rep, n_q_heads, n_kv_heads;
  float scale_log2;
  float *part_ml, *part_acc;
  int chunk0;
};

constexpr int kGatherThreads = 256;
constexpr int kGatherMaxLoads = 4;  // 16-byte loads per lane and page: pages up to 16 KiB
constexpr int kGatherIdBatch = 1024;  // miss-list entries of a block staged in LDS at a time

// The page stream's blocks share the miss lists of all kv heads, taken as one
// list in head order, in equal contiguous ranges (heads miss unequally: the
// busiest head of a step has ~20 % more pages than the average, and a stream
// split per head would end with a few blocks and an idle host link).  With
// `total` entries and `n_blocks` blocks, n_eff = min(n_blocks, total) of them
// work, block b on entries [b*total/n_eff, (b+1)*total/n_eff).  A block that
// crosses a head boundary leaves one partial per head it touched.
struct StreamRange {
  int64_t begin, end;
};
__device__ __forceinline__ StreamRange stream_range(int b, int n_blocks, int64_t total) {
  const int64_t n_eff = total < n_blocks ? total : n_blocks;
  if (b >= n_eff) return {0, 0};
  return {b * total / n_eff, (b + 1) * total / n_eff};
}

template <typename T, int kLanes, int kRows>
__device__ __forceinline__ void gather_attend_block(const GatherAttendArgs &g, const int block_x,
                                                    const int n_blocks) {
  constexpr int V = T::kVec;
  constexpr int D = kLanes * V;
  constexpr int kTokLanes = 2 * kLanes;
  constexpr int kWaves = kGatherThreads / 64;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int within = tid % kTokLanes;
  const bool is_v = within >= kLanes;
  const int c = within % kLanes;
  // this block's range of the concatenated miss lists
  int64_t total = 0;
  for (int hh = 0; hh < g.n_kv_heads; ++hh) total += g.miss_count[hh];
  const StreamRange range = stream_range(block_x, n_blocks, total);
  if (range.begin >= range.end) return;  // the merge does not count this block either

  __shared__ int32_t sm_slot[kGatherIdBatch], sm_page[kGatherIdBatch];
  __shared__ float sm_m[kWaves][kRows];
  __shared__ float sm_l[kWaves][kRows];
  __shared__ float sm_acc[kWaves][kRows][D];
  int64_t head_off = 0;
  for (int h = 0; h < g.n_kv_heads; ++h) {
  const int n_miss = g.miss_count[h];
  const int64_t lo64 = (range.begin > head_off ? range.begin : head_off) - head_off;
  const int64_t hi64 = (range.end < head_off + n_miss ? range.end : head_off + n_miss) - head_off;
  head_off += n_miss;
  if (lo64 >= hi64) continue;  // uniform: nothing of this head in the range
  const int first = (int)lo64, n_mine = (int)(hi64 - lo64);

  u32x4 qv[kRows];
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const int rr = r < g.rep ? r : g.rep - 1;
    qv[r] = load16(g.q + ((int64_t)(h * g.rep + rr) * g.q_head_stride) * T::kBytes + c * 16);
  }
  float m[kRows], l[kRows], acc[kRows][V];
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    m[r] = kMinusHuge;
    l[r] = 0.f;
#pragma unroll
    for (int i = 0; i < V; ++i) acc[r][i] = 0.f;
  }

  const int32_t *mpage = g.miss_page + (int64_t)h * g.K;
  const int32_t *mslot = g.miss_slot + (int64_t)h * g.K;
  // This block's entries (slot, page), staged in LDS a batch at a time: a page's
  // loads then depend on no other global load, and the next page is always in
  // flight while the current one is stored and attended.
  // Issues the loads of this block's n-th staged entry; dst == nullptr marks a
  // superseded one.  Always kGatherMaxLoads loads per lane, lanes with nothing to
  // fetch reading the query instead: with a fixed count the wait for one page's
  // data can leave the next page's loads outstanding.
  auto fetch = [&](int n, int n_batch, u32x4 *buf, char *&dst) {
    const bool real = n < n_batch;  // past the batch: the same loads, all of them idle
    const int32_t v = real ? sm_slot[n] : -1;
    const int32_t p = real ? sm_page[n] : 0;
    const char *src = g.dram + h * g.dram_head_stride + p * g.dram_page_stride;
    dst = v < 0 ? nullptr : g.hbm + h * g.hbm_head_stride + v * g.hbm_slot_stride;
#pragma unroll
    for (int u = 0; u < kGatherMaxLoads; ++u) {
      const int j = u * kGatherThreads + tid;
      buf[u] = load16(v >= 0 && j < g.page_vecs ? src + (int64_t)j * 16 : g.q);
    }
  };
  auto settle = [&](const u32x4 *buf, char *dst) {
    if (dst == nullptr) return;
#pragma unroll
    for (int u = 0; u < kGatherMaxLoads; ++u) {
      const int j = u * kGatherThreads + tid;
      if (j < g.page_vecs) store16(dst + (int64_t)j * 16, buf[u]);
    }
#pragma unroll
    for (int u = 0; u < kGatherMaxLoads; ++u) {
      if (u * kGatherThreads >= g.page_vecs) continue;  // uniform
      const bool tok = u * kGatherThreads + tid < g.page_vecs;
      const u32x4 data = tok ? buf[u] : u32x4{0, 0, 0, 0};
      float vf[V];
      unpack<T>(data, vf);
#pragma unroll
      for (int r = 0; r < kRows; ++r) {
        const float sk = group_sum<kLanes>(dot16<T>(qv[r], data)) * g.scale_log2;
        const float so = __shfl_xor(sk, kLanes, 64);  // a value lane takes its key lane's
        float sc = is_v ? so : sk;
        if (!tok) sc = -INFINITY;
        const float mn = fmaxf(m[r], sc);
        const float alpha = fast_exp2(m[r] - mn);
        const float pw = fast_exp2(sc - mn);
        m[r] = mn;
        l[r] = l[r] * alpha + pw;
#pragma unroll
        for (int x = 0; x < V; ++x) acc[r][x] = acc[r][x] * alpha + pw * vf[x];
      }
    }
  };

  for (int batch0 = 0; batch0 < n_mine; batch0 += kGatherIdBatch) {
    const int n_batch = n_mine - batch0 < kGatherIdBatch ? n_mine - batch0 : kGatherIdBatch;
    __syncthreads();  // the previous batch is no longer read
    for (int n = tid; n < n_batch; n += kGatherThreads) {
      const int64_t i = (int64_t)first + batch0 + n;
      sm_slot[n] = mslot[i];
      sm_page[n] = mpage[i];
    }
    __syncthreads();
    // two page buffers in turn: one is stored and attended while the other fills
    u32x4 a_buf[kGatherMaxLoads], b_buf[kGatherMaxLoads];
    char *a_dst = nullptr, *b_dst = nullptr;
    fetch(0, n_batch, a_buf, a_dst);
    for (int n = 0; n < n_batch; n += 2) {
      fetch(n + 1, n_batch, b_buf, b_dst);
      settle(a_buf, a_dst);
      fetch(n + 2, n_batch, a_buf, a_dst);
      settle(b_buf, b_dst);
    }
  }

  // Merge the tokens of a wave (lanes of equal position within a token pair up).
#pragma unroll
  for (int off = kTokLanes; off < 64; off <<= 1) {
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      const float mo = __shfl_xor(m[r], off, 64);
      const float lo = __shfl_xor(l[r], off, 64);
      const float mn = fmaxf(m[r], mo);
      const float wa = fast_exp2(m[r] - mn), wb = fast_exp2(mo - mn);
      l[r] = l[r] * wa + lo * wb;
#pragma unroll
      for (int x = 0; x < V; ++x) {
        const float ao = __shfl_xor(acc[r][x], off, 64);
        acc[r][x] = acc[r][x] * wa + ao * wb;
      }
      m[r] = mn;
    }
  }
  // Merge the waves through LDS; the value lanes of a wave's first token hold its state.
  if (is_v && lane < kTokLanes) {
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      if (c == 0) {
        sm_m[wave][r] = m[r];
        sm_l[wave][r] = l[r];
      }
#pragma unroll
      for (int x = 0; x < V; ++x) sm_acc[wave][r][c * V + x] = acc[r][x];
    }
  }
  __syncthreads();
  const int chunk_id = g.chunk0 + block_x;
  for (int item = tid; item < kRows * D; item += kGatherThreads) {
    const int r = item / D, d = item % D;
    if (r >= g.rep) continue;
    float mn = sm_m[0][r];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) mn = fmaxf(mn, sm_m[w][r]);
    float lt = 0.f, at = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const float wgt = fast_exp2(sm_m[w][r] - mn);
      lt += sm_l[w][r] * wgt;
      at += sm_acc[w][r][d] * wgt;
    }
    const int64_t slot = (int64_t)chunk_id * g.n_q_heads + (int64_t)h * g.rep + r;
    g.part_acc[slot * D + d] = at;
    if (d == 0) {
      g.part_ml[slot * 2] = mn;
      g.part_ml[slot * 2 + 1] = lt;
    }
  }
  }  // heads in this block's range (the next head's first barrier retires these reads)
}

template <typename T, int kLanes, int kRows>
__global__ void __launch_bounds__(kGatherThreads)
pages_gather_attend_kernel(const GatherAttendArgs g) {
  gather_attend_block<T, kLanes, kRows>(g, blockIdx.y * gridDim.x + blockIdx.x,
                                        gridDim.x * gridDim.y);
}

// Both of the above in one launch: blocks [0, g_blocks) of every kv head run the
// page stream, the others the first attention pass (prefix minus the slots under
// rewrite, plus the local segment).  One kernel instead of two on two streams
// keeps the step a plain chain of launches: no fork and join around the long
// pole of the step, each of which costs about 5 us of dependency latency.
static_assert(kGatherThreads == kAttnThreads, "one block shape for both roles");
template <typename T, int kLanes, int kRowsAttn, int kRowsGather>
__global__ void __launch_bounds__(kAttnThreads)
decode_stream_attend_kernel(const AttnArgs a, const GatherAttendArgs g, const int g_blocks) {
  if ((int)blockIdx.x < g_blocks) {
    if (blockIdx.z == 0)
      gather_attend_block<T, kLanes, kRowsGather>(g, blockIdx.y * g_blocks + blockIdx.x,
                                                  g_blocks * gridDim.y);
  } else {
    attention_split_block<T, kLanes, kRowsAttn, false>(a, (int)blockIdx.x - g_blocks);
  }
}

// Merge the partials of one query head.  One 512-thread block per head.  The
// softmax statistics are tiny, so every wave reduces them for itself (no
// barrier); then a thread owns four adjacent output channels of every 16th
// (at D = 128) chunk, reads the partial rows as 16-byte lanes, and the chunk
// lanes are folded through LDS.
//   kMergeAll   : every live chunk -> out
//   kMergePre   : prefix and local chunks -> out, and their merged, unnormalised
//                 state -> chunk `pre_chunk` (runs next to the page stream)
//   kMergeFinal : chunk `pre_chunk` + the live tail chunks -> out
constexpr int kMergeThreads = 512;
constexpr int kMergeStats = 2048;  // (max, sum) pairs staged in LDS
enum MergeMode { kMergeAll = 0, kMergePre = 1, kMergeFinal = 2 };

template <typename T>
__global__ void __launch_bounds__(kMergeThreads)
decode_attention_merge_kernel(const AttnArgs a, int mode, int head_dim, char *__restrict__ out,
                              int64_t out_head_stride, float *__restrict__ lse_out) {
  const int hq = blockIdx.x;
  const int t = threadIdx.x;
  const int lane = t & 63;
  const LocalLen ll = local_len(a);
  const int64_t l_len = ll.c_len + (ll.has_new ? 1 : 0);
  const int n_p = a.n_pchunks;                              // live prefix chunks (all of them)
  const int n_l = (int)((l_len + a.chunk - 1) / a.chunk);   // live local chunks
  int n_t = 0;                                              // live tail chunks
  int tail_chunk0 = a.n_pchunks + a.n_lchunks;
  if (a.gather_blocks > 0 && mode != kMergePre) {
    // the blocks of the page stream whose range met this kv head's miss list
    const int n_kv = a.n_q_heads / a.rep, hk = hq / a.rep;
    const int n_blocks = a.gather_blocks * n_kv;
    int64_t total = 0, off = 0;
    for (int hh = 0; hh < n_kv; ++hh) {
      const int mc = a.miss_count[hh];
      if (hh < hk) off += mc;
      total += mc;
    }
    const int64_t mine = a.miss_count[hk];
    if (mine > 0) {
      // entry x lies in block ceil((x+1)*n_eff/total) - 1 (ranges are floor(b*total/n_eff))
      const int64_t n_eff = total < n_blocks ? total : n_blocks;
      int64_t b_first, b_last;
      if (total < (1 << 24)) {  // the usual case: 32-bit divisions (n_eff <= 64)
        const uint32_t t32 = (uint32_t)total, n32 = (uint32_t)n_eff;
        b_first = (((uint32_t)off + 1u) * n32 + t32 - 1u) / t32 - 1u;
        b_last = ((uint32_t)(off + mine) * n32 + t32 - 1u) / t32 - 1u;
      } else {
        b_first = ((off + 1) * n_eff + total - 1) / total - 1;
        b_last = ((off + mine) * n_eff + total - 1) / total - 1;
      }
      n_t = (int)(b_last - b_first + 1);
      tail_chunk0 = a.gather_chunk0 + (int)b_first;
    }
  } else if (a.n_tchunks > 0 && mode != kMergePre) {
    const int64_t tail = (int64_t)a.miss_count[hq / a.rep] * a.page_size;
    n_t = (int)((tail + a.tail_chunk - 1) / a.tail_chunk);
  }
  const int n_first = mode == kMergeFinal ? 1 : n_p + n_l;  // chunks ahead of the tail's
  const int n_live = n_first + n_t;
  // i-th live chunk -> chunk id
  auto chunk_of = [&](int i) {
    if (i < n_first) return mode == kMergeFinal ? a.pre_chunk : i;
    return tail_chunk0 + (i - n_first);
  };

  // Stage the (max, sum) pairs of the live chunks in LDS with one load per
  // thread, then let every wave reduce them for itself (no second barrier).
  __shared__ float2 sm_ml[kMergeStats];
  const bool staged = n_live <= kMergeStats;
  if (staged) {
    for (int i = t; i < n_live; i += kMergeThreads)
      sm_ml[i] = *(const float2 *)(a.part_ml + ((int64_t)chunk_of(i) * a.n_q_heads + hq) * 2);
    __syncthreads();
  }
  auto stat = [&](int i) -> float2 {
    return staged ? sm_ml[i]
                  : *(const float2 *)(a.part_ml + ((int64_t)chunk_of(i) * a.n_q_heads + hq) * 2);
  };
  float mx = kMinusHuge;
  for (int i = lane; i < n_live; i += 64) mx = fmaxf(mx, stat(i).x);
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) mx = fmaxf(mx, __shfl_xor(mx, d, 64));
  float lt = 0.f;
  for (int i = lane; i < n_live; i += 64) {
    const float2 ml = stat(i);
    lt += ml.y * fast_exp2(ml.x - mx);
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) lt += __shfl_xor(lt, d, 64);
  const float inv = lt > 0.f ? 1.f / lt : 0.f;

  __shared__ float sm_acc[kMergeThreads * 4];
  const int quads = head_dim / 4;              // 16-byte lanes per row (head_dim % 4 == 0 here)
  const int lanes_c = kMergeThreads / quads;   // chunk lanes
  const int qd = t % quads, cl = t / quads;
  float at[4] = {0.f, 0.f, 0.f, 0.f};
  if (cl < lanes_c) {
    // four independent partial rows in flight per thread
    for (int i0 = cl; i0 < n_live; i0 += 4 * lanes_c) {
      float4 v[4];
      float w[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int i = i0 + u * lanes_c;
        const int ic = i < n_live ? i : cl;  // clamp the address, zero the weight
        const int64_t slot = (int64_t)chunk_of(ic) * a.n_q_heads + hq;
        v[u] = *(const float4 *)(a.part_acc + slot * head_dim + qd * 4);
        w[u] = i < n_live ? fast_exp2(stat(ic).x - mx) : 0.f;
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        at[0] = fmaf(v[u].x, w[u], at[0]);
        at[1] = fmaf(v[u].y, w[u], at[1]);
        at[2] = fmaf(v[u].z, w[u], at[2]);
        at[3] = fmaf(v[u].w, w[u], at[3]);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) sm_acc[t * 4 + i] = at[i];
  __syncthreads();
  const int64_t pre_slot = (int64_t)a.pre_chunk * a.n_q_heads + hq;
  for (int d = t; d < head_dim; d += kMergeThreads) {
    float s = 0.f;
    for (int c2 = 0; c2 < lanes_c; ++c2) s += sm_acc[(c2 * quads + d / 4) * 4 + (d & 3)];
    store_elem<T>(out, (int64_t)hq * out_head_stride + d, s * inv);
    if (mode == kMergePre) a.part_acc[pre_slot * head_dim + d] = s;
  }
  if (mode == kMergePre && t == 0) {
    a.part_ml[pre_slot * 2] = mx;
    a.part_ml[pre_slot * 2 + 1] = lt;
  }
  if (lse_out && t == 0)
    lse_out[hq] = lt > 0.f ? (mx + __builtin_amdgcn_logf(lt)) * kLn2 : -INFINITY;
}

static int pick_chunk(int64_t total_tokens, int n_kv_heads, int step_tokens) {
  // ~2 blocks per CU on a 256-CU part: every block pays a fixed prologue and a
  // merge epilogue, so few long chunks beat many short ones (measured on the
  // 128K workload: 31.9 us at 512 blocks, 32.6 us at 2048); never below one
  // unrolled round.
  int64_t want_blocks = 256 * 2;
#ifdef DA_TUNE
  if (const char *e = getenv("DA_ATTN_BLOCKS")) want_blocks = atoi(e);
#endif
  int64_t chunk = total_tokens * n_kv_heads / want_blocks;
  const int round = step_tokens * kAttnUnroll;
  if (chunk < round) chunk = round;
  if (chunk > 4096) chunk = 4096;
  return (int)(ceil_div(chunk, round) * round);
}

static int lanes_of(int head_dim, int dtype) {
  const int vec = dtype == DA_F32 ? 4 : 8;
  if (head_dim % vec) return 0;
  const int lanes = head_dim / vec;
  return (lanes >= 4 && lanes <= 64 && is_pow2(lanes)) ? lanes : 0;
}

constexpr int kGatherMaxBlocks = 64;  // blocks of a page stream, all kv heads together

struct ChunkPlan {
  int chunk, tail_chunk, n_p, n_l, n_t;
  // slots beyond the chunks: the merged state of the first pass, then (with a
  // tail) one per block and kv head of a gather-with-attention pass
  int64_t total() const { return (int64_t)n_p + n_l + n_t + 1 + (n_t > 0 ? kGatherMaxBlocks : 0); }
  int pre_chunk() const { return n_p + n_l + n_t; }
  int gather_chunk0() const { return n_p + n_l + n_t + 1; }
};
// The chunk geometry of a launch; a function of the shapes only, so that the
// workspace query and every phase of a step agree on it.
static ChunkPlan plan_chunks(int n_kv_heads, int lanes, int64_t p_len, int64_t c_capacity,
                             int64_t miss_tokens) {
  const int step_tokens = kAttnWaves * (64 / lanes);
  ChunkPlan p;
  p.chunk = pick_chunk(p_len + c_capacity, n_kv_heads, step_tokens);
  p.n_p = (int)ceil_div(p_len, p.chunk);
  p.n_l = (int)ceil_div(c_capacity, p.chunk);
  // the tail is short and every block starts with a dependent slot lookup:
  // one unrolled round per block keeps it wide instead of deep
  p.tail_chunk = step_tokens * kAttnUnroll;
  p.n_t = (int)ceil_div(miss_tokens, p.tail_chunk);
  return p;
}

static size_t attn_workspace_bytes(int n_q_heads, int head_dim, int64_t n_chunks) {
  return (size_t)n_chunks * n_q_heads * (head_dim + 2) * sizeof(float);
}

template <typename T, int kLanes, bool kTail>
static void launch_split(AttnArgs a, int first_chunk, int n_launch, int n_kv_heads,
                         hipStream_t s) {
  if (n_launch <= 0) return;
  a.chunk_base = first_chunk;
  const int rep = a.rep;
  // Up to 4 query rows per block; 8 (with a shorter unroll, ~240 vector registers,
  // two waves per SIMD) when the GQA group is that wide and rows are <= 256 bytes:
  // one read of K/V for 8 heads beats two reads for 4 + 4 (1M workload: 115 vs 137 us).
  const int rows = rep <= 1 ? 1 : (rep == 2 ? 2 : ((rep > 4 && kLanes <= 16) ? 8 : 4));
  const dim3 grid(n_launch, n_kv_heads, (unsigned)ceil_div(rep, rows));
  if (rows == 8) {
    hipLaunchKernelGGL((decode_attention_split_kernel<T, (kLanes <= 16 ? kLanes : 16), 8, kTail>), grid,
                       dim3(kAttnThreads), 0, s, a);
    return;
  }
  if (rows == 1)
    hipLaunchKernelGGL((decode_attention_split_kernel<T, kLanes, 1, kTail>), grid,
                       dim3(kAttnThreads), 0, s, a);
  else if (rows == 2)
    hipLaunchKernelGGL((decode_attention_split_kernel<T, kLanes, 2, kTail>), grid,
                       dim3(kAttnThreads), 0, s, a);
  else
    hipLaunchKernelGGL((decode_attention_split_kernel<T, kLanes, 4, kTail>), grid,
                       dim3(kAttnThreads), 0, s, a);
}

// DA_PHASE_FIRST: prefix (minus fresh slots) + local segment; DA_PHASE_SECOND: tail +
// merge.  Issued as two calls around a page stream, the first call also merges its own
// chunks (into `out` and into one partial), so that the second call, the part
// the step waits for, merges only that partial and the tail's.
// The page stream and the first attention pass as one launch.
template <typename T, int kLanes>
static void launch_stream_attend(AttnArgs a, const GatherAttendArgs &g, int g_blocks, int n_chunks,
                                 int n_kv_heads, hipStream_t s) {
  a.chunk_base = 0;
  const int rep = a.rep;
  if (rep > 4 && kLanes <= 16) {
    const dim3 grid(g_blocks + n_chunks, n_kv_heads, 1);
    hipLaunchKernelGGL((decode_stream_attend_kernel<T, (kLanes <= 16 ? kLanes : 16), 8, 8>), grid,
                       dim3(kAttnThreads), 0, s, a, g, g_blocks);
  } else {
    const dim3 grid(g_blocks + n_chunks, n_kv_heads, (unsigned)ceil_div(rep, 4));
    if (rep > 4)
      hipLaunchKernelGGL((decode_stream_attend_kernel<T, kLanes, 4, 8>), grid, dim3(kAttnThreads),
                         0, s, a, g, g_blocks);
    else
      hipLaunchKernelGGL((decode_stream_attend_kernel<T, kLanes, 4, 4>), grid, dim3(kAttnThreads),
                         0, s, a, g, g_blocks);
  }
}

template <typename T>
static int launch_attention(const AttnArgs &a, int phase, int n_kv_heads, int lanes, int head_dim,
                            void *out, int64_t out_head_stride, float *lse_out,
                            const GatherAttendArgs *stream_args, hipStream_t s) {
#define DA_ATTN_LAUNCH(tail, first, count)                                     \
  switch (lanes) {                                                             \
    case 4: launch_split<T, 4, tail>(a, first, count, n_kv_heads, s); break;   \
    case 8: launch_split<T, 8, tail>(a, first, count, n_kv_heads, s); break;   \
    case 16: launch_split<T, 16, tail>(a, first, count, n_kv_heads, s); break; \
    case 32: launch_split<T, 32, tail>(a, first, count, n_kv_heads, s); break; \
    case 64: launch_split<T, 64, tail>(a, first, count, n_kv_heads, s); break; \
  }
#define DA_ATTN_MERGE(mode)                                                                    \
  hipLaunchKernelGGL(decode_attention_merge_kernel<T>, dim3(a.n_q_heads), dim3(kMergeThreads), \
                     0, s, a, mode, head_dim, (char *)out, out_head_stride, lse_out)
  if (phase & DA_PHASE_STREAM) {
    const int n_chunks = a.n_pchunks + a.n_lchunks;
    switch (lanes) {
      case 4: launch_stream_attend<T, 4>(a, *stream_args, a.gather_blocks, n_chunks, n_kv_heads, s); break;
      case 8: launch_stream_attend<T, 8>(a, *stream_args, a.gather_blocks, n_chunks, n_kv_heads, s); break;
      case 16: launch_stream_attend<T, 16>(a, *stream_args, a.gather_blocks, n_chunks, n_kv_heads, s); break;
      case 32: launch_stream_attend<T, 32>(a, *stream_args, a.gather_blocks, n_chunks, n_kv_heads, s); break;
    }
    int rc = launch_status("da_decode_attention(page stream + first pass)");
    if (rc) return rc;
  } else if (phase & DA_PHASE_FIRST) {
    DA_ATTN_LAUNCH(false, 0, a.n_pchunks + a.n_lchunks)
    int rc = launch_status("da_decode_attention(split)");
    if (rc) return rc;
  }
  if (phase & DA_PHASE_FIRST_MERGE) {
    DA_ATTN_MERGE(kMergePre);
    int rc = launch_status("da_decode_attention(merge of the first pass)");
    if (rc) return rc;
  }
  if (phase & DA_PHASE_SECOND) {
    // everything in one call and no carried partial: one merge over all chunks
    const bool all = (phase & DA_PHASE_FIRST) && !(phase & DA_PHASE_FIRST_MERGE);
    if (a.gather_blocks > 0) {
      // the re-assigned slots were attended while they were copied
    } else if (a.n_tchunks > 0) {
      DA_ATTN_LAUNCH(true, a.n_pchunks + a.n_lchunks, a.n_tchunks)
      int rc = launch_status("da_decode_attention(tail)");
      if (rc) return rc;
    } else if (!all) {
      return DA_OK;  // the merge of the first pass already wrote the output
    }
    DA_ATTN_MERGE(all ? kMergeAll : kMergeFinal);
    return launch_status("da_decode_attention(merge)");
  }
#undef DA_ATTN_MERGE
#undef DA_ATTN_LAUNCH
  return DA_OK;
}


template <typename T, int kLanes>
static void launch_gather_attend(const GatherAttendArgs &g, dim3 grid, hipStream_t s) {
  if (g.rep <= 4)
    hipLaunchKernelGGL((pages_gather_attend_kernel<T, kLanes, 4>), grid, dim3(kGatherThreads), 0, s,
                       g);
  else
    hipLaunchKernelGGL((pages_gather_attend_kernel<T, kLanes, 8>), grid, dim3(kGatherThreads), 0, s,
                       g);
}

template <typename T>
static int dispatch_gather_attend(const GatherAttendArgs &g, int lanes, dim3 grid, hipStream_t s) {
  switch (lanes) {
    case 4: launch_gather_attend<T, 4>(g, grid, s); break;
    case 8: launch_gather_attend<T, 8>(g, grid, s); break;
    case 16: launch_gather_attend<T, 16>(g, grid, s); break;
    case 32: launch_gather_attend<T, 32>(g, grid, s); break;
    default: return fail(DA_ENOTSUP, "da_pages_gather_attend: rows of %d bytes", lanes * 16);
  }
  return launch_status("da_pages_gather_attend");
}

}  // namespace da

extern "C" int da_pages_gather_attend(
    const void *dram, int64_t dram_head_stride_bytes, int64_t dram_page_stride_bytes, void *hbm,
    int64_t hbm_head_stride_bytes, int64_t hbm_slot_stride_bytes, int page_size,
    const int32_t *miss_page, const int32_t *miss_slot, const int32_t *miss_count, int n_kv_heads,
    int k, int blocks_per_head, const void *q, int64_t q_head_stride, int n_q_heads, int head_dim,
    int dtype, float scale, int64_t p_len, int64_t c_capacity, void *workspace,
    size_t workspace_bytes, void *stream) {
  using namespace da;
  DA_REQUIRE(n_kv_heads > 0 && n_q_heads > 0 && n_q_heads % n_kv_heads == 0 && k > 0 &&
                 page_size > 0 && p_len >= 0 && c_capacity >= 0,
             "da_pages_gather_attend: bad geometry");
  DA_REQUIRE(dtype == DA_F32 || dtype == DA_F16 || dtype == DA_BF16,
             "da_pages_gather_attend: unknown dtype %d", dtype);
  DA_REQUIRE(dram && hbm && miss_page && miss_slot && miss_count && q && workspace,
             "da_pages_gather_attend: null pointer");
  DA_REQUIRE(blocks_per_head >= 1 && (int64_t)blocks_per_head * n_kv_heads <= kGatherMaxBlocks,
             "da_pages_gather_attend: blocks_per_head %d x %d kv heads not in 1..%d",
             blocks_per_head, n_kv_heads, kGatherMaxBlocks);
  const int lanes = lanes_of(head_dim, dtype);
  const int rep = n_q_heads / n_kv_heads;
  const int64_t page_vecs = (int64_t)page_size * 2 * lanes;
  if (!lanes || lanes > 32 || rep > 8 || page_vecs > kGatherThreads * kGatherMaxLoads ||
      n_kv_heads > 65535)
    return fail(DA_ENOTSUP,
                "da_pages_gather_attend: needs rows of 64..512 bytes, at most 8 query heads per kv "
                "head and pages up to %d bytes (use da_pages_gather and the tail pass instead)",
                kGatherThreads * kGatherMaxLoads * 16);
  const int vec = dtype == DA_F32 ? 4 : 8;
  DA_REQUIRE(dram_head_stride_bytes % 16 == 0 && dram_page_stride_bytes % 16 == 0 &&
                 hbm_head_stride_bytes % 16 == 0 && hbm_slot_stride_bytes % 16 == 0 &&
                 (uintptr_t)dram % 16 == 0 && (uintptr_t)hbm % 16 == 0 && (uintptr_t)q % 16 == 0 &&
                 q_head_stride % vec == 0 && (uintptr_t)workspace % 16 == 0,
             "da_pages_gather_attend: operands must be 16-byte aligned");
  const ChunkPlan p = plan_chunks(n_kv_heads, lanes, p_len, c_capacity, (int64_t)k * page_size);
  const size_t need = attn_workspace_bytes(n_q_heads, head_dim, p.total());
  DA_REQUIRE(workspace_bytes >= need, "da_pages_gather_attend: workspace %zu < %zu bytes",
             workspace_bytes, need);
  GatherAttendArgs g = {};
  g.dram = (const char *)dram;
  g.dram_head_stride = dram_head_stride_bytes;
  g.dram_page_stride = dram_page_stride_bytes;
  g.hbm = (char *)hbm;
  g.hbm_head_stride = hbm_head_stride_bytes;
  g.hbm_slot_stride = hbm_slot_stride_bytes;
  g.page_vecs = (int)page_vecs;
  g.miss_page = miss_page;
  g.miss_slot = miss_slot;
  g.miss_count = miss_count;
  g.K = k;
  g.q = (const char *)q;
  g.q_head_stride = q_head_stride;
  g.rep = rep;
  g.n_q_heads = n_q_heads;
  g.n_kv_heads = n_kv_heads;
  g.scale_log2 = scale * kLog2e;
  g.part_acc = (float *)workspace;
  g.part_ml = g.part_acc + (size_t)p.total() * n_q_heads * head_dim;
  g.chunk0 = p.gather_chunk0();
  const dim3 grid(blocks_per_head, n_kv_heads);
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case DA_F32: return dispatch_gather_attend<F32>(g, lanes, grid, s);
    case DA_F16: return dispatch_gather_attend<F16>(g, lanes, grid, s);
    default: return dispatch_gather_attend<BF16>(g, lanes, grid, s);
  }
}

extern "C" size_t da_decode_attention_workspace_bytes(int n_q_heads, int n_kv_heads,
                                                      int head_dim, int dtype, int64_t p_len,
                                                      int64_t c_capacity, int64_t miss_tokens) {
  using namespace da;
  if (n_q_heads <= 0 || n_kv_heads <= 0 || p_len < 0 || c_capacity < 0 || miss_tokens < 0)
    return 0;
  const int lanes = lanes_of(head_dim, dtype);
  if (!lanes) return 0;
  const ChunkPlan p = plan_chunks(n_kv_heads, lanes, p_len, c_capacity, miss_tokens);
  return attn_workspace_bytes(n_q_heads, head_dim, p.total()) + 16;
}

extern "C" int da_decode_attention_paged(
    const void *q, int64_t q_head_stride, int n_q_heads, int n_kv_heads, int head_dim, int dtype,
    const void *pk, const void *pv, int64_t p_tok_stride, int64_t p_head_stride, int64_t p_len,
    void *ck, void *cv, int64_t c_tok_stride, int64_t c_head_stride, int64_t c_capacity,
    int64_t c_len, const int32_t *c_len_dev, const void *new_k, const void *new_v,
    int64_t new_head_stride, float scale, void *out, int64_t out_head_stride, float *lse_out,
    void *workspace, size_t workspace_bytes, const da_paged_overlap *overlap, void *stream) {
  using namespace da;
  DA_REQUIRE(n_q_heads > 0 && n_kv_heads > 0 && n_q_heads % n_kv_heads == 0,
             "da_decode_attention: %d query heads do not split over %d kv heads", n_q_heads,
             n_kv_heads);
  DA_REQUIRE(dtype == DA_F32 || dtype == DA_F16 || dtype == DA_BF16,
             "da_decode_attention: unknown dtype %d", dtype);
  DA_REQUIRE(p_len >= 0 && c_capacity >= 0 && (c_len >= 0 || c_len_dev),
             "da_decode_attention: negative length");
  DA_REQUIRE(q && out && workspace, "da_decode_attention: null pointer");
  DA_REQUIRE(p_len == 0 || (pk && pv), "da_decode_attention: null prefix segment");
  DA_REQUIRE(c_capacity == 0 || (ck && cv), "da_decode_attention: null local cache");
  DA_REQUIRE((new_k == nullptr) == (new_v == nullptr),
             "da_decode_attention: new_k and new_v must come together");
  DA_REQUIRE(new_k == nullptr || c_capacity > 0,
             "da_decode_attention: appending needs a local cache");
  if (!c_len_dev)
    DA_REQUIRE(c_len + (new_k ? 1 : 0) <= c_capacity,
               "da_decode_attention: local cache overflow (%lld rows + new token > capacity %lld)",
               (long long)c_len, (long long)c_capacity);
  const int lanes = lanes_of(head_dim, dtype);
  if (!lanes)
    return fail(DA_ENOTSUP,
                "da_decode_attention: head_dim %d unsupported (row bytes must be 64..1024, a "
                "power of two)",
                head_dim);
  const int vec = dtype == DA_F32 ? 4 : 8;
  DA_REQUIRE(q_head_stride % vec == 0 && p_tok_stride % vec == 0 && p_head_stride % vec == 0 &&
                 c_tok_stride % vec == 0 && c_head_stride % vec == 0 &&
                 new_head_stride % vec == 0 && (uintptr_t)q % 16 == 0 && (uintptr_t)pk % 16 == 0 &&
                 (uintptr_t)pv % 16 == 0 && (uintptr_t)ck % 16 == 0 && (uintptr_t)cv % 16 == 0 &&
                 (uintptr_t)new_k % 16 == 0 && (uintptr_t)new_v % 16 == 0,
             "da_decode_attention: rows must be 16-byte aligned");
  if (n_kv_heads > 65535) return fail(DA_ENOTSUP, "da_decode_attention: too many kv heads");

  AttnArgs a = {};
  a.q = (const char *)q;
  a.q_head_stride = q_head_stride;
  a.rep = n_q_heads / n_kv_heads;
  a.pk = (const char *)pk;
  a.pv = (const char *)pv;
  a.p_tok_stride = p_tok_stride;
  a.p_head_stride = p_head_stride;
  a.p_len = p_len;
  a.ck = (char *)ck;
  a.cv = (char *)cv;
  a.c_tok_stride = c_tok_stride;
  a.c_head_stride = c_head_stride;
  a.c_capacity = c_capacity;
  a.c_len = c_len;
  a.c_len_dev = c_len_dev;
  a.new_k = (const char *)new_k;
  a.new_v = (const char *)new_v;
  a.new_head_stride = new_head_stride;
  a.scale_log2 = scale * kLog2e;
  a.n_q_heads = n_q_heads;
  int phase = 3;
  int64_t miss_tokens = 0;
  if (overlap) {
    DA_REQUIRE(overlap->page_size > 0 && p_len % overlap->page_size == 0,
               "da_decode_attention: the paged prefix must be whole pages");
    DA_REQUIRE(overlap->slot_epoch && overlap->epoch && overlap->miss_slot &&
                   overlap->miss_count && overlap->miss_capacity >= 0,
               "da_decode_attention: incomplete overlap description");
    DA_REQUIRE(overlap->phase >= 1 && overlap->phase <= 15, "da_decode_attention: bad phase %d",
               overlap->phase);
    DA_REQUIRE(!(overlap->phase & DA_PHASE_STREAM) ||
                   ((overlap->phase & DA_PHASE_FIRST) && overlap->gather_blocks >= 1),
               "da_decode_attention: DA_PHASE_STREAM goes with DA_PHASE_FIRST and gather_blocks >= 1");
    a.page_size = overlap->page_size;
    a.page_shift = -1;
    for (int b = 0; b < 31; ++b)
      if ((1 << b) == overlap->page_size) a.page_shift = b;
    a.slot_epoch = overlap->slot_epoch;
    a.slot_epoch_head_stride = overlap->slot_epoch_head_stride;
    a.epoch = overlap->epoch;
    a.miss_slot = overlap->miss_slot;
    a.miss_count = overlap->miss_count;
    a.miss_capacity = overlap->miss_capacity;
    miss_tokens = (int64_t)overlap->miss_capacity * overlap->page_size;
    phase = overlap->phase;
    DA_REQUIRE(overlap->gather_blocks >= 0 &&
                   (int64_t)overlap->gather_blocks * n_kv_heads <= kGatherMaxBlocks &&
                   (overlap->gather_blocks == 0 || miss_tokens > 0),
               "da_decode_attention: gather_blocks %d x %d kv heads out of range (at most %d)",
               overlap->gather_blocks, n_kv_heads, kGatherMaxBlocks);
    a.gather_blocks = overlap->gather_blocks;
  }
  const ChunkPlan p = plan_chunks(n_kv_heads, lanes, p_len, c_capacity, miss_tokens);
  a.chunk = p.chunk;
  a.tail_chunk = p.tail_chunk;
  a.n_pchunks = p.n_p;
  a.n_lchunks = p.n_l;
  a.n_tchunks = p.n_t;
  a.pre_chunk = p.pre_chunk();
  a.gather_chunk0 = p.gather_chunk0();
  const size_t need = attn_workspace_bytes(n_q_heads, head_dim, p.total());
  DA_REQUIRE(workspace_bytes >= need, "da_decode_attention: workspace %zu < %zu bytes",
             workspace_bytes, need);
  DA_REQUIRE((uintptr_t)workspace % 16 == 0,
             "da_decode_attention: workspace must be 16-byte aligned");
  a.part_acc = (float *)workspace;
  a.part_ml = a.part_acc + (size_t)p.total() * n_q_heads * head_dim;
  hipStream_t s = (hipStream_t)stream;
  if (p.n_p + p.n_l == 0) return fail(DA_EINVAL, "da_decode_attention: no key/value rows at all");
  GatherAttendArgs g = {};
  if (phase & DA_PHASE_STREAM) {
    const int64_t page_vecs = (int64_t)overlap->page_size * 2 * lanes;
    if (lanes > 32 || a.rep > 8 || page_vecs > kGatherThreads * kGatherMaxLoads)
      return fail(DA_ENOTSUP,
                  "da_decode_attention: DA_PHASE_STREAM needs rows of 64..512 bytes, at most 8 query "
                  "heads per kv head and pages up to %d bytes",
                  kGatherThreads * kGatherMaxLoads * 16);
    DA_REQUIRE(overlap->dram && overlap->hbm && overlap->miss_page,
               "da_decode_attention: DA_PHASE_STREAM without the page stream's operands");
    DA_REQUIRE(overlap->dram_head_stride_bytes % 16 == 0 &&
                   overlap->dram_page_stride_bytes % 16 == 0 &&
                   overlap->hbm_head_stride_bytes % 16 == 0 &&
                   overlap->hbm_slot_stride_bytes % 16 == 0 && (uintptr_t)overlap->dram % 16 == 0 &&
                   (uintptr_t)overlap->hbm % 16 == 0,
               "da_decode_attention: page stores must be 16-byte aligned");
    g.dram = (const char *)overlap->dram;
    g.dram_head_stride = overlap->dram_head_stride_bytes;
    g.dram_page_stride = overlap->dram_page_stride_bytes;
    g.hbm = (char *)overlap->hbm;
    g.hbm_head_stride = overlap->hbm_head_stride_bytes;
    g.hbm_slot_stride = overlap->hbm_slot_stride_bytes;
    g.page_vecs = (int)page_vecs;
    g.miss_page = overlap->miss_page;
    g.miss_slot = overlap->miss_slot;
    g.miss_count = overlap->miss_count;
    g.K = overlap->miss_capacity;
    g.q = a.q;
    g.q_head_stride = q_head_stride;
    g.rep = a.rep;
    g.n_q_heads = n_q_heads;
    g.n_kv_heads = n_kv_heads;
    g.scale_log2 = a.scale_log2;
    g.part_acc = a.part_acc;
    g.part_ml = a.part_ml;
    g.chunk0 = a.gather_chunk0;
  }
  switch (dtype) {
    case DA_F32:
      return launch_attention<F32>(a, phase, n_kv_heads, lanes, head_dim, out, out_head_stride,
                                   lse_out, &g, s);
    case DA_F16:
      return launch_attention<F16>(a, phase, n_kv_heads, lanes, head_dim, out, out_head_stride,
                                   lse_out, &g, s);
    default:
      return launch_attention<BF16>(a, phase, n_kv_heads, lanes, head_dim, out, out_head_stride,
                                    lse_out, &g, s);
  }
}

extern "C" int da_decode_attention(const void *q, int64_t q_head_stride, int n_q_heads,
                                   int n_kv_heads, int head_dim, int dtype, const void *pk,
                                   const void *pv, int64_t p_tok_stride, int64_t p_head_stride,
                                   int64_t p_len, void *ck, void *cv, int64_t c_tok_stride,
                                   int64_t c_head_stride, int64_t c_capacity, int64_t c_len,
                                   const int32_t *c_len_dev, const void *new_k,
                                   const void *new_v, int64_t new_head_stride, float scale,
                                   void *out, int64_t out_head_stride, float *lse_out,
                                   void *workspace, size_t workspace_bytes, void *stream) {
  return da_decode_attention_paged(q, q_head_stride, n_q_heads, n_kv_heads, head_dim, dtype, pk,
                                   pv, p_tok_stride, p_head_stride, p_len, ck, cv, c_tok_stride,
                                   c_head_stride, c_capacity, c_len, c_len_dev, new_k, new_v,
                                   new_head_stride, scale, out, out_head_stride, lse_out,
                                   workspace, workspace_bytes, nullptr, stream);
}
