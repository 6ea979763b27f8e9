// Decode attention, shared parts: the argument block, the 16-byte row loaders,
// the per-block split-K pass over one chunk of keys/values, and the chunk
// geometry of a launch.  Used by the split/merge launches (decode_attention.hip)
// and by the launch that also carries the page stream (stream_attention.hip).
#pragma once
#include "common.hpp"

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
constexpr int kAttnUnroll = 4;  // tokens in flight per lane group (even)

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

inline int pick_chunk(int64_t p_len, int64_t c_capacity, int n_kv_heads, int step_tokens) {
  // ~2 blocks per CU on a 256-CU part: every block pays a fixed prologue and a
  // merge epilogue, so few long chunks beat many short ones (measured on the
  // 128K workload: 31.9 us at 512 blocks, 32.6 us at 2048); never below one
  // unrolled round.
  const int64_t want_blocks = 256 * 2;
  int64_t chunk = (p_len + c_capacity) * n_kv_heads / want_blocks;
  const int round = step_tokens * kAttnUnroll;
  if (chunk < round) chunk = round;
  if (chunk > 4096) chunk = 4096;
  chunk = ceil_div(chunk, round) * round;
  // The two segments are cut separately, so each may add a short last chunk, and a
  // few blocks beyond what the part holds at once run as a second round behind
  // all the others (128K workload: 65 chunks x 8 heads = 520 blocks of 576 tokens
  // take 28.6 us, 59 x 8 = 472 blocks of 640 tokens 26.4 us).
  while (chunk < 4096 &&
         (ceil_div(p_len, chunk) + ceil_div(c_capacity, chunk)) * n_kv_heads > want_blocks)
    chunk += round;
  return (int)chunk;
}

inline int lanes_of(int head_dim, int dtype) {
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
inline ChunkPlan plan_chunks(int n_kv_heads, int lanes, int64_t p_len, int64_t c_capacity,
                             int64_t miss_tokens) {
  const int step_tokens = kAttnWaves * (64 / lanes);
  ChunkPlan p;
  p.chunk = pick_chunk(p_len, c_capacity, n_kv_heads, step_tokens);
  p.n_p = (int)ceil_div(p_len, p.chunk);
  p.n_l = (int)ceil_div(c_capacity, p.chunk);
  // the tail is short and every block starts with a dependent slot lookup:
  // one unrolled round per block keeps it wide instead of deep
  p.tail_chunk = step_tokens * kAttnUnroll;
  p.n_t = (int)ceil_div(miss_tokens, p.tail_chunk);
  return p;
}

inline size_t attn_workspace_bytes(int n_q_heads, int head_dim, int64_t n_chunks) {
  return (size_t)n_chunks * n_q_heads * (head_dim + 2) * sizeof(float);
}

}  // namespace da
