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
#include <type_traits>

#include "attention_mfma.hpp"
#include "page_stream.hpp"

namespace da {

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

  // Partial rows: a thread owns four adjacent channels (one 16-byte lane) of every
  // lanes_c-th live chunk, four rows in flight.  Their addresses do not depend on
  // the statistics, so the first batch (usually all of them) is requested before
  // the statistics are staged and reduced: one memory round trip instead of two.
  __shared__ float sm_acc[kMergeThreads * 4];
  const int quads = head_dim / 4;              // 16-byte lanes per row (head_dim % 4 == 0 here)
  const int lanes_c = kMergeThreads / quads;   // chunk lanes
  const int qd = t % quads, cl = t / quads;
  const bool rows_mine = cl < lanes_c && cl < n_live;
  float4 v[4];
  auto load_rows = [&](int i0) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i = i0 + u * lanes_c;
      const int ic = i < n_live ? i : cl;  // clamp the address; the weight will be zero
      const int64_t slot = (int64_t)chunk_of(ic) * a.n_q_heads + hq;
      v[u] = *(const float4 *)(a.part_acc + slot * head_dim + qd * 4);
    }
  };
  if (rows_mine) load_rows(cl);

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

  float at[4] = {0.f, 0.f, 0.f, 0.f};
  if (rows_mine) {
    for (int i0 = cl; i0 < n_live; i0 += 4 * lanes_c) {
      if (i0 != cl) load_rows(i0);
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int i = i0 + u * lanes_c;
        const float w = i < n_live ? fast_exp2(stat(i).x - mx) : 0.f;
        at[0] = fmaf(v[u].x, w, at[0]);
        at[1] = fmaf(v[u].y, w, at[1]);
        at[2] = fmaf(v[u].z, w, at[2]);
        at[3] = fmaf(v[u].w, w, at[3]);
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

// The matrix-core form of the pass, for the shapes it takes.
template <typename T, int kD>
static void launch_tile(const AttnArgs &a, int n_launch, int n_kv_heads, hipStream_t s) {
  const dim3 grid(n_launch, n_kv_heads, 1);
  if (a.rep <= 4)
    hipLaunchKernelGGL((decode_attention_tile_kernel<T, kD, 4>), grid, dim3(kAttnThreads), 0, s, a);
  else if (a.rep <= 8)
    hipLaunchKernelGGL((decode_attention_tile_kernel<T, kD, 8>), grid, dim3(kAttnThreads), 0, s, a);
  else
    hipLaunchKernelGGL((decode_attention_tile_kernel<T, kD, 16>), grid, dim3(kAttnThreads), 0, s, a);
}

template <typename T, int kLanes, bool kTail>
static void launch_split(AttnArgs a, int first_chunk, int n_launch, int n_kv_heads,
                         hipStream_t s) {
  if (n_launch <= 0) return;
  a.chunk_base = first_chunk;
  const int rep = a.rep;
  if constexpr (!kTail && T::kBytes == 2 && (kLanes == 8 || kLanes == 16 || kLanes == 32)) {
    const int dtype = std::is_same<T, BF16>::value ? DA_BF16 : DA_F16;
    if (tile_pass_supported(dtype, kLanes * 8, rep, a.slot_epoch != nullptr, a.page_size)) {
      launch_tile<T, kLanes * 8>(a, n_launch, n_kv_heads, s);
      return;
    }
  }
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
// DA_PHASE_STREAM: the page stream and the first pass as one launch.
template <typename T>
static int launch_attention(const AttnArgs &a, int dtype, int phase, int n_kv_heads, int lanes,
                            int head_dim, void *out, int64_t out_head_stride, float *lse_out,
                            const GatherAttendArgs *stream_args, float link_gbps, float block_gbps,
                            hipStream_t s) {
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
    int rc = launch_stream_attend(a, *stream_args, dtype, lanes, a.n_pchunks + a.n_lchunks,
                                  n_kv_heads, link_gbps, block_gbps, s);
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
    const bool all = ((phase & DA_PHASE_FIRST) && !(phase & DA_PHASE_FIRST_MERGE)) ||
                     (phase & DA_PHASE_MERGE_ALL);
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

}  // namespace da

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
    DA_REQUIRE(overlap->phase >= 1 && overlap->phase <= 31, "da_decode_attention: bad phase %d",
               overlap->phase);
    DA_REQUIRE(!(overlap->phase & DA_PHASE_MERGE_ALL) ||
                   ((overlap->phase & DA_PHASE_SECOND) && !(overlap->phase & DA_PHASE_FIRST_MERGE)),
               "da_decode_attention: DA_PHASE_MERGE_ALL goes with DA_PHASE_SECOND and without "
               "DA_PHASE_FIRST_MERGE");
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
  float link_gbps = 0.f, block_gbps = 0.f;
  if (phase & DA_PHASE_STREAM) {
    DA_REQUIRE(overlap->link_gbps >= 0.f && overlap->block_gbps >= 0.f,
               "da_decode_attention: negative rate in the overlap description");
    link_gbps = overlap->link_gbps;
    block_gbps = overlap->block_gbps;
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
      return launch_attention<F32>(a, dtype, phase, n_kv_heads, lanes, head_dim, out,
                                   out_head_stride, lse_out, &g, link_gbps, block_gbps, s);
    case DA_F16:
      return launch_attention<F16>(a, dtype, phase, n_kv_heads, lanes, head_dim, out,
                                   out_head_stride, lse_out, &g, link_gbps, block_gbps, s);
    default:
      return launch_attention<BF16>(a, dtype, phase, n_kv_heads, lanes, head_dim, out,
                                    out_head_stride, lse_out, &g, link_gbps, block_gbps, s);
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

// ---- the same attention for callers that cannot allocate -------------------
// The partial results live in a file-scope device array instead of a workspace
// the caller brings.  The array's name is only a host-side handle: the device
// address is looked up once per device with hipGetSymbolAddress and kept; every
// GPU holds its own copy of the array at its own address.
namespace da {
constexpr size_t kStaticScratchBytes = DA_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static void *volatile scratch_ptr[kMaxDevices];  // device address of `scratch`, per device

// Device address of `scratch` on the current device.  Two threads that race on
// the first call both look the address up and store the same value.
static int static_scratch(void **ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return fail((int)e, "da_decode_attention_static: hipGetDevice: %s", hipGetErrorString(e));
  }
  if (dev < 0 || dev >= kMaxDevices)
    return fail(DA_ENOTSUP, "da_decode_attention_static: device %d beyond the %d this library tracks",
                dev, kMaxDevices);
  void *p = __atomic_load_n(&scratch_ptr[dev], __ATOMIC_ACQUIRE);
  if (!p) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      (void)hipGetLastError();
      return fail(e != hipSuccess ? (int)e : DA_EINVAL,
                  "da_decode_attention_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
    }
    __atomic_store_n(&scratch_ptr[dev], p, __ATOMIC_RELEASE);
  }
  *ptr = p;
  return DA_OK;
}
}  // namespace da

extern "C" size_t da_decode_attention_static_capacity(void) { return da::kStaticScratchBytes; }

extern "C" int da_decode_attention_static(const void *q, int64_t q_head_stride, int n_q_heads,
                                          int n_kv_heads, int head_dim, int dtype, const void *pk,
                                          const void *pv, int64_t p_tok_stride,
                                          int64_t p_head_stride, int64_t p_len, void *ck, void *cv,
                                          int64_t c_tok_stride, int64_t c_head_stride,
                                          int64_t c_capacity, int64_t c_len,
                                          const int32_t *c_len_dev, const void *new_k,
                                          const void *new_v, int64_t new_head_stride, float scale,
                                          void *out, int64_t out_head_stride, float *lse_out,
                                          void *stream) {
  using namespace da;
  const size_t need = da_decode_attention_workspace_bytes(n_q_heads, n_kv_heads, head_dim, dtype,
                                                          p_len, c_capacity, 0);
  if (need == 0)
    return fail(DA_EINVAL, "da_decode_attention_static: bad shape (heads %d/%d, head_dim %d, dtype %d, "
                "lengths %lld/%lld)", n_q_heads, n_kv_heads, head_dim, dtype, (long long)p_len,
                (long long)c_capacity);
  if (need > kStaticScratchBytes)
    return fail(DA_ENOTSUP,
                "da_decode_attention_static: this shape needs %zu bytes of partial results, the "
                "built-in buffer holds %zu; use da_decode_attention with a workspace",
                need, kStaticScratchBytes);
  void *ws = nullptr;
  int rc = static_scratch(&ws);
  if (rc) return rc;
  return da_decode_attention_paged(q, q_head_stride, n_q_heads, n_kv_heads, head_dim, dtype, pk, pv,
                                   p_tok_stride, p_head_stride, p_len, ck, cv, c_tok_stride,
                                   c_head_stride, c_capacity, c_len, c_len_dev, new_k, new_v,
                                   new_head_stride, scale, out, out_head_stride, lse_out, ws,
                                   kStaticScratchBytes, nullptr, stream);
}
