// Page stream with attention riding on it.  A block copies its range of the
// miss lists (all kv heads taken as one list, see stream_range) from the host
// page store into their slots, 16 bytes per lane, and the registers the page passes
// through also feed the attention of this step's query over that page: the
// re-assigned slots then need no second pass after the stream has finished.
// A page holds page_size tokens, each token its K row followed by its V row,
// so 2*kLanes adjacent lanes hold one token: the lower kLanes its key (they
// produce the score), the upper kLanes its value (they keep the softmax state
// and the weighted sum).  The next page's loads are issued before the current
// page is stored and attended, so the host link never waits for arithmetic.
// Every block with an entry to copy leaves one partial (all query rows of the
// kv head) at chunk id chunk0 + block_x for each kv head its range touched.
#pragma once
#include "attention_core.hpp"

namespace da {

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
      buf[u] = load16_stream(v >= 0 && j < g.page_vecs ? src + (int64_t)j * 16 : g.q);
    }
  };
  auto settle = [&](const u32x4 *buf, char *dst) {
    if (dst == nullptr) return;
#pragma unroll
    for (int u = 0; u < kGatherMaxLoads; ++u) {
      const int j = u * kGatherThreads + tid;
      // (streaming stores: a slot is next read a step later, behind the whole first pass)
      if (j < g.page_vecs) store16_stream(dst + (int64_t)j * 16, buf[u]);
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

// The page stream and the first attention pass as one launch (stream_attention.hip).
// link_gbps / block_gbps: what a kernel's reads of the host store reach on this box,
// and what one workgroup alone on its compute unit reads from HBM (0 = defaults).
int launch_stream_attend(const AttnArgs &a, const GatherAttendArgs &g, int dtype, int lanes,
                         int n_chunks, int n_kv_heads, float link_gbps, float block_gbps,
                         hipStream_t s);

}  // namespace da
