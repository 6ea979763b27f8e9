// Launches that carry the page stream: the attending stream alone
// (da_pages_gather_attend) and the stream plus the first attention pass in one
// grid (what da_decode_attention_paged issues for DA_PHASE_STREAM).  Neither
// has a counterpart in the reference, which copies pages with index_select /
// index_copy_ (dram_attention/lru_cache.py:224-241) before it attends.
#include <type_traits>

#include "attention_mfma.hpp"
#include "page_stream.hpp"

namespace da {

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

// Whether the page stream of a launch is long enough to hide a first attention
// pass that only n_core blocks per kv head compute, each walking every
// n_core-th chunk.  The stream is bound by the host link (link_bytes_per_us, the
// rate of reads issued by a kernel on this box: the caller measures it); a block
// alone on its compute unit reads a chunk at block_bytes_per_us plus a
// microsecond of set-up; the pass should be over at 0.7 of the stream.  Only
// time depends on the two rates, never a result: whoever computes a chunk
// leaves the same partial.
struct StreamRates {
  float link_bytes_per_us, block_bytes_per_us;
};
constexpr float kDefaultLinkGBps = 54.f, kDefaultBlockGBps = 30.f;
__device__ __forceinline__ bool stream_hides_few_blocks(int64_t stream_bytes, int64_t chunk_bytes,
                                                        int n_chunks, int n_core,
                                                        const StreamRates &r) {
  const float stream_us = (float)stream_bytes / r.link_bytes_per_us;
  const float chunk_us = (float)chunk_bytes / r.block_bytes_per_us + 1.0f;
  const float rounds = (float)((n_chunks + n_core - 1) / n_core);
  return rounds * chunk_us <= stream_us * 0.7f;
}

// The same with the matrix-core form of the attention pass (one block takes all
// query rows of a kv head, so the grid has no row dimension).
// One launch, two roles, blocks numbered in one dimension and dispatched in that
// order: for every kv head its g_blocks blocks of the page stream and n_core
// blocks of the first attention pass, then one block for every other chunk.
// Next to a short stream every attention block computes one chunk.  Next to a
// long one only the core blocks work, on every n_core-th chunk of their head
// (same chunks, same partial results, whoever computes them), and the others
// leave at once: the few blocks dispatched first land on compute units of their
// own, where a block of the stream is not slowed by attention blocks beside it
// (and does not slow them: an attention block that shares a compute unit with a
// stream block takes four times as long per chunk), and the pass, though it takes
// longer, still ends well before the stream does.  128K shape, 59 chunks per kv
// head: 182.2 us per step instead of 184.1.
template <typename T, int kLanes, int kRowsAttn, int kRowsGather>
__global__ void __launch_bounds__(kAttnThreads)
decode_stream_attend_tile_kernel(const AttnArgs a, const GatherAttendArgs g, const int g_blocks,
                                 const int n_core, const int n_chunks, const StreamRates rates) {
  const int b = blockIdx.x;
  const int per_head = g_blocks + n_core;
  const int n_first = per_head * g.n_kv_heads;
  if (b < n_first && b % per_head < g_blocks) {
    gather_attend_block<T, kLanes, kRowsGather>(g, b / per_head * g_blocks + b % per_head,
                                                g_blocks * g.n_kv_heads);
    return;
  }
  int64_t missed = 0;
  for (int hh = 0; hh < g.n_kv_heads; ++hh) missed += g.miss_count[hh];
  const bool few = stream_hides_few_blocks(missed * g.page_vecs * 16,
                                           (int64_t)a.chunk * kLanes * 16 * 2, n_chunks, n_core,
                                           rates);
  int h, first;
  if (b < n_first) {
    h = b / per_head;
    first = b % per_head - g_blocks;
  } else {
    if (few) return;
    const int rest = n_chunks - n_core;
    h = (b - n_first) / rest;
    first = n_core + (b - n_first) % rest;
  }
  if (!few) {
    attention_tile_block<T, kLanes * 8, kRowsAttn>(a, first, h);
    return;
  }
  // (streaming loads: the pass has time, and the next step's scorer finds its
  // summaries still in the memory-side cache: 128K shape, 0.4 us per step)
  for (int c = first; c < n_chunks; c += n_core) {
    attention_tile_block<T, kLanes * 8, kRowsAttn, true>(a, c, h);
    __syncthreads();  // the block's LDS is used again
  }
}

template <typename T, int kLanes>
static void launch_stream_attend(AttnArgs a, const GatherAttendArgs &g, int g_blocks, int n_chunks,
                                 int n_kv_heads, const StreamRates &rates, hipStream_t s) {
  a.chunk_base = 0;
  const int rep = a.rep;
  // (rows of 512 bytes stay with the vector pass here: both roles' LDS would not fit a block)
  if constexpr (T::kBytes == 2 && (kLanes == 8 || kLanes == 16)) {
    const int dtype = std::is_same<T, BF16>::value ? DA_BF16 : DA_F16;
    if (tile_pass_supported(dtype, kLanes * 8, rep, a.slot_epoch != nullptr, a.page_size)) {
      // core blocks and stream blocks together stay well below the number of compute units
      int n_core = 64 / n_kv_heads > 1 ? 64 / n_kv_heads : 1;
      if (n_core > n_chunks) n_core = n_chunks;
      const dim3 grid((g_blocks + n_chunks) * n_kv_heads, 1, 1);
      if (rep > 4)
        hipLaunchKernelGGL((decode_stream_attend_tile_kernel<T, kLanes, 8, 8>), grid,
                           dim3(kAttnThreads), 0, s, a, g, g_blocks, n_core, n_chunks, rates);
      else
        hipLaunchKernelGGL((decode_stream_attend_tile_kernel<T, kLanes, 4, 4>), grid,
                           dim3(kAttnThreads), 0, s, a, g, g_blocks, n_core, n_chunks, rates);
      return;
    }
  }
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
static int dispatch_stream_attend(const AttnArgs &a, const GatherAttendArgs &g, int lanes,
                                  int n_chunks, int n_kv_heads, const StreamRates &rates,
                                  hipStream_t s) {
  switch (lanes) {
    case 4: launch_stream_attend<T, 4>(a, g, a.gather_blocks, n_chunks, n_kv_heads, rates, s); break;
    case 8: launch_stream_attend<T, 8>(a, g, a.gather_blocks, n_chunks, n_kv_heads, rates, s); break;
    case 16: launch_stream_attend<T, 16>(a, g, a.gather_blocks, n_chunks, n_kv_heads, rates, s); break;
    case 32: launch_stream_attend<T, 32>(a, g, a.gather_blocks, n_chunks, n_kv_heads, rates, s); break;
    default: return fail(DA_ENOTSUP, "page stream with attention: rows of %d bytes", lanes * 16);
  }
  return launch_status("da_decode_attention(page stream + first pass)");
}

int launch_stream_attend(const AttnArgs &a, const GatherAttendArgs &g, int dtype, int lanes,
                         int n_chunks, int n_kv_heads, float link_gbps, float block_gbps,
                         hipStream_t s) {
  // 1 GB/s = 1000 bytes per microsecond; 0 = the rates of the box this was tuned on
  const StreamRates rates = {(link_gbps > 0.f ? link_gbps : kDefaultLinkGBps) * 1000.f,
                             (block_gbps > 0.f ? block_gbps : kDefaultBlockGBps) * 1000.f};
  switch (dtype) {
    case DA_F32: return dispatch_stream_attend<F32>(a, g, lanes, n_chunks, n_kv_heads, rates, s);
    case DA_F16: return dispatch_stream_attend<F16>(a, g, lanes, n_chunks, n_kv_heads, rates, s);
    default: return dispatch_stream_attend<BF16>(a, g, lanes, n_chunks, n_kv_heads, rates, s);
  }
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
