// LRU lookup / touch / evict / slot-assign for one decode step, and the
// grid-wide gather that fills the assigned slots from the DRAM page store.
// Counterpart of dram_attention/lru_triton_kernel.py:6-194 of the reference.
//
// The reference walks the K requested pages of a head serially (one Triton
// program per head) and needs a full stable argsort of the access times first.
// When K <= N_hbm the walk is order-independent except for which victim each
// distinct missed page receives, and that is fixed by ranks:
//   the i-th distinct missed page (in visiting order) takes the slot with the
//   i-th smallest (access_time, slot) after this step's hits were touched.
// Proof sketch: touched slots carry the largest time, so they sort behind the
// M <= K - T victims consumed; a victim's old page is resident and untouched,
// hence not among the requests, so no later request observes the eviction.
// So the kernel does: touch hits and find the first occurrence of every missed
// page (an open-addressing table in LDS, page -> lowest request position; for
// more than 4096 requests per head an atomicMin marker in the page->slot map),
// rank those occurrences with ballots and a scan over the waves, take the M
// least-recent untouched slots in order (from the caller's candidate list, or
// select_sorted over all slots), and rewrite both maps in parallel.
// K > N_hbm (victims may wrap onto pages touched in the same step) keeps the
// reference's literal serial walk on one lane per head.
//
// Bound: latency; algorithmic bytes are the metadata only.
#include "lru_keys.hpp"

namespace da {

constexpr int kLruMaxK = 8192;  // distinct-miss list kept in LDS (parallel path)

constexpr int kLruTableMaxK = 4096;  // requests per head whose first misses are found in LDS
constexpr int kLruBitmapSlots = 65536;  // slots per head whose hits are noted in LDS
constexpr int32_t kNotFetched = -2;  // (a slot's old page was not requested ahead of time)

struct LruShared {
  SelectShared sel;
  int32_t miss_page[kLruMaxK];
  int16_t request_entry[kLruTableMaxK];  // per request: its entry of the page table, or kHit / kNoPage
  uint32_t touched[kLruBitmapSlots / 32];  // one bit per slot: hit in this step
  uint32_t wave_count[kSelWaves];
  uint32_t n_miss;
};
constexpr int16_t kHit = -1, kNoPage = -2;

__device__ __forceinline__ void atomic_min_signed(int32_t *p, int32_t v) { atomicMin(p, v); }
__device__ __forceinline__ void atomic_min_signed(int64_t *p, int64_t v) {
  atomicMin((long long *)p, (long long)v);
}
// Marker a missing page's map entry carries between phases A and B: the
// position of its first request, shifted far below the "absent" value -1.
constexpr int64_t kMarkerBase = -(int64_t(1) << 30);

template <typename IdxT, typename MapT, typename TimeT>
__global__ void __launch_bounds__(kSelThreads)
lru_update_kernel(const IdxT *__restrict__ idx_all, int64_t idx_head_stride, int K,
                  int64_t n_dram_pages, int n_hbm, int32_t *step_ptr, int bump,
                  TimeT *time_all, int64_t time_head_stride, MapT *d2h_all,
                  int64_t d2h_head_stride, MapT *h2d_all, int64_t h2d_head_stride,
                  uint8_t *hit_mask, int32_t *miss_page_out, int32_t *miss_slot_out,
                  int32_t *miss_count, int32_t *slot_epoch_all, int32_t *ticket, int serial,
                  const int32_t *cand_all_in, int k_cand) {
  const int32_t *cand_all = cand_all_in;
  __shared__ LruShared sm;
  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = t >> 6;
  const int h = blockIdx.x;
  const IdxT *idx = idx_all + h * idx_head_stride;
  TimeT *time = time_all + h * time_head_stride;
  MapT *d2h = d2h_all + h * d2h_head_stride;
  MapT *h2d = h2d_all + h * h2d_head_stride;
  uint8_t *hit = hit_mask ? hit_mask + (int64_t)h * K : nullptr;
  int32_t *mpage = miss_page_out + (int64_t)h * K;
  int32_t *mslot = miss_slot_out + (int64_t)h * K;
  int32_t *slot_epoch = slot_epoch_all ? slot_epoch_all + (int64_t)h * n_hbm : nullptr;

  // Every wave reads the step for itself and waits for the value right here
  // (and for the stamp of the candidate list, requested with it).
  int32_t stamp_read = cand_all != nullptr ? cand_all[(int64_t)gridDim.x * k_cand + h] : 0;
  int32_t step_read = *step_ptr;
  asm volatile("" : "+v"(step_read), "+v"(stamp_read)::"memory");  // the values have arrived: what follows cannot pass the reads
  const int32_t step_before = __builtin_amdgcn_readfirstlane(step_read);
  // The list describes the access times as they were when the step counter read
  // `stamp`; every update that bumps the counter changes them.  A list made at
  // another step (or handed to a call that does not bump, whose stamps cannot tell
  // two states apart) is ignored, and the kernel orders the slots itself.
  if (!(bump && __builtin_amdgcn_readfirstlane(stamp_read) == step_before)) cand_all = nullptr;
  const int32_t step = step_before + (bump ? 1 : 0);
  const TimeT now = (TimeT)step;
  // The last head to have read the step publishes the bumped value and re-arms the
  // ticket for the next call.  A head is sixteen readers, one per wave, so it takes
  // its ticket behind the first block barrier of its path: every wave of the block
  // has waited for its own read before it arrives there, and whoever draws the last
  // ticket knows that every read of every head is done; the kernel boundary publishes
  // the stores.  Taken that early rather than at the end, the ticket's trip to memory
  // is over long before the block is.
  auto draw_ticket = [&]() {
    if (bump && t == 0) {
      const int32_t done = atomicAdd(ticket, 1);
      if (done == (int32_t)gridDim.x - 1) {
        *step_ptr = step;
        *ticket = 0;
      }
    }
  };

  if (serial) {
    // -- literal restatement of the reference's three launches ---------------
    for (int k = t; k < K; k += kSelThreads) {
      const int64_t p = (int64_t)idx[k];
      if (p < 0 || p >= n_dram_pages) continue;
      const int64_t s = (int64_t)d2h[p];
      if (s >= 0) time[s] = now;
    }
    __syncthreads();
    draw_ticket();
    LeastRecentKey<TimeT> key{time};
    const uint32_t *order = select_sorted(key, n_hbm, n_hbm, sm.sel);  // full stable order
    if (t == 0) {
      int ep = 0, m = 0;
      for (int k = 0; k < K; ++k) {
        const int64_t p = (int64_t)idx[k];
        if (p < 0 || p >= n_dram_pages) {
          if (hit) hit[k] = 0;
          continue;
        }
        const int64_t s = (int64_t)d2h[p];
        if (s < 0) {
          const int32_t v = (int32_t)order[ep];
          time[v] = now;
          const int64_t old = (int64_t)h2d[v];
          if (old >= 0 && old < n_dram_pages) d2h[old] = (MapT)-1;
          h2d[v] = (MapT)p;
          d2h[p] = (MapT)v;
          mpage[m] = (int32_t)p;
          mslot[m] = v;
          sm.miss_page[v] = m;  // the latest entry that targets slot v (n_hbm <= kLruMaxK here)
          if (slot_epoch) slot_epoch[v] = step;
          ++m;
          ep = ep + 1 == n_hbm ? 0 : ep + 1;
          if (hit) hit[k] = 0;
        } else {
          time[s] = now;
          if (hit) hit[k] = 1;
        }
      }
      sm.n_miss = (uint32_t)m;
      miss_count[h] = m;
    }
    __syncthreads();
    // Only the last entry that targets a slot is live: the slot may have been handed
    // out again later in the walk, to another page or to the same page once more
    // (evicted and requested again), and a consumer that walks the list must meet
    // every slot once.
    const int m = (int)sm.n_miss;
    for (int i = t; i < m; i += kSelThreads)
      if (sm.miss_page[mslot[i]] != i) mslot[i] = -1;
  } else {
    uint32_t n_miss = 0;  // distinct misses so far (the same in every thread)
    const uint64_t below = lane == 0 ? 0ull : (~0ull >> (64 - lane));
    // With the LDS table, hits are also noted in an LDS bitmap, and the head of the
    // candidate list and the pages its slots hold are requested right away, long
    // before the victims are chosen: choosing and re-mapping them then needs no
    // further trip to global memory.
    const bool use_bitmap = K <= kLruTableMaxK && n_hbm <= kLruBitmapSlots;
    int32_t ahead_slot = -1, ahead_old = kNotFetched;
    if (use_bitmap && cand_all != nullptr && t < k_cand) {
      ahead_slot = cand_all[(int64_t)h * k_cand + t];
      if (ahead_slot < 0 || ahead_slot >= n_hbm) ahead_slot = -1;  // not a slot: ignored
      if (ahead_slot >= 0) ahead_old = (int32_t)h2d[ahead_slot];   // (page ids fit 32 bits)
    }
    if (K <= kLruTableMaxK) {
      // -- phases A and B through an LDS table --------------------------------
      // A missed page goes into an open-addressing table in LDS (page -> lowest
      // request position, twice as many entries as requests), and every request
      // remembers its entry: the first occurrences are then found and ranked
      // without another look at global memory.  The table borrows the selection
      // area, which is idle until the victims are chosen.
      int table_bits = 1;
      while ((1 << table_bits) < 2 * K) ++table_bits;
      const uint32_t mask = (1u << table_bits) - 1u;
      int32_t *tab_page = (int32_t *)sm.sel.sel;  // 64 KiB: 2 x 8192 words at most
      int32_t *tab_pos = tab_page + (mask + 1u);
      for (uint32_t i = t; i <= mask; i += kSelThreads) {
        tab_page[i] = -1;
        tab_pos[i] = 0x7fffffff;
      }
      if (use_bitmap)
        for (int i = t; i < (n_hbm + 31) / 32; i += kSelThreads) sm.touched[i] = 0;
      __syncthreads();
      draw_ticket();
      // (the requests of all rounds are in flight together: two trips to memory for
      // the phase, however many rounds of 1024 requests a head has)
      constexpr int kRounds = kLruTableMaxK / kSelThreads;
      int64_t page_of[kRounds], slot_of[kRounds];
#pragma unroll
      for (int r = 0; r < kRounds; ++r) {
        const int k = r * kSelThreads + t;
        page_of[r] = k < K ? (int64_t)idx[k] : -1;
      }
#pragma unroll
      for (int r = 0; r < kRounds; ++r) {
        if (page_of[r] >= n_dram_pages) page_of[r] = -1;
        slot_of[r] = page_of[r] >= 0 ? (int64_t)d2h[page_of[r]] : -1;
      }
#pragma unroll
      for (int r = 0; r < kRounds; ++r) {
        const int k = r * kSelThreads + t;
        if (k >= K) continue;
        const int64_t p = page_of[r];
        int16_t entry = kNoPage;
        if (p >= 0) {
          const int64_t s = slot_of[r];
          if (s >= 0) {
            time[s] = now;
            if (use_bitmap) atomicOr(&sm.touched[s >> 5], 1u << (s & 31));
            entry = kHit;
          } else {
            uint32_t e = ((uint32_t)p * 2654435761u) >> (32 - table_bits);
            while (true) {
              const int32_t old = atomicCAS(&tab_page[e], -1, (int32_t)p);
              if (old == -1 || old == (int32_t)p) break;
              e = (e + 1u) & mask;
            }
            atomicMin(&tab_pos[e], k);  // smallest k wins
            entry = (int16_t)e;
          }
        }
        sm.request_entry[k] = entry;
      }
      __syncthreads();
      for (int base = 0; base < K; base += kSelThreads) {
        const int k = base + t;
        bool first = false;
        int32_t p = -1;
        if (k < K) {
          const int16_t entry = sm.request_entry[k];
          if (entry >= 0) {
            first = tab_pos[entry] == k;
            p = tab_page[entry];
          }
          if (hit) hit[k] = (entry != kNoPage && !first) ? 1 : 0;
        }
        const uint64_t m_first = __ballot(first);
        if (lane == 0) sm.wave_count[wave] = (uint32_t)__popcll(m_first);
        __syncthreads();
        uint32_t round;
        const uint32_t before = n_miss + waves_prefix(sm.wave_count, round);
        if (first) sm.miss_page[before + (uint32_t)__popcll(m_first & below)] = p;
        n_miss += round;
        __syncthreads();  // miss_page is complete so far; wave_count may be rewritten
      }
    } else {
    // -- phase A: touch hits, mark the first occurrence of every missed page --
    for (int k = t; k < K; k += kSelThreads) {
      const int64_t p = (int64_t)idx[k];
      if (p < 0 || p >= n_dram_pages) continue;
      const int64_t s = (int64_t)d2h[p];
      if (s >= 0)
        time[s] = now;
      else
        atomic_min_signed(&d2h[p], (MapT)(kMarkerBase + k));  // smallest k wins
    }
    __syncthreads();
    draw_ticket();
    // -- phase B: rank the first occurrences in visiting order ---------------
    for (int base = 0; base < K; base += kSelThreads) {
      const int k = base + t;
      bool first = false;
      int64_t p = -1;
      if (k < K) {
        p = (int64_t)idx[k];
        if (p >= 0 && p < n_dram_pages) first = (int64_t)d2h[p] == kMarkerBase + k;
        if (hit) hit[k] = (p >= 0 && p < n_dram_pages && !first) ? 1 : 0;
      }
      const uint64_t m_first = __ballot(first);
      if (lane == 0) sm.wave_count[wave] = (uint32_t)__popcll(m_first);
      __syncthreads();
      uint32_t round;
      const uint32_t before = n_miss + waves_prefix(sm.wave_count, round);
      if (first) sm.miss_page[before + (uint32_t)__popcll(m_first & below)] = (int32_t)p;
      n_miss += round;
      __syncthreads();  // miss_page is complete so far; wave_count may be rewritten
    }
    }
    const int m = (int)n_miss;
    // -- phase C: the m least recently used slots, in eviction order ---------
    const uint32_t *victims = nullptr;
    if (m > 0 && cand_all != nullptr && m <= k_cand) {
      // The caller's list of the k_cand least recent slots, made before this call
      // touched anything: untouched slots keep their order and still precede every
      // touched one, so the first m untouched entries are the victims.
      uint32_t kept = 0;  // untouched entries found so far (the same in every thread)
      int32_t *old_page = (int32_t *)sm.sel.sel;  // per victim: the page it held (the table is done with)
      for (int base = 0; base < k_cand && kept < (uint32_t)m; base += kSelThreads) {
        const int i = base + t;
        const bool ahead = use_bitmap && base == 0;
        int32_t slot = ahead ? ahead_slot : i < k_cand ? cand_all[(int64_t)h * k_cand + i] : -1;
        if (slot >= n_hbm) slot = -1;
        const bool untouched =
            slot >= 0 && (use_bitmap ? !((sm.touched[slot >> 5] >> (slot & 31)) & 1u) : time[slot] != now);
        const uint64_t m_un = __ballot(untouched);
        if (lane == 0) sm.wave_count[wave] = (uint32_t)__popcll(m_un);
        __syncthreads();
        uint32_t total;
        const uint32_t before = waves_prefix(sm.wave_count, total);
        if (untouched) {
          const uint32_t at = kept + before + (uint32_t)__popcll(m_un & below);
          sm.sel.idx_out[at] = (uint32_t)slot;
          old_page[at] = ahead ? ahead_old : kNotFetched;
        }
        kept += total;
        __syncthreads();  // idx_out is complete so far; wave_count may be rewritten
      }
      if (kept >= (uint32_t)m) victims = sm.sel.idx_out;  // else: too many were touched
    }
    const bool have_old = victims != nullptr;
    if (m > 0 && victims == nullptr) {
      LeastRecentKey<TimeT> key{time};
      victims = select_sorted(key, n_hbm, m, sm.sel);
    }
    // -- phase D: hand slot i to the i-th distinct missed page ---------------
    for (int i = t; i < m; i += kSelThreads) {
      const int32_t p = sm.miss_page[i];
      const int32_t v = (int32_t)victims[i];
      const int32_t noted = have_old ? ((const int32_t *)sm.sel.sel)[i] : kNotFetched;
      const int64_t old = noted != kNotFetched ? (int64_t)noted : (int64_t)h2d[v];
      if (old >= 0 && old < n_dram_pages) d2h[old] = (MapT)-1;
      h2d[v] = (MapT)p;
      d2h[p] = (MapT)v;
      time[v] = now;
      mpage[i] = p;
      mslot[i] = v;
      if (slot_epoch) slot_epoch[v] = step;
    }
    if (t == 0) miss_count[h] = m;
  }

}

// One 256-thread block per (entry, head), striding over the head's miss list.
// Every lane moves 16 bytes at a time with all of a page's loads issued before
// the first store, so a wave keeps several KiB of host-link reads in flight.
__global__ void __launch_bounds__(256)
pages_gather_kernel(const char *__restrict__ dram, int64_t dram_head_stride,
                    int64_t dram_page_stride, char *__restrict__ hbm, int64_t hbm_head_stride,
                    int64_t hbm_slot_stride, int64_t page_bytes,
                    const int32_t *__restrict__ miss_page, const int32_t *__restrict__ miss_slot,
                    const int32_t *__restrict__ miss_count, int K) {
  const int h = blockIdx.y;
  const int m = miss_count[h];
  const int64_t vecs = page_bytes / 16;
  for (int i = blockIdx.x; i < m; i += gridDim.x) {
    const int32_t v = miss_slot[(int64_t)h * K + i];
    if (v < 0) continue;
    const int32_t p = miss_page[(int64_t)h * K + i];
    const char *src = dram + h * dram_head_stride + p * dram_page_stride;
    char *dst = hbm + h * hbm_head_stride + v * hbm_slot_stride;
    for (int64_t j0 = threadIdx.x; j0 < vecs; j0 += 4 * 256) {
      u32x4 r[4];
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (j0 + u * 256 < vecs) r[u] = load16(src + (j0 + u * 256) * 16);
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (j0 + u * 256 < vecs) store16(dst + (j0 + u * 256) * 16, r[u]);
    }
  }
}

template <typename IdxT, typename MapT>
static void launch_lru_time(int time_type, dim3 grid, hipStream_t s, const void *idx,
                            int64_t idx_hs, int K, int64_t P, int n_hbm, int32_t *step, int bump,
                            void *time, int64_t time_hs, void *d2h, int64_t d2h_hs, void *h2d,
                            int64_t h2d_hs, uint8_t *hit, int32_t *mp, int32_t *ms, int32_t *mc,
                            int32_t *se, int32_t *ticket, int serial, const int32_t *cand,
                            int k_cand) {
  if (time_type == DA_TIME_F32)
    hipLaunchKernelGGL((lru_update_kernel<IdxT, MapT, float>), grid, dim3(kSelThreads), 0, s,
                       (const IdxT *)idx, idx_hs, K, P, n_hbm, step, bump, (float *)time, time_hs,
                       (MapT *)d2h, d2h_hs, (MapT *)h2d, h2d_hs, hit, mp, ms, mc, se, ticket, serial,
                       cand, k_cand);
  else
    hipLaunchKernelGGL((lru_update_kernel<IdxT, MapT, int32_t>), grid, dim3(kSelThreads), 0, s,
                       (const IdxT *)idx, idx_hs, K, P, n_hbm, step, bump, (int32_t *)time,
                       time_hs, (MapT *)d2h, d2h_hs, (MapT *)h2d, h2d_hs, hit, mp, ms, mc, se, ticket,
                       serial, cand, k_cand);
}

}  // namespace da

extern "C" size_t da_lru_update_workspace_bytes(int, int, int64_t, int) { return 256; }

extern "C" int da_lru_update(const void *idx, int64_t idx_head_stride, int idx_itype,
                             int n_kv_heads, int k, int64_t n_dram_pages, int n_hbm_pages,
                             int32_t *step, int flags, void *access_time,
                             int64_t time_head_stride, int time_type, void *d2h,
                             int64_t d2h_head_stride, void *h2d, int64_t h2d_head_stride,
                             int map_itype, uint8_t *hit_mask, int32_t *miss_page,
                             int32_t *miss_slot, int32_t *miss_count, int32_t *slot_epoch,
                             const int32_t *candidates, int k_cand, void *workspace,
                             size_t workspace_bytes, void *stream) {
  using namespace da;
  DA_REQUIRE(k_cand >= 0 && k_cand <= kSelMaxK && (k_cand == 0 || candidates != nullptr),
             "da_lru_update: bad candidate list (%d entries, at most %d)", k_cand, kSelMaxK);
  DA_REQUIRE(n_kv_heads >= 0 && k >= 0 && n_dram_pages >= 0 && n_hbm_pages >= 0,
             "da_lru_update: bad geometry (heads %d k %d pages %lld slots %d)", n_kv_heads, k,
             (long long)n_dram_pages, n_hbm_pages);
  DA_REQUIRE(idx_itype == DA_I32 || idx_itype == DA_I64, "da_lru_update: bad idx type");
  DA_REQUIRE(map_itype == DA_I32 || map_itype == DA_I64, "da_lru_update: bad map type");
  DA_REQUIRE(time_type == DA_TIME_F32 || time_type == DA_TIME_I32,
             "da_lru_update: bad access-time type");
  if (n_kv_heads == 0) return DA_OK;
  DA_REQUIRE(step && access_time && d2h && h2d && miss_page && miss_slot && miss_count,
             "da_lru_update: null pointer");
  DA_REQUIRE(k == 0 || idx, "da_lru_update: null index list");
  DA_REQUIRE(workspace && workspace_bytes >= da_lru_update_workspace_bytes(0, 0, 0, 0),
             "da_lru_update: workspace too small");
  DA_REQUIRE(n_hbm_pages > 0 || k == 0, "da_lru_update: no HBM slots");
  DA_REQUIRE(n_dram_pages <= 0x7fffffff, "da_lru_update: page ids must fit int32");
  DA_REQUIRE((flags & ~(DA_LRU_BUMP_STEP | DA_LRU_SERIAL_WALK)) == 0, "da_lru_update: unknown flags %d", flags);
  const int bump_step = (flags & DA_LRU_BUMP_STEP) ? 1 : 0;
  // The parallel form rests on the stamp of this call being larger than every stored
  // access time (touched slots then sort behind all others).  With DA_LRU_BUMP_STEP
  // the stamp is the bumped step counter, which is; a caller-supplied stamp may tie
  // with stored times, and then only the literal walk gives the reference's result
  // (a slot hit earlier in the walk can be chosen as a victim later in it).
  const bool stamp_may_tie = !bump_step;
  const int serial = ((flags & DA_LRU_SERIAL_WALK) || k > n_hbm_pages || k > kLruMaxK ||
                      stamp_may_tie) ? 1 : 0;
  if (serial && n_hbm_pages > kSelMaxK)
    return fail(DA_ENOTSUP,
                "da_lru_update: %s needs the serial walk, which orders at most %d slots (%d here)",
                stamp_may_tie && k <= n_hbm_pages && !(flags & DA_LRU_SERIAL_WALK)
                    ? "a caller-supplied time stamp (no DA_LRU_BUMP_STEP), which may tie with "
                      "stored access times,"
                    : "this call (more requests than slots, or DA_LRU_SERIAL_WALK)",
                kSelMaxK, n_hbm_pages);
  dim3 grid(n_kv_heads);
  hipStream_t s = (hipStream_t)stream;
  int32_t *ticket = (int32_t *)workspace;
#define DA_LRU_ARGS                                                                          \
  time_type, grid, s, idx, idx_head_stride, k, n_dram_pages, n_hbm_pages, step, bump_step,   \
      access_time, time_head_stride, d2h, d2h_head_stride, h2d, h2d_head_stride, hit_mask,   \
      miss_page, miss_slot, miss_count, slot_epoch, ticket, serial,                          \
      (k_cand > 0 ? candidates : nullptr), k_cand
  if (idx_itype == DA_I64 && map_itype == DA_I64)
    launch_lru_time<int64_t, int64_t>(DA_LRU_ARGS);
  else if (idx_itype == DA_I64)
    launch_lru_time<int64_t, int32_t>(DA_LRU_ARGS);
  else if (map_itype == DA_I64)
    launch_lru_time<int32_t, int64_t>(DA_LRU_ARGS);
  else
    launch_lru_time<int32_t, int32_t>(DA_LRU_ARGS);
#undef DA_LRU_ARGS
  return launch_status("da_lru_update");
}

extern "C" int da_pages_gather(const void *dram, int64_t dram_head_stride_bytes,
                               int64_t dram_page_stride_bytes, void *hbm,
                               int64_t hbm_head_stride_bytes, int64_t hbm_slot_stride_bytes,
                               int64_t page_bytes, const int32_t *miss_page,
                               const int32_t *miss_slot, const int32_t *miss_count,
                               int n_kv_heads, int k, int max_blocks, void *stream) {
  using namespace da;
  DA_REQUIRE(n_kv_heads >= 0 && k >= 0 && page_bytes >= 0, "da_pages_gather: bad geometry");
  if (n_kv_heads == 0 || k == 0 || page_bytes == 0) return DA_OK;
  DA_REQUIRE(dram && hbm && miss_page && miss_slot && miss_count, "da_pages_gather: null pointer");
  DA_REQUIRE(page_bytes % 16 == 0 && dram_head_stride_bytes % 16 == 0 &&
                 dram_page_stride_bytes % 16 == 0 && hbm_head_stride_bytes % 16 == 0 &&
                 hbm_slot_stride_bytes % 16 == 0 && (uintptr_t)dram % 16 == 0 &&
                 (uintptr_t)hbm % 16 == 0,
             "da_pages_gather: pages must be 16-byte aligned multiples of 16 bytes");
  DA_REQUIRE(n_kv_heads <= 65535, "da_pages_gather: too many heads");
  // Few, fat workgroups: ~32 blocks (16 KiB of reads in flight each) already
  // saturate the host link, and more concurrent page streams only lower it.
  int cap = (max_blocks > 0 ? max_blocks : 32) / n_kv_heads;
  if (cap < 1) cap = 1;
  const int per_head = k < cap ? k : cap;
  dim3 grid(per_head, n_kv_heads);
  hipLaunchKernelGGL(pages_gather_kernel, grid, dim3(256), 0, (hipStream_t)stream,
                     (const char *)dram, dram_head_stride_bytes, dram_page_stride_bytes,
                     (char *)hbm, hbm_head_stride_bytes, hbm_slot_stride_bytes, page_bytes,
                     miss_page, miss_slot, miss_count, k);
  return launch_status("da_pages_gather");
}
