// Ordered top-k page selection, one 1024-thread workgroup per score row.
// Counterpart of torch.argsort(ip, descending=True)[..., :k] in
// dram_attention/topk_selector.py:61 of the reference, with the tie order the
// reference leaves open fixed to "lowest page index first" (a stable sort).
//
// Bound: latency (a row is a few tens of KiB and stays in L2); algorithmic
// bytes = rows*P*4 read + rows*kp*8 written.
#include "lru_keys.hpp"

namespace da {

struct ScoreKey {
  const float *row;
  bool aligned;  // row starts on a 16-byte boundary
  __device__ __forceinline__ uint32_t operator()(int i) const { return float_order_key(row[i]); }
  __device__ __forceinline__ void load4(int i, uint32_t *k) const {
    float4 v;
    if (aligned) {
      v = *(const float4 *)(row + i);
    } else {
      v = make_float4(row[i], row[i + 1], row[i + 2], row[i + 3]);
    }
    k[0] = float_order_key(v.x);
    k[1] = float_order_key(v.y);
    k[2] = float_order_key(v.z);
    k[3] = float_order_key(v.w);
  }
};

// The k_cand least recently used slots of kv head h, in eviction order, into
// out[h, 0..k_cand).  Independent of this step's scores, so it rides along with
// the top-k launch (one more workgroup per head) and the LRU update that follows
// only has to drop the slots it touched from this list.
struct LruCandidateArgs {
  const void *access_time;  // (Hkv, n_slots), fp32 or int32; null: no candidates
  int64_t time_head_stride;
  int time_is_i32;
  int n_slots, k_cand;
  int32_t *out;  // (Hkv, k_cand) lists, then Hkv stamp words
  const int32_t *step;  // the LRU step counter: its value now is the list's stamp
  int n_heads;
};

template <typename TimeT>
__device__ __forceinline__ void lru_candidates_block(const LruCandidateArgs &c, int h,
                                                     SelectShared &sm) {
  LeastRecentKey<TimeT> key{(const TimeT *)c.access_time + h * c.time_head_stride};
  int32_t *dst = c.out + (int64_t)h * c.k_cand;
  // The stamp says which state of the access times the list describes: the update
  // that consumes the list compares it with the step it reads.
  if (threadIdx.x == 0) c.out[(int64_t)c.n_heads * c.k_cand + h] = *c.step;
  select_sorted(key, c.n_slots, c.k_cand, sm,
                direct([=](uint32_t rank, uint32_t slot) { dst[rank] = (int32_t)slot; }));
}

template <typename IdxT>
__global__ void __launch_bounds__(kSelThreads)
topk_pages_kernel(const float *__restrict__ scores, int64_t row_stride, int64_t head_stride,
                  int n_rows, int rep, int n_pages, int kp, IdxT *__restrict__ out,
                  int64_t out_seq_stride, int64_t out_head_stride, int64_t out_rep_stride,
                  const LruCandidateArgs cand) {
  __shared__ SelectShared sm;
  const int n = blockIdx.x;  // score row (query row); row n_rows: the LRU candidates of head h
  const int h = blockIdx.y;
  if (n >= n_rows) {
    if (cand.time_is_i32)
      lru_candidates_block<int32_t>(cand, h, sm);
    else
      lru_candidates_block<float>(cand, h, sm);
    return;
  }
  const float *row = scores + n * row_stride + h * head_stride;
  ScoreKey key{row, ((uintptr_t)row & 15) == 0};
  IdxT *dst = out + (n / rep) * out_seq_stride + h * out_head_stride + (n % rep) * out_rep_stride;
  select_sorted(key, n_pages, kp, sm,
                direct([=](uint32_t rank, uint32_t page) { dst[rank] = (IdxT)page; }));
}

// Long rows in two launches.  A single workgroup keeps 16384 keys in registers
// and has to read a longer row again in every pass; cut into parts of at most
// that many pages, each part goes to a workgroup of its own (more of the part
// busy, nothing read twice), which leaves its kp best as candidates, and a second
// launch picks the row's kp best among the candidates of its parts.  The k
// largest of a union lie in the union of the k largest of its pieces, and the
// candidates are laid out part after part, each sorted by (score descending, page
// ascending): among equal scores the position in that layout rises with the page
// number, so the second selection breaks ties exactly as one pass over the
// whole row would.
struct SplitPlan {
  int n_parts;   // 1: no split
  int part_len;  // pages per part (a multiple of 4, so 16-byte loads stay aligned)
  int64_t row_words() const { return (int64_t)n_parts * kp; }
  int kp;
};
inline SplitPlan plan_split(int64_t n_pages, int kp) {
  SplitPlan p{1, (int)n_pages, kp};
  const int reg_keys = kSelRegKeys * kSelThreads;
  if (n_pages <= reg_keys || kp <= 0) return p;
  int parts = (int)((n_pages + reg_keys - 1) / reg_keys);
  if (parts > 16) parts = 16;
  int len = (int)(((n_pages + parts - 1) / parts + 3) & ~(int64_t)3);
  // every part must hold kp pages, the last one included, for the fixed layout
  while (parts > 1 && (len < kp || n_pages - (int64_t)(parts - 1) * len < kp)) {
    --parts;
    len = (int)(((n_pages + parts - 1) / parts + 3) & ~(int64_t)3);
  }
  if (parts > 1 && (int64_t)(parts - 1) * len >= n_pages) return p;  // rounding emptied the last part
  p.n_parts = parts;
  p.part_len = len;
  return p;
}

__global__ void __launch_bounds__(kSelThreads)
topk_parts_kernel(const float *__restrict__ scores, int64_t row_stride, int64_t head_stride,
                  int n_rows, int n_pages, int kp, int n_parts, int part_len,
                  uint32_t *__restrict__ cand_key, uint32_t *__restrict__ cand_page) {
  __shared__ SelectShared sm;
  const int h = blockIdx.y;
  const int n = blockIdx.x / n_parts, part = blockIdx.x % n_parts;
  const int first = part * part_len;
  const int len = n_pages - first < part_len ? n_pages - first : part_len;
  const float *row = scores + n * row_stride + h * head_stride + first;
  ScoreKey key{row, ((uintptr_t)row & 15) == 0};
  const int64_t base = (((int64_t)n * gridDim.y + h) * n_parts + part) * kp;
  select_sorted(key, len, kp, sm, direct([=](uint32_t rank, uint32_t i) {
                  cand_key[base + rank] = key(i);
                  cand_page[base + rank] = (uint32_t)first + i;
                }));
}

struct CandidateKey {
  const uint32_t *row;
  bool aligned;
  __device__ __forceinline__ uint32_t operator()(int i) const { return row[i]; }
  __device__ __forceinline__ void load4(int i, uint32_t *k) const {
    if (aligned) {
      const uint4 v = *(const uint4 *)(row + i);
      k[0] = v.x;
      k[1] = v.y;
      k[2] = v.z;
      k[3] = v.w;
    } else {
      k[0] = row[i];
      k[1] = row[i + 1];
      k[2] = row[i + 2];
      k[3] = row[i + 3];
    }
  }
};

template <typename IdxT>
__global__ void __launch_bounds__(kSelThreads)
topk_merge_kernel(const uint32_t *__restrict__ cand_key, const uint32_t *__restrict__ cand_page,
                  int n_rows, int rep, int kp, int n_parts, IdxT *__restrict__ out,
                  int64_t out_seq_stride, int64_t out_head_stride, int64_t out_rep_stride,
                  const LruCandidateArgs cand) {
  __shared__ SelectShared sm;
  const int n = blockIdx.x, h = blockIdx.y;
  if (n >= n_rows) {
    // The LRU candidates ride in this launch, the one with few workgroups: the
    // parts of the 1M shape fill the device exactly (64 rows x 4 parts on 256
    // compute units, one workgroup each), and eight more would run as a second round.
    if (cand.time_is_i32)
      lru_candidates_block<int32_t>(cand, h, sm);
    else
      lru_candidates_block<float>(cand, h, sm);
    return;
  }
  const int64_t base = ((int64_t)n * gridDim.y + h) * n_parts * kp;
  CandidateKey key{cand_key + base, (((uintptr_t)(cand_key + base)) & 15) == 0};
  IdxT *dst = out + (n / rep) * out_seq_stride + h * out_head_stride + (n % rep) * out_rep_stride;
  select_sorted(key, n_parts * kp, kp, sm, direct([=](uint32_t rank, uint32_t i) {
                  dst[rank] = (IdxT)cand_page[base + i];
                }));
}

}  // namespace da

extern "C" size_t da_topk_pages_workspace_bytes(int n_rows, int n_heads, int64_t n_pages, int kp) {
  if (n_rows <= 0 || n_heads <= 0 || n_pages <= 0 || kp <= 0 || kp > n_pages) return 0;
  const da::SplitPlan p = da::plan_split(n_pages, kp);
  if (p.n_parts == 1) return 0;
  return (size_t)n_rows * n_heads * p.row_words() * 2 * sizeof(uint32_t);
}

extern "C" int da_topk_pages_lru(const float *scores, int64_t row_stride, int64_t head_stride,
                                 int n_rows, int rep, int n_heads, int64_t n_pages, int kp,
                                 void *out, int64_t out_seq_stride, int64_t out_head_stride,
                                 int64_t out_rep_stride, int out_itype, const void *access_time,
                                 int64_t time_head_stride, int time_type, int n_hbm_pages,
                                 int k_cand, int32_t *candidates, const int32_t *step,
                                 void *workspace, size_t workspace_bytes, void *stream) {
  using namespace da;
  DA_REQUIRE(n_rows >= 0 && n_heads >= 0 && n_pages >= 0 && kp >= 0 && rep >= 1,
             "da_topk_pages: bad geometry (rows %d heads %d pages %lld kp %d rep %d)", n_rows,
             n_heads, (long long)n_pages, kp, rep);
  DA_REQUIRE(kp <= n_pages, "da_topk_pages: kp %d exceeds the %lld pages of a row", kp,
             (long long)n_pages);
  DA_REQUIRE(out_itype == DA_I32 || out_itype == DA_I64, "da_topk_pages: bad index type %d",
             out_itype);
  LruCandidateArgs cand = {};
  if (candidates != nullptr && k_cand > 0) {
    DA_REQUIRE(access_time && n_hbm_pages > 0 && k_cand <= n_hbm_pages && k_cand <= kSelMaxK,
               "da_topk_pages_lru: %d candidates of %d slots (at most %d)", k_cand, n_hbm_pages,
               kSelMaxK);
    DA_REQUIRE(time_type == DA_TIME_F32 || time_type == DA_TIME_I32,
               "da_topk_pages_lru: bad access-time type");
    DA_REQUIRE(step != nullptr, "da_topk_pages_lru: a candidate list needs the step counter");
    cand.step = step;
    cand.n_heads = n_heads;
    cand.access_time = access_time;
    cand.time_head_stride = time_head_stride;
    cand.time_is_i32 = time_type == DA_TIME_I32;
    cand.n_slots = n_hbm_pages;
    cand.k_cand = k_cand;
    cand.out = candidates;
  }
  const bool with_cand = cand.out != nullptr;
  const bool with_topk = n_rows > 0 && kp > 0;
  if (n_heads == 0 || (!with_topk && !with_cand)) return DA_OK;
  DA_REQUIRE(!with_topk || (scores && out), "da_topk_pages: null pointer");
  if (kp > kSelMaxK)
    return fail(DA_ENOTSUP, "da_topk_pages: kp %d above the %d survivors sorted in LDS", kp,
                kSelMaxK);
  if (n_pages > 0x7fffffff || n_heads > 65535)
    return fail(DA_ENOTSUP, "da_topk_pages: row length or head count out of range");
  const int rows = with_topk ? n_rows : 0;
  hipStream_t s = (hipStream_t)stream;
  const SplitPlan plan = with_topk ? plan_split(n_pages, kp) : SplitPlan{1, 0, kp};
  const size_t split_bytes = (size_t)rows * n_heads * plan.row_words() * 2 * sizeof(uint32_t);
  if (plan.n_parts > 1 && workspace != nullptr && workspace_bytes >= split_bytes &&
      (int64_t)rows * plan.n_parts < 0x7fffffff) {
    uint32_t *cand_key = (uint32_t *)workspace;
    uint32_t *cand_page = cand_key + (size_t)rows * n_heads * plan.row_words();
    dim3 grid1(rows * plan.n_parts, n_heads), grid2(rows + (with_cand ? 1 : 0), n_heads);
    hipLaunchKernelGGL(topk_parts_kernel, grid1, dim3(kSelThreads), 0, s, scores, row_stride,
                       head_stride, rows, (int)n_pages, kp, plan.n_parts, plan.part_len, cand_key,
                       cand_page);
    if (out_itype == DA_I64)
      hipLaunchKernelGGL(topk_merge_kernel<int64_t>, grid2, dim3(kSelThreads), 0, s, cand_key,
                         cand_page, rows, rep, kp, plan.n_parts, (int64_t *)out, out_seq_stride,
                         out_head_stride, out_rep_stride, cand);
    else
      hipLaunchKernelGGL(topk_merge_kernel<int32_t>, grid2, dim3(kSelThreads), 0, s, cand_key,
                         cand_page, rows, rep, kp, plan.n_parts, (int32_t *)out, out_seq_stride,
                         out_head_stride, out_rep_stride, cand);
    return launch_status("da_topk_pages");
  }
  dim3 grid(rows + (with_cand ? 1 : 0), n_heads);
  if (out_itype == DA_I64)
    hipLaunchKernelGGL(topk_pages_kernel<int64_t>, grid, dim3(kSelThreads), 0, s, scores,
                       row_stride, head_stride, rows, rep, (int)n_pages, kp, (int64_t *)out,
                       out_seq_stride, out_head_stride, out_rep_stride, cand);
  else
    hipLaunchKernelGGL(topk_pages_kernel<int32_t>, grid, dim3(kSelThreads), 0, s, scores,
                       row_stride, head_stride, rows, rep, (int)n_pages, kp, (int32_t *)out,
                       out_seq_stride, out_head_stride, out_rep_stride, cand);
  return launch_status("da_topk_pages");
}

extern "C" int da_topk_pages(const float *scores, int64_t row_stride, int64_t head_stride,
                             int n_rows, int rep, int n_heads, int64_t n_pages, int kp, void *out,
                             int64_t out_seq_stride, int64_t out_head_stride,
                             int64_t out_rep_stride, int out_itype, void *workspace,
                             size_t workspace_bytes, void *stream) {
  return da_topk_pages_lru(scores, row_stride, head_stride, n_rows, rep, n_heads, n_pages, kp, out,
                           out_seq_stride, out_head_stride, out_rep_stride, out_itype, nullptr, 0,
                           DA_TIME_F32, 0, 0, nullptr, nullptr, workspace, workspace_bytes, stream);
}
