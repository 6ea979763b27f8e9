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
  int32_t *out;  // (Hkv, k_cand)
};

template <typename TimeT>
__device__ __forceinline__ void lru_candidates_block(const LruCandidateArgs &c, int h,
                                                     SelectShared &sm) {
  LeastRecentKey<TimeT> key{(const TimeT *)c.access_time + h * c.time_head_stride};
  const uint32_t *order = select_sorted(key, c.n_slots, c.k_cand, sm);
  int32_t *dst = c.out + (int64_t)h * c.k_cand;
  for (int j = threadIdx.x; j < c.k_cand; j += kSelThreads) dst[j] = (int32_t)order[j];
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
  const uint32_t *best = select_sorted(key, n_pages, kp, sm);
  IdxT *dst = out + (n / rep) * out_seq_stride + h * out_head_stride + (n % rep) * out_rep_stride;
  for (int j = threadIdx.x; j < kp; j += kSelThreads) dst[j] = (IdxT)best[j];
}

}  // namespace da

extern "C" size_t da_topk_pages_workspace_bytes(int, int, int64_t, int) { return 0; }

extern "C" int da_topk_pages_lru(const float *scores, int64_t row_stride, int64_t head_stride,
                                 int n_rows, int rep, int n_heads, int64_t n_pages, int kp,
                                 void *out, int64_t out_seq_stride, int64_t out_head_stride,
                                 int64_t out_rep_stride, int out_itype, const void *access_time,
                                 int64_t time_head_stride, int time_type, int n_hbm_pages,
                                 int k_cand, int32_t *candidates, void *stream) {
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
  dim3 grid(rows + (with_cand ? 1 : 0), n_heads);
  hipStream_t s = (hipStream_t)stream;
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
  (void)workspace;
  (void)workspace_bytes;
  return da_topk_pages_lru(scores, row_stride, head_stride, n_rows, rep, n_heads, n_pages, kp, out,
                           out_seq_stride, out_head_stride, out_rep_stride, out_itype, nullptr, 0,
                           DA_TIME_F32, 0, 0, nullptr, stream);
}
