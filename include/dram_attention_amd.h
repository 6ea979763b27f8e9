/*
 * C ABI of libdramattn.so — hand-written gfx950 (MI355X) kernels for the
 * generate-stage hot path of DRAM Attention.
 *
 * The reference (a pure-Python package) has no FFI of its own; every entry
 * point below replaces a Triton kernel, a torch op or a flash-attn call on the
 * reference's decode path and cites it.  Conventions shared by all calls:
 *
 *   - plain C types only; every pointer is BORROWED device-accessible memory
 *     (HBM, or pinned host memory mapped into the device address space);
 *   - strides are in ELEMENTS of the tensor's dtype unless the name ends in
 *     `_bytes`; the innermost (head_dim) axis is always contiguous;
 *   - work is enqueued on `stream` (a hipStream_t passed as void*, NULL = the
 *     default stream) and the call returns without synchronising;
 *   - nothing is allocated or freed; scratch memory comes in through
 *     `workspace` arguments whose size the matching *_workspace_bytes() gives;
 *   - the return value is DA_OK (0), a negative DA_E* code for a rejected
 *     argument (nothing was launched), or a positive hipError_t from the
 *     launch; da_last_error_string() describes the last failure of the
 *     calling thread.
 */
#ifndef DRAM_ATTENTION_AMD_H
#define DRAM_ATTENTION_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DA_OK 0
#define DA_EINVAL (-1)  /* malformed argument (null pointer, bad size, bad dtype) */
#define DA_ENOTSUP (-2) /* well-formed but outside what the kernels cover */

/* element types of K/V/q tensors */
#define DA_F32 0
#define DA_F16 1
#define DA_BF16 2
/* integer types of index / mapping tensors, and of page_access_time */
#define DA_I32 0
#define DA_I64 1
#define DA_TIME_F32 0
#define DA_TIME_I32 1

/* Library version: major*10000 + minor*100 + patch. */
int da_version(void);

/* Text for the last non-zero return value on this thread ("" if none). */
const char *da_last_error_string(void);

/*
 * Device-visible address of a pinned (hipHostMalloc'd) host buffer, so that
 * kernels can read pages straight out of host DRAM.  Replaces the implicit UVA
 * dereference of the pinned `dram_kv_cache` tensor inside
 * dram_attention/lru_triton_kernel.py:81-89.
 */
int da_host_device_pointer(const void *host_ptr, void **device_ptr);

/*
 * Prefill — causal attention over the whole prompt, one query row per prompt
 * token: out[t, j, :] = softmax_{s <= t}(q[t, j, :] . k[s, j / rep, :] * scale) v[s, j / rep, :].
 * Replaces flash_attn_func(xq, xk, xv, causal=True) in
 * dram_attention/dram_attention.py:136 (batch 1, as the module asserts, :128).
 *   q, out : (S, Hq, D), element strides (tok_stride, head_stride, 1)
 *   k, v   : (S, Hkv, D) likewise; query head j reads kv head j / (Hq / Hkv)
 *   scale  : softmax scale (flash-attn's default is D^-0.5), positive
 *   lse_out: optional (Hq, S) fp32, natural log of the softmax denominator
 * bf16 or fp16 with head_dim 64 or 128 (DA_ENOTSUP otherwise): tiled flash
 * attention with both products on the matrix cores, fp32 accumulation, the
 * softmax weights rounded to the input type for the second product (as
 * flash-attn rounds them).  No workspace.
 */
int da_prefill_attention(const void *q, int64_t q_tok_stride, int64_t q_head_stride,
                         const void *k, int64_t k_tok_stride, int64_t k_head_stride,
                         const void *v, int64_t v_tok_stride, int64_t v_head_stride,
                         int64_t seq_len, int n_q_heads, int n_kv_heads, int head_dim,
                         int dtype, float scale, void *out, int64_t o_tok_stride,
                         int64_t o_head_stride, float *lse_out, void *stream);

/*
 * Subsystem 1 — per-page, per-channel min and max of the keys.
 * Replaces torch.aminmax + torch.stack in
 * dram_attention/topk_selector.py:31-34.
 *   k        : (Hkv, P*page, D) keys, element strides (k_head_stride, k_tok_stride, 1)
 *   out      : (Hkv, P, 2, D) contiguous, same dtype; [...,0,:] = min, [...,1,:] = max
 * NaNs propagate as in torch.aminmax.
 */
int da_page_minmax(const void *k, int64_t k_head_stride, int64_t k_tok_stride,
                   int n_kv_heads, int64_t n_pages, int page_size, int head_dim,
                   int dtype, void *out, void *stream);

/*
 * Subsystem 1b — build the paged KV store from the prompt's keys and values.
 * Replaces the torch copies of LRUCache.__init__, dram_attention/lru_cache.py:131-141
 * (interleaved page layout in the pinned store) and :191-209 (initial slots).
 *   k, v  : (Hkv, n_pages*page_size, D) views, element strides (head_stride,
 *           tok_stride, 1)
 *   dram  : device-visible base of the (Hkv, n_pages, page_size*2*D) page store
 *           (token t of a page: K row at t*2D, V row at t*2D+D), or NULL
 *   hbm   : base of the slot array, or NULL; page p lands in slot
 *           p - first_resident_page when that is in [0, n_slots)
 * Strides of dram / hbm in bytes.  Rows must be a multiple of 16 bytes
 * (DA_ENOTSUP otherwise).
 */
int da_pages_build(const void *k, const void *v, int64_t tok_stride, int64_t head_stride,
                   int n_kv_heads, int64_t n_pages, int page_size, int head_dim, int dtype,
                   void *dram, int64_t dram_head_stride_bytes, int64_t dram_page_stride_bytes,
                   void *hbm, int64_t hbm_head_stride_bytes, int64_t hbm_slot_stride_bytes,
                   int64_t first_resident_page, int64_t n_slots, void *stream);

/*
 * Subsystem 2 — Quest upper-bound page score
 *     score[n,h,l] = sum_d max(q[n,h,d]*mm[h,l,0,d], q[n,h,d]*mm[h,l,1,d]).
 * Replaces _max_inner_product_kernel / max_inner_product in
 * dram_attention/max_ip_triton_kernel.py:20-124 (formula: max_ip_ref, :127-133).
 *   q      : (n_rows, H, D), element strides (q_row_stride, q_head_stride, 1)
 *   minmax : (H, L, 2, D), element strides (mm_head_stride, mm_page_stride, mm_r_stride, 1)
 *   out    : (n_rows, H, L) with element strides (out_row_stride, out_head_stride, 1);
 *            out_dtype is DA_F32 or equal to `dtype`.
 * Arithmetic follows the reference kernel for bf16 and fp32: for bf16 each
 * product is rounded to bf16, the maximum and the sum over D are fp32 (Triton
 * promotes bf16 operands of tl.maximum to fp32), fp32 is fp32 throughout.
 * fp16 takes the bf16 scheme (products rounded to fp16, fp32 maximum and sum,
 * one rounding at the end): a deliberate deviation.  Triton would keep fp16
 * through the maximum AND the sum, in a reduction order it picks, which no
 * restatement can reproduce; the reference only checks the dtype of that case
 * (max_ip_triton_kernel_test.py:18-26), so fp16 parity is unpinned and the
 * result here is the more accurate one.  `flags`:
 *   DA_SCORE_ROUND          : the fp32 sum is rounded to the input type before it
 *                             is stored (the value the reference ranks on, :99),
 *                             also when out_dtype is DA_F32
 *   DA_SCORE_ORDERED_BOUNDS : the caller vouches that minmax[h,l,0,d] <=
 *                             minmax[h,l,1,d] everywhere (or both NaN), as
 *                             da_page_minmax writes them.  The larger product is
 *                             then q * (q >= 0 ? max : min): same values, and
 *                             bf16 summaries with fp32 output and head_dim 32,
 *                             64 or 128 take a kernel with less than half the
 *                             vector instructions (products by packed dot
 *                             instructions, the sum over D on the matrix cores).
 *                             With bounds that are not ordered the result is
 *                             the sum of those products, not the reference's.
 */
#define DA_SCORE_ROUND 1
#define DA_SCORE_ORDERED_BOUNDS 2
int da_page_score(const void *q, int64_t q_row_stride, int64_t q_head_stride,
                  const void *minmax, int64_t mm_head_stride, int64_t mm_page_stride,
                  int64_t mm_r_stride, int n_rows, int n_heads, int64_t n_pages,
                  int head_dim, int dtype, void *out, int64_t out_row_stride,
                  int64_t out_head_stride, int out_dtype, int flags, void *stream);

/*
 * Subsystem 3 — ordered top-k page selection per score row.
 * Replaces torch.argsort(ip, descending=True)[..., :k] in
 * dram_attention/topk_selector.py:61 and the layout shuffle in
 * dram_attention/lru_cache.py:263-264.
 *   scores : fp32, row (n, h) starts at n*row_stride + h*head_stride, n_pages long
 *   out    : the kp page indices of row (n, h), best first, written at
 *            (n / rep)*out_seq_stride + h*out_head_stride + (n % rep)*out_rep_stride
 * Order: descending score; equal scores by ascending page index (a stable
 * descending sort).  -0.0 equals +0.0; NaN ranks above +inf (torch's order).
 * workspace: da_topk_pages_workspace_bytes(...) bytes (0 for rows of up to 16384
 * pages), no initial state needed.  Longer rows are cut into parts that one
 * workgroup each reduces to kp candidates, and a second launch selects among the
 * candidates (same result, ties included); without a workspace of that size
 * (NULL is allowed) one workgroup per row walks the whole row instead.
 */
size_t da_topk_pages_workspace_bytes(int n_rows, int n_heads, int64_t n_pages, int kp);
int da_topk_pages(const float *scores, int64_t row_stride, int64_t head_stride,
                  int n_rows, int rep, int n_heads, int64_t n_pages, int kp,
                  void *out, int64_t out_seq_stride, int64_t out_head_stride,
                  int64_t out_rep_stride, int out_itype, void *workspace,
                  size_t workspace_bytes, void *stream);

/*
 * da_topk_pages, and in the same launch (one more workgroup per head) the list of
 * the k_cand least recently used slots of every head, in eviction order, for the
 * da_lru_update that follows (see its `candidates`).  The order of the slots
 * does not depend on this step's scores, so it is computed next to the top-k
 * instead of inside the LRU update, which every later launch of the step waits
 * for.  Needs n_heads == Hkv; k_cand <= min(N_hbm, 8192); candidates == NULL or
 * k_cand == 0 gives plain da_topk_pages.  n_rows == 0 or kp == 0 with a list
 * requested computes the list only.
 *   candidates : n_heads * k_cand + n_heads int32: the lists, (n_heads, k_cand),
 *                followed by one stamp word per head
 *   step       : the LRU step counter da_lru_update will be given (required with
 *                a list); its value at the time of this launch is stored as the
 *                stamp of every head's list
 */
int da_topk_pages_lru(const float *scores, int64_t row_stride, int64_t head_stride,
                      int n_rows, int rep, int n_heads, int64_t n_pages, int kp,
                      void *out, int64_t out_seq_stride, int64_t out_head_stride,
                      int64_t out_rep_stride, int out_itype, const void *access_time,
                      int64_t time_head_stride, int time_type, int n_hbm_pages, int k_cand,
                      int32_t *candidates, const int32_t *step, void *workspace,
                      size_t workspace_bytes, void *stream);

/*
 * Subsystem 4a — LRU lookup / touch / evict / slot-assign for one decode step.
 * Replaces _update_page_access_time_, torch.argsort(page_access_time,
 * stable=True) and the metadata half of _load_lru_cache_inline_kernel in
 * dram_attention/lru_triton_kernel.py:6-194 (and current_step.add_(1),
 * dram_attention/lru_cache.py:224, when DA_LRU_BUMP_STEP is set in `flags`).
 *   idx          : (Hkv, K) requested DRAM pages in visiting order (itype idx_itype)
 *   step         : one int32; with DA_LRU_BUMP_STEP the kernel uses *step+1 and stores it
 *   access_time  : (Hkv, N_hbm) last-use step per slot (fp32 or int32)
 *   d2h          : (Hkv, P) slot of each DRAM page or -1;  h2d : (Hkv, N_hbm) page per slot
 *                  (both of itype map_itype); updated in place
 *   hit_mask     : optional (Hkv, K) bytes, 1 = page was resident when visited
 *   miss_page/miss_slot : (Hkv, K) int32, the i-th distinct missed page of a
 *                  head and the slot it was given; miss_count : (Hkv) int32
 *   candidates   : optional, as da_topk_pages_lru writes it (Hkv lists of k_cand
 *                  int32, then Hkv stamp words): the k_cand least recently used
 *                  slots of every head in eviction order.  The kernel then finds
 *                  its victims by dropping the slots this call touches from that
 *                  list instead of ordering all slots again (it orders them itself
 *                  whenever the list is too short).  A list is only used when its
 *                  stamp equals *step as this call reads it and DA_LRU_BUMP_STEP is
 *                  set: every bumping update changes the access times and the
 *                  counter together, so a list made before an earlier update (a
 *                  stale list) is recognised and ignored, with the same result as
 *                  passing none; so is any list handed to a call that does not
 *                  bump.  Entries that are no slot number are ignored.
 *                  NULL / k_cand = 0: no list.
 *   slot_epoch   : optional (Hkv, N_hbm) int32; a slot handed to a missed page
 *                  gets the step value, so a later kernel can tell which slots
 *                  the page stream of this step is (still) writing
 * The end state equals the reference's serial walk for every input; K <=
 * N_hbm with DA_LRU_BUMP_STEP runs fully parallel, K > N_hbm falls back to one
 * serial lane per head.  Without DA_LRU_BUMP_STEP the time stamp is the
 * caller's *step and may tie with stored access times, where only the literal
 * walk is right: such calls take it too.  The walk orders at most 8192 slots
 * per head: a call that needs it with more slots is refused (DA_ENOTSUP).
 * DA_LRU_SERIAL_WALK in `flags` takes that literal walk for any K (a checking
 * and benchmarking aid: the result is the same, only slower).
 * A miss_slot of -1 marks an entry whose slot was re-assigned later in the
 * same call (possible only when K > N_hbm); da_pages_gather skips it.
 * workspace: da_lru_update_workspace_bytes(...) bytes, ZEROED ONCE by the
 * caller before the first call and left alone afterwards.
 */
#define DA_LRU_BUMP_STEP 1
#define DA_LRU_SERIAL_WALK 2

size_t da_lru_update_workspace_bytes(int n_kv_heads, int k, int64_t n_dram_pages,
                                     int n_hbm_pages);
int da_lru_update(const void *idx, int64_t idx_head_stride, int idx_itype,
                  int n_kv_heads, int k, int64_t n_dram_pages, int n_hbm_pages,
                  int32_t *step, int flags, void *access_time,
                  int64_t time_head_stride, int time_type, void *d2h,
                  int64_t d2h_head_stride, void *h2d, int64_t h2d_head_stride,
                  int map_itype, uint8_t *hit_mask, int32_t *miss_page,
                  int32_t *miss_slot, int32_t *miss_count, int32_t *slot_epoch,
                  const int32_t *candidates, int k_cand, void *workspace,
                  size_t workspace_bytes, void *stream);

/*
 * Subsystem 4b — stream the missed pages into their HBM slots.
 * Replaces the page copy loop of _load_lru_cache_inline_kernel,
 * dram_attention/lru_triton_kernel.py:80-98 (8 serial programs reading host
 * memory) by a grid-wide gather: every wave copies 16-byte lanes of one page.
 *   dram : device-visible base of the (Hkv, P, page_bytes) page store
 *   hbm  : base of the (Hkv, N_hbm, page_bytes) slot array
 * Entry i < miss_count[h] of head h copies page miss_page[h,i] to slot
 * miss_slot[h,i]; page_bytes must be a multiple of 16.  max_blocks bounds the
 * number of workgroups (0 = the default, 32: a few fat workgroups saturate the
 * host link, more concurrent page streams only lower its throughput).
 */
int da_pages_gather(const void *dram, int64_t dram_head_stride_bytes,
                    int64_t dram_page_stride_bytes, void *hbm,
                    int64_t hbm_head_stride_bytes, int64_t hbm_slot_stride_bytes,
                    int64_t page_bytes, const int32_t *miss_page,
                    const int32_t *miss_slot, const int32_t *miss_count,
                    int n_kv_heads, int k, int max_blocks, void *stream);

/*
 * Subsystem 5 — split-K decode attention for ONE query token over
 *   [prefix segment] ++ [local segment (c_len rows)] ++ [the new token],
 * with the new key/value appended in place at row c_len of the local cache and
 * all partial results merged through their log-sum-exp.  Replaces both
 * flash_attn_with_kvcache calls and _combine_attention in
 * dram_attention/dram_attention.py:191-238.
 *   q            : (Hq, D), head stride q_head_stride; q head j uses kv head j / (Hq/Hkv)
 *   pk, pv       : prefix keys / values, (Hkv, p_len, D) with element strides
 *                  (p_head_stride, p_tok_stride, 1); p_len may be 0
 *   ck, cv       : local cache, (capacity, Hkv, D) addressed with (c_tok_stride, c_head_stride, 1)
 *   c_len        : rows already valid in the local cache; if c_len_dev is not
 *                  NULL the count is *c_len_dev + c_len (a device position
 *                  counter plus a host offset, which may be negative)
 *   new_k, new_v : (Hkv, D) of the current token (head stride new_head_stride),
 *                  or NULL to attend over the c_len cached rows only
 *   out          : (Hq, D) in `dtype`;  lse_out : optional (Hq) fp32, natural log
 * fp32 accumulation throughout.  bf16/fp16 inputs with head_dim 64, 128 or 256
 * and at most 16 query heads per kv head run both products on the matrix
 * cores (the softmax weights are rounded to the input type for the second
 * product, as flash-attn rounds them); other shapes use packed dot
 * instructions on the vector units.
 * workspace: da_decode_attention_workspace_bytes(...) bytes, 16-byte aligned, no
 * initial state; `miss_tokens` is 0 here (see da_decode_attention_paged).
 */
size_t da_decode_attention_workspace_bytes(int n_q_heads, int n_kv_heads, int head_dim,
                                           int dtype, int64_t p_len, int64_t c_capacity,
                                           int64_t miss_tokens);
int da_decode_attention(const void *q, int64_t q_head_stride, int n_q_heads,
                        int n_kv_heads, int head_dim, int dtype, const void *pk,
                        const void *pv, int64_t p_tok_stride, int64_t p_head_stride,
                        int64_t p_len, void *ck, void *cv, int64_t c_tok_stride,
                        int64_t c_head_stride, int64_t c_capacity, int64_t c_len,
                        const int32_t *c_len_dev, const void *new_k, const void *new_v,
                        int64_t new_head_stride, float scale, void *out,
                        int64_t out_head_stride, float *lse_out, void *workspace,
                        size_t workspace_bytes, void *stream);

/*
 * da_decode_attention for callers that cannot allocate device memory or bring a
 * workspace: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  It has no counterpart in the reference.  Same arguments
 * and results as da_decode_attention, minus the workspace: the partial results
 * of the split pass live in a device array built into the library,
 * DA_STATIC_SCRATCH_BYTES per GPU for the life of the process
 * (da_decode_attention_static_capacity() returns the figure).  The call makes
 * no hipMalloc / hipFree.  Shapes whose partial results exceed the array
 * (da_decode_attention_workspace_bytes(..., miss_tokens = 0) > capacity) are
 * refused with DA_ENOTSUP and nothing is launched.  All calls on one GPU share
 * that GPU's array: calls that overlap in time on one GPU (two streams, two
 * threads) race; calls that follow each other on one stream do not, and no
 * state is carried from one call to the next.
 */
#define DA_STATIC_SCRATCH_BYTES (8u << 20)
size_t da_decode_attention_static_capacity(void);
int da_decode_attention_static(const void *q, int64_t q_head_stride, int n_q_heads,
                               int n_kv_heads, int head_dim, int dtype, const void *pk,
                               const void *pv, int64_t p_tok_stride, int64_t p_head_stride,
                               int64_t p_len, void *ck, void *cv, int64_t c_tok_stride,
                               int64_t c_head_stride, int64_t c_capacity, int64_t c_len,
                               const int32_t *c_len_dev, const void *new_k, const void *new_v,
                               int64_t new_head_stride, float scale, void *out,
                               int64_t out_head_stride, float *lse_out, void *stream);

/*
 * The same attention when the prefix is the slot array of the LRU page cache
 * and the missed pages of this step are streamed in concurrently on another
 * stream (no counterpart in the reference, whose page copies and attention are
 * serialised on one stream, dram_attention/dram_attention.py:161-172).
 * `phase` is a set of DA_PHASE_* bits, carried out in this order:
 *   DA_PHASE_FIRST       : local segment + every slot whose slot_epoch differs
 *                          from *epoch; may run while da_pages_gather is still
 *                          writing the other slots
 *   DA_PHASE_FIRST_MERGE : merges the partial results of DA_PHASE_FIRST into one
 *                          partial kept in the workspace, and into `out` (the
 *                          result without the slots the second pass covers);
 *                          may also run next to the page stream
 *   DA_PHASE_SECOND      : the slots listed in miss_slot[h, 0..miss_count[h])
 *                          (entries of -1 are skipped), then the merge that
 *                          writes the complete `out` and `lse_out`; issue it
 *                          after the page stream has completed.  Without
 *                          DA_PHASE_FIRST in the same call it merges the tail with
 *                          the partial DA_PHASE_FIRST_MERGE left in the workspace.
 * When the page stream of the step was da_pages_gather_attend, which attends
 * over the re-assigned slots itself, set `gather_blocks` to its
 * blocks_per_head: DA_PHASE_SECOND is then only the final merge.
 *   DA_PHASE_STREAM      : together with DA_PHASE_FIRST: the page stream itself
 *                          (the work of da_pages_gather_attend, with
 *                          `gather_blocks` workgroups per kv head) runs inside
 *                          the launch of the first pass, no second stream
 *                          needed.  STREAM | FIRST | SECOND is a whole step in
 *                          two launches.  Same shape limits as
 *                          da_pages_gather_attend (DA_ENOTSUP otherwise).
 *   DA_PHASE_MERGE_ALL   : together with DA_PHASE_SECOND in a call of its own, after
 *                          a call with DA_PHASE_FIRST (and STREAM) but no
 *                          FIRST_MERGE: there is no carried partial, the final
 *                          merge takes every chunk.  Lets a caller issue the
 *                          merge apart from the first pass (on another stream,
 *                          so that the next layer's page stream need not wait
 *                          for it) at the cost of no extra launch.
 * With two streams: FIRST | FIRST_MERGE next to the page stream, SECOND after the join.
 * FIRST | SECOND in one call (the page stream already complete) needs no
 * FIRST_MERGE.
 * The calls of a step must be given identical arguments otherwise.  The
 * workspace needs miss_tokens = miss_capacity * page_size.
 */
#define DA_PHASE_FIRST 1
#define DA_PHASE_SECOND 2
#define DA_PHASE_FIRST_MERGE 4
#define DA_PHASE_STREAM 8
#define DA_PHASE_MERGE_ALL 16

typedef struct da_paged_overlap {
  int32_t page_size;              /* tokens per slot; p_len = slots * page_size */
  int32_t phase;                  /* DA_PHASE_* bits */
  const int32_t *slot_epoch;      /* (Hkv, slots), written by da_lru_update */
  int64_t slot_epoch_head_stride; /* elements */
  const int32_t *epoch;           /* the LRU step counter after da_lru_update */
  const int32_t *miss_slot;       /* (Hkv, miss_capacity) */
  const int32_t *miss_count;      /* (Hkv) */
  int32_t miss_capacity;
  int32_t gather_blocks;          /* blocks_per_head of da_pages_gather_attend, else 0 */
  /* DA_PHASE_STREAM only: the operands of the page stream, as da_pages_gather_attend takes them */
  const void *dram;
  int64_t dram_head_stride_bytes, dram_page_stride_bytes;
  void *hbm;
  int64_t hbm_head_stride_bytes, hbm_slot_stride_bytes;
  const int32_t *miss_page;       /* (Hkv, miss_capacity) */
  /* DA_PHASE_STREAM only: two rates of the machine, in GB/s, from which the launch
   * decides whether the page stream of a step is long enough to leave the first
   * pass to a few workgroups per kv head (which then keep off the compute units
   * the stream runs on).  link_gbps: what reads of the pinned store issued by a
   * kernel reach over the host link; block_gbps: what one workgroup alone on its
   * compute unit reads from HBM.  0 = the values of the box the library was tuned
   * on (54 and 30).  They move time only: the results do not depend on them. */
  float link_gbps, block_gbps;
} da_paged_overlap;

int da_decode_attention_paged(const void *q, int64_t q_head_stride, int n_q_heads,
                              int n_kv_heads, int head_dim, int dtype, const void *pk,
                              const void *pv, int64_t p_tok_stride, int64_t p_head_stride,
                              int64_t p_len, void *ck, void *cv, int64_t c_tok_stride,
                              int64_t c_head_stride, int64_t c_capacity, int64_t c_len,
                              const int32_t *c_len_dev, const void *new_k, const void *new_v,
                              int64_t new_head_stride, float scale, void *out,
                              int64_t out_head_stride, float *lse_out, void *workspace,
                              size_t workspace_bytes, const da_paged_overlap *overlap,
                              void *stream);

/*
 * Subsystem 4b + 5 — the page stream with this step's attention riding on it
 * (no counterpart in the reference, which copies pages first and attends
 * afterwards, dram_attention/lru_triton_kernel.py:80-98 then
 * dram_attention/dram_attention.py:191-238).  Copies exactly what
 * da_pages_gather copies; the registers a page passes through also feed the
 * attention of query `q` over that page, so that the step needs no second pass
 * over the re-assigned slots once the stream has finished.
 *   page layout : page_size tokens, each token its K row (head_dim) followed by
 *                 its V row; dram / hbm strides in bytes as for da_pages_gather
 *   q           : (Hq, head_dim), element stride q_head_stride
 *   workspace   : the workspace of this step's da_decode_attention_paged calls
 *                 (same p_len, c_capacity, and miss_capacity = k); every block
 *                 with an entry to copy leaves one partial result in it
 *   blocks_per_head : workgroups per kv head; blocks_per_head * Hkv <= 64 (few
 *                 fat ones: 32 in all saturate the host link).  The blocks
 *                 share the miss lists of all heads in equal parts, whatever
 *                 each head's count.  Pass the same value as
 *                 da_paged_overlap.gather_blocks to DA_PHASE_SECOND
 * DA_ENOTSUP when rows are not 64..512 bytes, Hq / Hkv > 8 or a page exceeds
 * 16 KiB (and Hkv > 64 leaves no valid blocks_per_head): use da_pages_gather and the tail pass of DA_PHASE_SECOND then.
 */
int da_pages_gather_attend(const void *dram, int64_t dram_head_stride_bytes,
                           int64_t dram_page_stride_bytes, void *hbm,
                           int64_t hbm_head_stride_bytes, int64_t hbm_slot_stride_bytes,
                           int page_size, const int32_t *miss_page, const int32_t *miss_slot,
                           const int32_t *miss_count, int n_kv_heads, int k,
                           int blocks_per_head, const void *q, int64_t q_head_stride,
                           int n_q_heads, int head_dim, int dtype, float scale, int64_t p_len,
                           int64_t c_capacity, void *workspace, size_t workspace_bytes,
                           void *stream);

#ifdef __cplusplus
}
#endif
#endif /* DRAM_ATTENTION_AMD_H */
