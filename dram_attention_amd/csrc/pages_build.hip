// Builds the paged KV store of the LRU cache from the prompt's keys and values:
// one pass that writes every page in the interleaved layout (token t of a page:
// K row at t*2D, V row at t*2D+D) into the host page store, through its
// device-visible address, and the pages that start out resident into their HBM
// slots.  Counterpart of the torch copies in LRUCache.__init__ of the reference,
// dram_attention/lru_cache.py:131-141 (page layout, pinned store) and :191-209
// (initial slots: the last N_hbm pages in slots 0..N_hbm-1).
//
// Bound: host link (every byte of K and V crosses it once, as posted writes);
// algorithmic bytes = 2*S*Hkv*D*e read from HBM, the same written to the host,
// N_hbm*page_bytes*Hkv written to HBM.
#include "common.hpp"

namespace da {

__global__ void __launch_bounds__(256)
pages_build_kernel(const char *__restrict__ k, const char *__restrict__ v, int64_t tok_stride_b,
                   int64_t head_stride_b, int64_t n_pages, int page_size, int lanes,
                   char *__restrict__ dram, int64_t dram_head_stride, int64_t dram_page_stride,
                   char *__restrict__ hbm, int64_t hbm_head_stride, int64_t hbm_slot_stride,
                   int64_t first_resident, int64_t n_slots) {
  const int h = blockIdx.y;
  const int tok_lanes = 2 * lanes;             // 16-byte lanes per token (K row, V row)
  const int page_vecs = page_size * tok_lanes;
  for (int64_t p = blockIdx.x; p < n_pages; p += gridDim.x) {
    char *dst = dram ? dram + h * dram_head_stride + p * dram_page_stride : nullptr;
    const int64_t slot = p - first_resident;
    char *dst2 = (hbm && slot >= 0 && slot < n_slots)
                     ? hbm + h * hbm_head_stride + slot * hbm_slot_stride
                     : nullptr;
    for (int j0 = threadIdx.x; j0 < page_vecs; j0 += 4 * 256) {
      u32x4 r[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int j = j0 + u * 256;
        if (j < page_vecs) {
          const int tok = j / tok_lanes, within = j % tok_lanes;
          const char *src = (within >= lanes ? v : k) + h * head_stride_b +
                            (p * page_size + tok) * tok_stride_b + (within % lanes) * 16;
          r[u] = load16(src);
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int j = j0 + u * 256;
        if (j < page_vecs) {
          if (dst) store16(dst + (int64_t)j * 16, r[u]);
          if (dst2) store16(dst2 + (int64_t)j * 16, r[u]);
        }
      }
    }
  }
}

}  // namespace da

extern "C" int da_pages_build(const void *k, const void *v, int64_t tok_stride, int64_t head_stride,
                              int n_kv_heads, int64_t n_pages, int page_size, int head_dim,
                              int dtype, void *dram, int64_t dram_head_stride_bytes,
                              int64_t dram_page_stride_bytes, void *hbm,
                              int64_t hbm_head_stride_bytes, int64_t hbm_slot_stride_bytes,
                              int64_t first_resident_page, int64_t n_slots, void *stream) {
  using namespace da;
  DA_REQUIRE(n_kv_heads >= 0 && n_pages >= 0 && page_size > 0 && head_dim > 0 && n_slots >= 0,
             "da_pages_build: bad geometry");
  DA_REQUIRE(dtype == DA_F32 || dtype == DA_F16 || dtype == DA_BF16,
             "da_pages_build: unknown dtype %d", dtype);
  if (n_kv_heads == 0 || n_pages == 0) return DA_OK;
  DA_REQUIRE(k && v && (dram || hbm), "da_pages_build: null pointer");
  const int e = elem_size(dtype);
  const int64_t row_bytes = (int64_t)head_dim * e;
  if (row_bytes % 16 != 0 || n_kv_heads > 65535)
    return fail(DA_ENOTSUP, "da_pages_build: rows of %lld bytes (need a multiple of 16)",
                (long long)row_bytes);
  DA_REQUIRE((tok_stride * e) % 16 == 0 && (head_stride * e) % 16 == 0 &&
                 (uintptr_t)k % 16 == 0 && (uintptr_t)v % 16 == 0 && (uintptr_t)dram % 16 == 0 &&
                 (uintptr_t)hbm % 16 == 0 && dram_head_stride_bytes % 16 == 0 &&
                 dram_page_stride_bytes % 16 == 0 && hbm_head_stride_bytes % 16 == 0 &&
                 hbm_slot_stride_bytes % 16 == 0,
             "da_pages_build: operands must be 16-byte aligned");
  const int lanes = (int)(row_bytes / 16);
  DA_REQUIRE((int64_t)page_size * 2 * lanes <= 0x7fffffff, "da_pages_build: page too large");
  const int64_t blocks = n_pages < 2048 ? n_pages : 2048;
  dim3 grid((unsigned)blocks, n_kv_heads);
  hipLaunchKernelGGL(pages_build_kernel, grid, dim3(256), 0, (hipStream_t)stream, (const char *)k,
                     (const char *)v, tok_stride * e, head_stride * e, n_pages, page_size, lanes,
                     (char *)dram, dram_head_stride_bytes, dram_page_stride_bytes, (char *)hbm,
                     hbm_head_stride_bytes, hbm_slot_stride_bytes, first_resident_page, n_slots);
  return launch_status("da_pages_build");
}
