// Per-page, per-channel min/max of the keys (the Quest page summaries).
// Counterpart of torch.aminmax + torch.stack in
// dram_attention/topk_selector.py:31-34 of the reference.
//
// Bound: HBM.  Algorithmic bytes = Hkv*P*page*D*e read + Hkv*P*2*D*e written.
// One lane owns a 16-byte column chunk of one (page, head) and walks the
// page's rows; adjacent lanes own adjacent chunks, heads vary next, so a wave
// reads whole contiguous rows when the keys are laid out (token, head, dim).
#include "common.hpp"

namespace da {

// min/max that let NaN win, as torch.aminmax does.
__device__ __forceinline__ float nan_min(float m, float x) { return (x < m || x != x) ? x : m; }
__device__ __forceinline__ float nan_max(float m, float x) { return (x > m || x != x) ? x : m; }

template <typename T>
__device__ __forceinline__ u32x4 repack(const float *f);
template <>
__device__ __forceinline__ u32x4 repack<F32>(const float *f) {
  u32x4 v;
#pragma unroll
  for (int i = 0; i < 4; ++i) v[i] = __builtin_bit_cast(uint32_t, f[i]);
  return v;
}
template <>
__device__ __forceinline__ u32x4 repack<F16>(const float *f) {
  u32x4 v;
#pragma unroll
  for (int i = 0; i < 4; ++i) v[i] = pack_f16(f[2 * i], f[2 * i + 1]);
  return v;
}
template <>
__device__ __forceinline__ u32x4 repack<BF16>(const float *f) {
  u32x4 v;
#pragma unroll
  for (int i = 0; i < 4; ++i) v[i] = pack_bf16(f[2 * i], f[2 * i + 1]);
  return v;
}

// Vector path: head_dim is a multiple of the 16-byte lane width and every
// stride keeps 16-byte alignment.
template <typename T>
__global__ void __launch_bounds__(256)
page_minmax_vec_kernel(const char *__restrict__ k, int64_t head_stride, int64_t tok_stride,
                       int n_heads, int64_t n_pages, int page, int chunks_per_row,
                       char *__restrict__ out) {
  constexpr int V = T::kVec;
  const int64_t items = n_pages * n_heads * chunks_per_row;
  for (int64_t it = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; it < items;
       it += (int64_t)gridDim.x * blockDim.x) {
    const int c = (int)(it % chunks_per_row);
    const int64_t ph = it / chunks_per_row;
    const int h = (int)(ph % n_heads);
    const int64_t p = ph / n_heads;
    const char *src =
        k + (h * head_stride + p * page * tok_stride + (int64_t)c * V) * T::kBytes;
    float mn[V], mx[V], f[V];
    unpack<T>(load16(src), mn);
#pragma unroll
    for (int i = 0; i < V; ++i) mx[i] = mn[i];
    for (int t = 1; t < page; ++t) {
      unpack<T>(load16(src + (int64_t)t * tok_stride * T::kBytes), f);
#pragma unroll
      for (int i = 0; i < V; ++i) {
        mn[i] = nan_min(mn[i], f[i]);
        mx[i] = nan_max(mx[i], f[i]);
      }
    }
    const int64_t d = (int64_t)chunks_per_row * V;
    char *dst = out + (((int64_t)h * n_pages + p) * 2 * d + (int64_t)c * V) * T::kBytes;
    store16(dst, repack<T>(mn));
    store16(dst + d * T::kBytes, repack<T>(mx));
  }
}

// Scalar path for any head_dim / alignment.
template <typename T>
__global__ void __launch_bounds__(256)
page_minmax_scalar_kernel(const void *__restrict__ k, int64_t head_stride, int64_t tok_stride,
                          int n_heads, int64_t n_pages, int page, int head_dim,
                          void *__restrict__ out) {
  const int64_t items = n_pages * n_heads * head_dim;
  for (int64_t it = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; it < items;
       it += (int64_t)gridDim.x * blockDim.x) {
    const int d = (int)(it % head_dim);
    const int64_t ph = it / head_dim;
    const int h = (int)(ph % n_heads);
    const int64_t p = ph / n_heads;
    const int64_t base = h * head_stride + p * page * tok_stride + d;
    float mn = load_elem<T>(k, base), mx = mn;
    for (int t = 1; t < page; ++t) {
      const float x = load_elem<T>(k, base + (int64_t)t * tok_stride);
      mn = nan_min(mn, x);
      mx = nan_max(mx, x);
    }
    const int64_t o = (((int64_t)h * n_pages + p) * 2) * head_dim + d;
    store_elem<T>(out, o, mn);
    store_elem<T>(out, o + head_dim, mx);
  }
}

template <typename T>
static int launch_page_minmax(const void *k, int64_t head_stride, int64_t tok_stride, int n_heads,
                              int64_t n_pages, int page, int head_dim, void *out,
                              hipStream_t stream) {
  constexpr int V = T::kVec;
  const bool vec = head_dim % V == 0 && head_stride % V == 0 && tok_stride % V == 0 &&
                   ((uintptr_t)k % 16) == 0 && ((uintptr_t)out % 16) == 0;
  if (vec) {
    const int chunks = head_dim / V;
    const int64_t items = n_pages * n_heads * chunks;
    const int blocks = (int)(ceil_div(items, 256) < 65536 ? ceil_div(items, 256) : 65536);
    hipLaunchKernelGGL(page_minmax_vec_kernel<T>, dim3(blocks), dim3(256), 0, stream,
                       (const char *)k, head_stride, tok_stride, n_heads, n_pages, page, chunks,
                       (char *)out);
  } else {
    const int64_t items = n_pages * n_heads * head_dim;
    const int blocks = (int)(ceil_div(items, 256) < 65536 ? ceil_div(items, 256) : 65536);
    hipLaunchKernelGGL(page_minmax_scalar_kernel<T>, dim3(blocks), dim3(256), 0, stream, k,
                       head_stride, tok_stride, n_heads, n_pages, page, head_dim, out);
  }
  return launch_status("da_page_minmax");
}

}  // namespace da

extern "C" int da_page_minmax(const void *k, int64_t k_head_stride, int64_t k_tok_stride,
                              int n_kv_heads, int64_t n_pages, int page_size, int head_dim,
                              int dtype, void *out, void *stream) {
  using namespace da;
  DA_REQUIRE(n_kv_heads >= 0 && n_pages >= 0 && page_size > 0 && head_dim > 0,
             "da_page_minmax: bad geometry (heads %d pages %lld page %d dim %d)", n_kv_heads,
             (long long)n_pages, page_size, head_dim);
  if (n_kv_heads == 0 || n_pages == 0) return DA_OK;
  DA_REQUIRE(k && out, "da_page_minmax: null pointer");
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case DA_F32:
      return launch_page_minmax<F32>(k, k_head_stride, k_tok_stride, n_kv_heads, n_pages,
                                     page_size, head_dim, out, s);
    case DA_F16:
      return launch_page_minmax<F16>(k, k_head_stride, k_tok_stride, n_kv_heads, n_pages,
                                     page_size, head_dim, out, s);
    case DA_BF16:
      return launch_page_minmax<BF16>(k, k_head_stride, k_tok_stride, n_kv_heads, n_pages,
                                      page_size, head_dim, out, s);
  }
  return fail(DA_EINVAL, "da_page_minmax: unknown dtype %d", dtype);
}
