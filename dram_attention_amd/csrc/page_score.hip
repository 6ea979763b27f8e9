// Quest upper-bound page scorer:
//   score[n,h,l] = sum_d max(q[n,h,d]*min[h,l,d], q[n,h,d]*max[h,l,d]).
// Counterpart of _max_inner_product_kernel in
// dram_attention/max_ip_triton_kernel.py:20-92 of the reference.
//
// Bound: HBM.  Algorithmic bytes = H*L*2*D*e (the page summaries, read once
// and shared by every query row of the head) + n*H*L*4 written.
//
// Vector path: a page's min row and max row are D*e bytes each; kLanes =
// D*e/16 adjacent lanes cover one row with 16-byte loads, so a 64-lane wave
// scores 64/kLanes pages per step from fully used cache lines.  Each lane
// keeps its slice of up to kRows query rows in registers, accumulates in fp32
// and the kLanes partial sums are folded with wavefront shuffles.
#include <type_traits>

#include "common.hpp"
#include "page_score_tile.hpp"

namespace da {

// For 16-bit inputs the reference multiplies in the input type (each product
// rounded) and promotes to fp32 for max and sum.  Rounding to nearest is
// monotonic, so max(rnd(a), rnd(b)) == rnd(max(a, b)): one rounding per pair.
template <typename T>
__device__ __forceinline__ float bound_term(float q, float mn, float mx) {
  return round_to<T>(fmaxf(q * mn, q * mx));
}

// Sum of the V bound terms of one 16-byte lane slice.  For 16-bit inputs two
// maxima are rounded by one packed convert and added to the fp32 accumulator
// by a dot product with (1, 1): rounding and accumulation in two instructions.
template <typename T>
__device__ __forceinline__ float slice_bound(const float *q, const float *mn, const float *mx);
template <>
__device__ __forceinline__ float slice_bound<F32>(const float *q, const float *mn,
                                                  const float *mx) {
  float a = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) a += fmaxf(q[i] * mn[i], q[i] * mx[i]);
  return a;
}
template <>
__device__ __forceinline__ float slice_bound<BF16>(const float *q, const float *mn,
                                                   const float *mx) {
  const bf16x2 ones = as_bf16x2(0x3f803f80u);
  float a = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i += 2) {
    const uint32_t pair = pack_bf16(fmaxf(q[i] * mn[i], q[i] * mx[i]),
                                    fmaxf(q[i + 1] * mn[i + 1], q[i + 1] * mx[i + 1]));
    a = __builtin_amdgcn_fdot2_f32_bf16(as_bf16x2(pair), ones, a, false);
  }
  return a;
}
template <>
__device__ __forceinline__ float slice_bound<F16>(const float *q, const float *mn,
                                                  const float *mx) {
  const f16x2 ones = as_f16x2(0x3c003c00u);
  float a = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i += 2) {
    const uint32_t pair = pack_f16(fmaxf(q[i] * mn[i], q[i] * mx[i]),
                                   fmaxf(q[i + 1] * mn[i + 1], q[i + 1] * mx[i + 1]));
    a = __builtin_amdgcn_fdot2(as_f16x2(pair), ones, a, false);
  }
  return a;
}

template <typename T, int kLanes, int kRows, int kUnroll, typename OutT>
__global__ void __launch_bounds__(256)
page_score_vec_kernel(const char *__restrict__ q, int64_t q_row_stride, int64_t q_head_stride,
                      const char *__restrict__ mm, int n_rows, int64_t n_pages,
                      OutT *__restrict__ out, int64_t out_row_stride, int64_t out_head_stride,
                      int round_out, int rounds) {
  constexpr int V = T::kVec;
  constexpr int kGroups = 64 / kLanes;  // pages per wave step
  constexpr int kRowBytes = kLanes * 16;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int c = lane % kLanes;
  const int g = lane / kLanes;
  const int h = blockIdx.y;
  const int row0 = blockIdx.z * kRows;

  float qf[kRows][V];
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const int n = row0 + r < n_rows ? row0 + r : n_rows - 1;
    unpack<T>(load16(q + (n * q_row_stride + h * q_head_stride + (int64_t)c * V) * T::kBytes),
              qf[r]);
  }

  const int64_t pages_per_round = (int64_t)(blockDim.x >> 6) * kGroups * kUnroll;
  const char *head_base = mm + (int64_t)h * n_pages * 2 * kRowBytes;

  for (int round = 0; round < rounds; ++round) {
  const int64_t p_first = ((int64_t)blockIdx.x * rounds + round) * pages_per_round +
                          (int64_t)wave * kGroups * kUnroll;
  if (p_first - (int64_t)wave * kGroups * kUnroll >= n_pages) break;
  u32x4 vmin[kUnroll], vmax[kUnroll];
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    int64_t p = p_first + u * kGroups + g;
    if (p >= n_pages) p = n_pages - 1;  // clamp: result discarded below
    const char *src = head_base + p * 2 * kRowBytes + c * 16;
    vmin[u] = load16(src);
    vmax[u] = load16(src + kRowBytes);
  }
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    float fmin_[V], fmax_[V];
    unpack<T>(vmin[u], fmin_);
    unpack<T>(vmax[u], fmax_);
    float acc[kRows];
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      acc[r] = group_sum<kLanes>(slice_bound<T>(qf[r], fmin_, fmax_));
    }
    const int64_t p = p_first + u * kGroups + g;
    if (p < n_pages) {
      // lane c of a group stores row c (rows beyond kLanes fall to lane 0)
#pragma unroll
      for (int r = 0; r < kRows; ++r) {
        const bool mine = (kLanes >= kRows) ? (c == r) : (c == 0);
        if (mine && row0 + r < n_rows) {
          float v = acc[r];
          if (round_out) v = round_to<T>(v);
          out[(row0 + r) * out_row_stride + h * out_head_stride + p] = (OutT)v;
        }
      }
    }
  }
  }  // rounds
}

// Generic path: any head_dim, any strides.  One wave per page, lanes stride
// over the channels, one query row at a time.
template <typename T, typename OutT>
__global__ void __launch_bounds__(256)
page_score_generic_kernel(const void *__restrict__ q, int64_t q_row_stride,
                          int64_t q_head_stride, const void *__restrict__ mm,
                          int64_t mm_head_stride, int64_t mm_page_stride, int64_t mm_r_stride,
                          int n_rows, int64_t n_pages, int head_dim, OutT *__restrict__ out,
                          int64_t out_row_stride, int64_t out_head_stride, int round_out) {
  const int lane = threadIdx.x & 63;
  const int64_t p = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int h = blockIdx.y;
  if (p >= n_pages) return;
  const int64_t base = h * mm_head_stride + p * mm_page_stride;
  for (int n = 0; n < n_rows; ++n) {
    float a = 0.f;
    for (int d = lane; d < head_dim; d += 64) {
      const float qv = load_elem<T>(q, n * q_row_stride + h * q_head_stride + d);
      a += bound_term<T>(qv, load_elem<T>(mm, base + d), load_elem<T>(mm, base + mm_r_stride + d));
    }
    a = group_sum<64>(a);
    if (lane == 0) {
      if (round_out) a = round_to<T>(a);
      out[n * out_row_stride + h * out_head_stride + p] = (OutT)a;
    }
  }
}

template <typename T, int kLanes, typename OutT>
static void launch_vec(const void *q, int64_t qrs, int64_t qhs, const void *mm, int n_rows,
                       int n_heads, int64_t n_pages, OutT *out, int64_t ors, int64_t ohs,
                       int round_out, hipStream_t s) {
  constexpr int kGroups = 64 / kLanes;
  // rounds of pages per block: one, i.e. as many blocks as the row allows (several
  // rounds per block, amortising the query load, measured no faster)
  const int rounds = 1;
  if (n_rows <= 4) {
    constexpr int kRows = 4, kUnroll = 2;
    dim3 grid((unsigned)ceil_div(n_pages, 4 * kGroups * kUnroll * rounds), n_heads, 1);
    hipLaunchKernelGGL((page_score_vec_kernel<T, kLanes, kRows, kUnroll, OutT>), grid, dim3(256),
                       0, s, (const char *)q, qrs, qhs, (const char *)mm, n_rows, n_pages, out,
                       ors, ohs, round_out, rounds);
  } else {
    constexpr int kRows = 8, kUnroll = 2;
    dim3 grid((unsigned)ceil_div(n_pages, 4 * kGroups * kUnroll * rounds), n_heads,
              (unsigned)ceil_div(n_rows, kRows));
    hipLaunchKernelGGL((page_score_vec_kernel<T, kLanes, kRows, kUnroll, OutT>), grid, dim3(256),
                       0, s, (const char *)q, qrs, qhs, (const char *)mm, n_rows, n_pages, out,
                       ors, ohs, round_out, rounds);
  }
}

template <typename T, typename OutT>
static int launch_page_score(const void *q, int64_t qrs, int64_t qhs, const void *mm,
                             int64_t mhs, int64_t mps, int64_t mrs, int n_rows, int n_heads,
                             int64_t n_pages, int head_dim, OutT *out, int64_t ors, int64_t ohs,
                             int round_out, bool ordered, hipStream_t s) {
  constexpr int V = T::kVec;
  const int lanes = head_dim % V == 0 ? head_dim / V : 0;
  const bool vec = lanes >= 1 && lanes <= 64 && is_pow2(lanes) && mrs == head_dim &&
                   mps == 2 * (int64_t)head_dim && mhs == n_pages * 2 * head_dim &&
                   qrs % V == 0 && qhs % V == 0 && ((uintptr_t)q % 16) == 0 &&
                   ((uintptr_t)mm % 16) == 0 && n_heads <= 65535 && n_rows <= 8 * 65535;
  if constexpr (std::is_same<T, BF16>::value && std::is_same<OutT, float>::value) {
    // bf16 summaries with ordered bounds, fp32 scores: the decode step's form
    if (vec && ordered && n_rows <= 8 * 65535 &&
        page_score_tile_supported(head_dim, n_pages, ors, ohs, out, q, mm, qrs, qhs)) {
      const bool wide = n_rows > 4;
      switch (head_dim) {
        case 32:
          if (wide) launch_page_score_tile<1, 8>(q, qrs, qhs, mm, n_rows, n_heads, n_pages, out, ors, ohs, round_out, s);
          else launch_page_score_tile<1, 4>(q, qrs, qhs, mm, n_rows, n_heads, n_pages, out, ors, ohs, round_out, s);
          break;
        case 64:
          if (wide) launch_page_score_tile<2, 8>(q, qrs, qhs, mm, n_rows, n_heads, n_pages, out, ors, ohs, round_out, s);
          else launch_page_score_tile<2, 4>(q, qrs, qhs, mm, n_rows, n_heads, n_pages, out, ors, ohs, round_out, s);
          break;
        default:
          if (wide) launch_page_score_tile<4, 8>(q, qrs, qhs, mm, n_rows, n_heads, n_pages, out, ors, ohs, round_out, s);
          else launch_page_score_tile<4, 4>(q, qrs, qhs, mm, n_rows, n_heads, n_pages, out, ors, ohs, round_out, s);
      }
      return launch_status("da_page_score");
    }
  }
  if (vec) {
#define DA_SCORE_CASE(L)                                                                     \
  case L:                                                                                    \
    launch_vec<T, L, OutT>(q, qrs, qhs, mm, n_rows, n_heads, n_pages, out, ors, ohs,         \
                           round_out, s);                                                    \
    break;
    switch (lanes) {
      DA_SCORE_CASE(1)
      DA_SCORE_CASE(2)
      DA_SCORE_CASE(4)
      DA_SCORE_CASE(8)
      DA_SCORE_CASE(16)
      DA_SCORE_CASE(32)
      DA_SCORE_CASE(64)
    }
#undef DA_SCORE_CASE
  } else {
    if (n_heads > 65535) return fail(DA_ENOTSUP, "da_page_score: more than 65535 heads");
    dim3 grid((unsigned)ceil_div(n_pages, 4), n_heads, 1);
    hipLaunchKernelGGL((page_score_generic_kernel<T, OutT>), grid, dim3(256), 0, s, q, qrs, qhs,
                       mm, mhs, mps, mrs, n_rows, n_pages, head_dim, out, ors, ohs, round_out);
  }
  return launch_status("da_page_score");
}

template <typename T>
struct Storage;
template <>
struct Storage<F32> { typedef float type; };
template <>
struct Storage<F16> { typedef _Float16 type; };
template <>
struct Storage<BF16> { typedef __bf16 type; };

template <typename T>
static int dispatch_out(const void *q, int64_t qrs, int64_t qhs, const void *mm, int64_t mhs,
                        int64_t mps, int64_t mrs, int n_rows, int n_heads, int64_t n_pages,
                        int head_dim, void *out, int64_t ors, int64_t ohs, bool out_f32,
                        int round_out, bool ordered, hipStream_t s) {
  if (out_f32)
    return launch_page_score<T, float>(q, qrs, qhs, mm, mhs, mps, mrs, n_rows, n_heads, n_pages,
                                       head_dim, (float *)out, ors, ohs, round_out, ordered, s);
  typedef typename Storage<T>::type O;
  return launch_page_score<T, O>(q, qrs, qhs, mm, mhs, mps, mrs, n_rows, n_heads, n_pages,
                                 head_dim, (O *)out, ors, ohs, round_out, ordered, s);
}

}  // namespace da

extern "C" int da_page_score(const void *q, int64_t q_row_stride, int64_t q_head_stride,
                             const void *minmax, int64_t mm_head_stride, int64_t mm_page_stride,
                             int64_t mm_r_stride, int n_rows, int n_heads, int64_t n_pages,
                             int head_dim, int dtype, void *out, int64_t out_row_stride,
                             int64_t out_head_stride, int out_dtype, int flags, void *stream) {
  using namespace da;
  DA_REQUIRE(n_rows >= 0 && n_heads >= 0 && n_pages >= 0 && head_dim > 0,
             "da_page_score: bad geometry (rows %d heads %d pages %lld dim %d)", n_rows, n_heads,
             (long long)n_pages, head_dim);
  DA_REQUIRE(dtype == DA_F32 || dtype == DA_F16 || dtype == DA_BF16,
             "da_page_score: unknown dtype %d", dtype);
  DA_REQUIRE(out_dtype == DA_F32 || out_dtype == dtype,
             "da_page_score: out_dtype must be fp32 or the input dtype");
  if (n_rows == 0 || n_heads == 0 || n_pages == 0) return DA_OK;
  DA_REQUIRE(q && minmax && out, "da_page_score: null pointer");
  DA_REQUIRE((flags & ~(DA_SCORE_ROUND | DA_SCORE_ORDERED_BOUNDS)) == 0,
             "da_page_score: unknown flag bits %d", flags);
  hipStream_t s = (hipStream_t)stream;
  const bool out_f32 = out_dtype == DA_F32;
  const int round_to_input = flags & DA_SCORE_ROUND;
  const bool ordered = (flags & DA_SCORE_ORDERED_BOUNDS) != 0;
  switch (dtype) {
    case DA_F32:
      return dispatch_out<F32>(q, q_row_stride, q_head_stride, minmax, mm_head_stride,
                               mm_page_stride, mm_r_stride, n_rows, n_heads, n_pages, head_dim,
                               out, out_row_stride, out_head_stride, true, 0, ordered, s);
    case DA_F16:
      return dispatch_out<F16>(q, q_row_stride, q_head_stride, minmax, mm_head_stride,
                               mm_page_stride, mm_r_stride, n_rows, n_heads, n_pages, head_dim,
                               out, out_row_stride, out_head_stride, out_f32, round_to_input, ordered, s);
    default:
      return dispatch_out<BF16>(q, q_row_stride, q_head_stride, minmax, mm_head_stride,
                                mm_page_stride, mm_r_stride, n_rows, n_heads, n_pages, head_dim,
                                out, out_row_stride, out_head_stride, out_f32, round_to_input, ordered, s);
  }
}
