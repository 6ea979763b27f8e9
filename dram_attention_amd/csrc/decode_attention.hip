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
#include "common.hpp"

namespace da {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kMinusHuge = -1.0e30f;  // finite stand-in for -inf as a running max
constexpr int kAttnThreads = 256;
constexpr int kAttnWaves = kAttnThreads / 64;
constexpr int kAttnUnroll = 4;

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// 16 bytes of q against 16 bytes of k, fp32 accumulate.
template <typename T>
__device__ __forceinline__ float dot16(const u32x4 &q, const u32x4 &k);
template <>
__device__ __forceinline__ float dot16<F32>(const u32x4 &q, const u32x4 &k) {
  float a = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
    a = fmaf(as_f32(q[i]), as_f32(k[i]), a);
  return a;
}
template <>
__device__ __forceinline__ float dot16<BF16>(const u32x4 &q, const u32x4 &k) {
  float a = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
    a = __builtin_amdgcn_fdot2_f32_bf16(as_bf16x2(q[i]), as_bf16x2(k[i]), a, false);
  return a;
}
template <>
__device__ __forceinline__ float dot16<F16>(const u32x4 &q, const u32x4 &k) {
  float a = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
    a = __builtin_amdgcn_fdot2(as_f16x2(q[i]), as_f16x2(k[i]), a, false);
  return a;
}

struct AttnArgs {
  const char *q;
  int64_t q_head_stride;  // elements
  int rep;                // query heads per kv head
  const char *pk, *pv;    // prefix segment
  int64_t p_tok_stride, p_head_stride, p_len;
  char *ck, *cv;  // local cache
  int64_t c_tok_stride, c_head_stride, c_capacity, c_len;
  const int32_t *c_len_dev;
  const char *new_k, *new_v;
  int64_t new_head_stride;
  float scale_log2;  // softmax scale * log2(e)
  int chunk;         // tokens per block
  int n_pchunks;     // chunks of the prefix segment (the rest belong to the local segment)
  int n_chunks;      // grid.x
  int n_q_heads;
  float *part_ml;   // (n_chunks, Hq, 2): running max (log2 domain), sum
  float *part_acc;  // (n_chunks, Hq, D)
};

template <typename T, int kLanes, int kRows>
__global__ void __launch_bounds__(kAttnThreads)
decode_attention_split_kernel(const AttnArgs a) {
  constexpr int V = T::kVec;
  constexpr int kGroups = 64 / kLanes;  // tokens per wave step
  constexpr int kStepTokens = kAttnWaves * kGroups;
  constexpr int D = kLanes * V;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int c = lane % kLanes;
  const int g = lane / kLanes;
  const int h = blockIdx.y;
  const int row0 = blockIdx.z * kRows;  // first query row of the GQA group handled here
  const int chunk_id = blockIdx.x;

  // Which segment, which token range.
  const bool local = chunk_id >= a.n_pchunks;
  int64_t c_len = a.c_len;
  if (a.c_len_dev) c_len = *a.c_len_dev;
  if (c_len < 0) c_len = 0;
  const bool has_new = a.new_k != nullptr && c_len < a.c_capacity;
  if (c_len > a.c_capacity) c_len = a.c_capacity;
  const int64_t seg_len = local ? c_len + (has_new ? 1 : 0) : a.p_len;
  const int64_t t_begin = (int64_t)(local ? chunk_id - a.n_pchunks : chunk_id) * a.chunk;
  if (t_begin >= seg_len) return;  // the merge kernel skips this chunk as well
  const int64_t t_end = t_begin + a.chunk < seg_len ? t_begin + a.chunk : seg_len;

  const char *kbase, *vbase;
  int64_t tok_stride_b;
  if (local) {
    kbase = a.ck + h * a.c_head_stride * T::kBytes + c * 16;
    vbase = a.cv + h * a.c_head_stride * T::kBytes + c * 16;
    tok_stride_b = a.c_tok_stride * T::kBytes;
  } else {
    kbase = a.pk + h * a.p_head_stride * T::kBytes + c * 16;
    vbase = a.pv + h * a.p_head_stride * T::kBytes + c * 16;
    tok_stride_b = a.p_tok_stride * T::kBytes;
  }
  const char *newk = nullptr, *newv = nullptr;
  if (local && has_new) {
    newk = a.new_k + h * a.new_head_stride * T::kBytes + c * 16;
    newv = a.new_v + h * a.new_head_stride * T::kBytes + c * 16;
  }

  u32x4 qv[kRows];
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const int rr = row0 + r < a.rep ? row0 + r : a.rep - 1;
    qv[r] = load16(a.q + ((int64_t)(h * a.rep + rr) * a.q_head_stride) * T::kBytes + c * 16);
  }

  float m[kRows], l[kRows], acc[kRows][V];
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    m[r] = kMinusHuge;
    l[r] = 0.f;
#pragma unroll
    for (int i = 0; i < V; ++i) acc[r][i] = 0.f;
  }

  const int64_t my_off = wave * kGroups + g;
  for (int64_t base = t_begin; base < t_end; base += (int64_t)kStepTokens * kAttnUnroll) {
    // `base` is the same for the whole block, so the wave-wide vote below sees
    // every lane; lanes past the chunk end compute on a clamped row, masked.
    const int64_t t0 = base + my_off;
    u32x4 kk[kAttnUnroll], vv[kAttnUnroll];
    bool valid[kAttnUnroll];
#pragma unroll
    for (int u = 0; u < kAttnUnroll; ++u) {
      const int64_t tok = t0 + (int64_t)u * kStepTokens;
      valid[u] = tok < t_end;
      const int64_t tk = valid[u] ? tok : t_begin;  // clamp the address, mask the score
      const bool is_new = newk != nullptr && tk == c_len;
      const char *kp = is_new ? newk : kbase + tk * tok_stride_b;
      const char *vp = is_new ? newv : vbase + tk * tok_stride_b;
      kk[u] = load16(kp);
      vv[u] = load16(vp);
      if (is_new && valid[u] && blockIdx.z == 0) {
        // the append: this lane group owns the new token's row
        store16(a.ck + (h * a.c_head_stride + c_len * a.c_tok_stride) * T::kBytes + c * 16, kk[u]);
        store16(a.cv + (h * a.c_head_stride + c_len * a.c_tok_stride) * T::kBytes + c * 16, vv[u]);
      }
    }
#pragma unroll
    for (int u = 0; u < kAttnUnroll; ++u) {
      float s[kRows];
      bool grow = false;
#pragma unroll
      for (int r = 0; r < kRows; ++r) {
        s[r] = group_sum<kLanes>(dot16<T>(qv[r], kk[u])) * a.scale_log2;
        if (!valid[u]) s[r] = -INFINITY;
        grow |= s[r] > m[r];
      }
      if (__any(grow)) {  // rare after the first few tokens: rescale lazily
#pragma unroll
        for (int r = 0; r < kRows; ++r) {
          const float mn = fmaxf(m[r], s[r]);
          const float alpha = fast_exp2(m[r] - mn);
          m[r] = mn;
          l[r] *= alpha;
#pragma unroll
          for (int i = 0; i < V; ++i) acc[r][i] *= alpha;
        }
      }
      float vf[V];
      unpack<T>(vv[u], vf);
#pragma unroll
      for (int r = 0; r < kRows; ++r) {
        const float p = fast_exp2(s[r] - m[r]);
        l[r] += p;
#pragma unroll
        for (int i = 0; i < V; ++i) acc[r][i] = fmaf(p, vf[i], acc[r][i]);
      }
    }
  }

  // Merge the lane groups of the wave (butterfly over the group index).
#pragma unroll
  for (int off = kLanes; off < 64; off <<= 1) {
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      const float mo = __shfl_xor(m[r], off, 64);
      const float lo = __shfl_xor(l[r], off, 64);
      const float mn = fmaxf(m[r], mo);
      const float wa = fast_exp2(m[r] - mn), wb = fast_exp2(mo - mn);
      l[r] = l[r] * wa + lo * wb;
#pragma unroll
      for (int i = 0; i < V; ++i) {
        const float ao = __shfl_xor(acc[r][i], off, 64);
        acc[r][i] = acc[r][i] * wa + ao * wb;
      }
      m[r] = mn;
    }
  }

  // Merge the waves through LDS; wave w's state sits in sm_*[w].
  __shared__ float sm_m[kAttnWaves][kRows];
  __shared__ float sm_l[kAttnWaves][kRows];
  __shared__ float sm_acc[kAttnWaves][kRows][D];
  if (g == 0) {
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      if (c == 0) {
        sm_m[wave][r] = m[r];
        sm_l[wave][r] = l[r];
      }
#pragma unroll
      for (int i = 0; i < V; ++i) sm_acc[wave][r][c * V + i] = acc[r][i];
    }
  }
  __syncthreads();
  for (int item = threadIdx.x; item < kRows * D; item += kAttnThreads) {
    const int r = item / D, d = item % D;
    if (row0 + r >= a.rep) continue;
    float mn = sm_m[0][r];
#pragma unroll
    for (int w = 1; w < kAttnWaves; ++w) mn = fmaxf(mn, sm_m[w][r]);
    float lt = 0.f, at = 0.f;
#pragma unroll
    for (int w = 0; w < kAttnWaves; ++w) {
      const float wgt = fast_exp2(sm_m[w][r] - mn);
      lt += sm_l[w][r] * wgt;
      at += sm_acc[w][r][d] * wgt;
    }
    const int64_t hq = (int64_t)h * a.rep + row0 + r;
    const int64_t slot = (int64_t)chunk_id * a.n_q_heads + hq;
    a.part_acc[slot * D + d] = at;
    if (d == 0) {
      a.part_ml[slot * 2] = mn;
      a.part_ml[slot * 2 + 1] = lt;
    }
  }
}

// Merge the partials of one query head.  One 256-thread block per head; a
// thread owns four adjacent output channels of every (256 / (D/4))-th chunk,
// so the chunk rows are read as 16-byte lanes and the chunk loop is short.
template <typename T>
__global__ void __launch_bounds__(256)
decode_attention_merge_kernel(const AttnArgs a, int head_dim, char *__restrict__ out,
                              int64_t out_head_stride, float *__restrict__ lse_out) {
  const int hq = blockIdx.x;
  const int t = threadIdx.x;
  int64_t c_len = a.c_len;
  if (a.c_len_dev) c_len = *a.c_len_dev;
  if (c_len < 0) c_len = 0;
  const bool has_new = a.new_k != nullptr && c_len < a.c_capacity;
  if (c_len > a.c_capacity) c_len = a.c_capacity;
  const int64_t l_len = c_len + (has_new ? 1 : 0);
  const int n_p = (int)((a.p_len + a.chunk - 1) / a.chunk);  // live prefix chunks
  const int n_l = (int)((l_len + a.chunk - 1) / a.chunk);    // live local chunks
  const int n_live = n_p + n_l;

  __shared__ float sm_red[256];
  __shared__ float sm_acc[256 * 4];
  // pass 1: global max over the live chunks
  float mx = kMinusHuge;
  for (int i = t; i < n_live; i += 256) {
    const int ch = i < n_p ? i : a.n_pchunks + (i - n_p);
    mx = fmaxf(mx, a.part_ml[((int64_t)ch * a.n_q_heads + hq) * 2]);
  }
  sm_red[t] = mx;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if (t < s) sm_red[t] = fmaxf(sm_red[t], sm_red[t + s]);
    __syncthreads();
  }
  mx = sm_red[0];
  __syncthreads();
  // pass 2: the softmax denominator
  float lt = 0.f;
  for (int i = t; i < n_live; i += 256) {
    const int ch = i < n_p ? i : a.n_pchunks + (i - n_p);
    const float *ml = a.part_ml + ((int64_t)ch * a.n_q_heads + hq) * 2;
    lt += ml[1] * fast_exp2(ml[0] - mx);
  }
  sm_red[t] = lt;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if (t < s) sm_red[t] += sm_red[t + s];
    __syncthreads();
  }
  lt = sm_red[0];
  const float inv = lt > 0.f ? 1.f / lt : 0.f;
  // pass 3: weighted sum of the partial output rows
  const int quads = head_dim / 4;        // 16-byte lanes per row (head_dim % 4 == 0 here)
  const int lanes_c = 256 / quads;       // chunk lanes
  const int qd = t % quads, cl = t / quads;
  float at[4] = {0.f, 0.f, 0.f, 0.f};
  if (cl < lanes_c) {
    for (int i = cl; i < n_live; i += lanes_c) {
      const int ch = i < n_p ? i : a.n_pchunks + (i - n_p);
      const int64_t slot = (int64_t)ch * a.n_q_heads + hq;
      const float w = fast_exp2(a.part_ml[slot * 2] - mx);
      const float4 v = *(const float4 *)(a.part_acc + slot * head_dim + qd * 4);
      at[0] = fmaf(v.x, w, at[0]);
      at[1] = fmaf(v.y, w, at[1]);
      at[2] = fmaf(v.z, w, at[2]);
      at[3] = fmaf(v.w, w, at[3]);
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) sm_acc[t * 4 + i] = at[i];
  __syncthreads();
  for (int d = t; d < head_dim; d += 256) {
    float s = 0.f;
    for (int c2 = 0; c2 < lanes_c; ++c2) s += sm_acc[(c2 * quads + d / 4) * 4 + (d & 3)];
    store_elem<T>(out, (int64_t)hq * out_head_stride + d, s * inv);
  }
  if (lse_out && t == 0)
    lse_out[hq] = lt > 0.f ? (mx + __builtin_amdgcn_logf(lt)) * kLn2 : -INFINITY;
}

static int pick_chunk(int64_t total_tokens, int n_kv_heads, int step_tokens) {
  // aim at ~8 blocks per CU on a 256-CU part, never below one unrolled round
  const int64_t want_blocks = 256 * 8;
  int64_t chunk = total_tokens * n_kv_heads / want_blocks;
  const int round = step_tokens * kAttnUnroll;
  if (chunk < round) chunk = round;
  if (chunk > 4096) chunk = 4096;
  return (int)(ceil_div(chunk, round) * round);
}

static int lanes_of(int head_dim, int dtype) {
  const int vec = dtype == DA_F32 ? 4 : 8;
  if (head_dim % vec) return 0;
  const int lanes = head_dim / vec;
  return (lanes >= 4 && lanes <= 64 && is_pow2(lanes)) ? lanes : 0;
}

static size_t attn_workspace_bytes(int n_q_heads, int head_dim, int64_t n_chunks) {
  return (size_t)n_chunks * n_q_heads * (head_dim + 2) * sizeof(float);
}

// Upper bound of the chunk count for a geometry (chunk size is fixed by the
// same rule at launch, from the same numbers).
static int64_t plan_chunks(int n_q_heads_unused, int n_kv_heads, int lanes, int64_t p_len,
                           int64_t c_capacity, int *chunk_out, int *n_p_out) {
  (void)n_q_heads_unused;
  const int step_tokens = kAttnWaves * (64 / lanes);
  const int chunk = pick_chunk(p_len + c_capacity, n_kv_heads, step_tokens);
  const int64_t n_p = ceil_div(p_len, chunk);
  const int64_t n_l = ceil_div(c_capacity, chunk);
  if (chunk_out) *chunk_out = chunk;
  if (n_p_out) *n_p_out = (int)n_p;
  return n_p + n_l;
}

template <typename T, int kLanes>
static void launch_split(const AttnArgs &a, int n_kv_heads, hipStream_t s) {
  const int rep = a.rep;
  if (rep <= 1) {
    dim3 grid(a.n_chunks, n_kv_heads, 1);
    hipLaunchKernelGGL((decode_attention_split_kernel<T, kLanes, 1>), grid, dim3(kAttnThreads), 0,
                       s, a);
  } else if (rep == 2) {
    dim3 grid(a.n_chunks, n_kv_heads, 1);
    hipLaunchKernelGGL((decode_attention_split_kernel<T, kLanes, 2>), grid, dim3(kAttnThreads), 0,
                       s, a);
  } else {
    dim3 grid(a.n_chunks, n_kv_heads, (unsigned)ceil_div(rep, 4));
    hipLaunchKernelGGL((decode_attention_split_kernel<T, kLanes, 4>), grid, dim3(kAttnThreads), 0,
                       s, a);
  }
}

template <typename T>
static int launch_attention(const AttnArgs &a, int n_kv_heads, int lanes, int head_dim, void *out,
                            int64_t out_head_stride, float *lse_out, hipStream_t s) {
  switch (lanes) {
    case 4: launch_split<T, 4>(a, n_kv_heads, s); break;
    case 8: launch_split<T, 8>(a, n_kv_heads, s); break;
    case 16: launch_split<T, 16>(a, n_kv_heads, s); break;
    case 32: launch_split<T, 32>(a, n_kv_heads, s); break;
    case 64: launch_split<T, 64>(a, n_kv_heads, s); break;
  }
  int rc = launch_status("da_decode_attention(split)");
  if (rc) return rc;
  hipLaunchKernelGGL(decode_attention_merge_kernel<T>, dim3(a.n_q_heads), dim3(256), 0, s, a,
                     head_dim, (char *)out, out_head_stride, lse_out);
  return launch_status("da_decode_attention(merge)");
}

}  // namespace da

extern "C" size_t da_decode_attention_workspace_bytes(int n_q_heads, int n_kv_heads,
                                                      int head_dim, int dtype, int64_t p_len,
                                                      int64_t c_capacity) {
  using namespace da;
  if (n_q_heads <= 0 || n_kv_heads <= 0 || p_len < 0 || c_capacity < 0) return 0;
  const int lanes = lanes_of(head_dim, dtype);
  if (!lanes) return 0;
  const int64_t n = plan_chunks(n_q_heads, n_kv_heads, lanes, p_len, c_capacity, nullptr, nullptr);
  return attn_workspace_bytes(n_q_heads, head_dim, n) + 16;
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
  using namespace da;
  DA_REQUIRE(n_q_heads > 0 && n_kv_heads > 0 && n_q_heads % n_kv_heads == 0,
             "da_decode_attention: %d query heads do not split over %d kv heads", n_q_heads,
             n_kv_heads);
  DA_REQUIRE(dtype == DA_F32 || dtype == DA_F16 || dtype == DA_BF16,
             "da_decode_attention: unknown dtype %d", dtype);
  DA_REQUIRE(p_len >= 0 && c_capacity >= 0 && c_len >= 0, "da_decode_attention: negative length");
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

  AttnArgs a;
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
  int chunk = 0, n_p = 0;
  const int64_t n_chunks = plan_chunks(n_q_heads, n_kv_heads, lanes, p_len, c_capacity, &chunk, &n_p);
  a.chunk = chunk;
  a.n_pchunks = n_p;
  a.n_chunks = (int)n_chunks;
  const size_t need = attn_workspace_bytes(n_q_heads, head_dim, n_chunks);
  DA_REQUIRE(workspace_bytes >= need, "da_decode_attention: workspace %zu < %zu bytes",
             workspace_bytes, need);
  DA_REQUIRE((uintptr_t)workspace % 16 == 0, "da_decode_attention: workspace must be 16-byte aligned");
  a.part_acc = (float *)workspace;
  a.part_ml = a.part_acc + (size_t)n_chunks * n_q_heads * head_dim;
  hipStream_t s = (hipStream_t)stream;
  if (n_chunks == 0) {
    // nothing to attend over: the merge kernel alone writes zeros / -inf
    a.n_chunks = 0;
  }
  switch (dtype) {
    case DA_F32:
      if (n_chunks == 0) break;
      return launch_attention<F32>(a, n_kv_heads, lanes, head_dim, out, out_head_stride, lse_out, s);
    case DA_F16:
      if (n_chunks == 0) break;
      return launch_attention<F16>(a, n_kv_heads, lanes, head_dim, out, out_head_stride, lse_out, s);
    default:
      if (n_chunks == 0) break;
      return launch_attention<BF16>(a, n_kv_heads, lanes, head_dim, out, out_head_stride, lse_out, s);
  }
  return fail(DA_EINVAL, "da_decode_attention: no key/value rows at all");
}
