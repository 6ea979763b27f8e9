// The split-K pass of decode attention on the matrix cores, for 16-bit keys and
// values and GQA groups of up to 16 query heads: the same work and the same
// partial results as attention_split_block, with both contractions as MFMAs.
//
// A wave takes the chunk's tokens in tiles of 16.  With the group's query rows
// padded to 16, both products of a tile are 16x16 outputs:
//   S^T (tokens x rows)  = K (tokens x D) * Q^T (D x rows)      D/32 MFMAs, k = 32
//   O^T (D x rows)      += V^T (D x tokens) * P^T (tokens x rows)  D/16 MFMAs, k = 16
// Computing S transposed is what makes the second product free of shuffles: the
// accumulator layout of a 16x16 MFMA (lane l holds rows 4*(l/16)..+3 of column
// l%16) is exactly the B-operand layout of the k = 16 MFMA (lane l holds
// k = 4*(l/16)..+3 of column l%16), so exp2(S^T - m), rounded to the value type,
// feeds the second product as it stands.  K rows are the A operand of the first
// product straight from global memory (lane l: token l%16, 16 bytes at dims
// 32*s + 8*(l/16)).  V must be transposed (an A operand holds four tokens of one
// channel per lane): the wave writes the tile's V rows to LDS as loaded and reads
// them back with the transposing LDS load of gfx950, which hands lane i of a
// 16-lane group element i%4 of the 8-byte chunks addressed by lanes 4*j + i/4.
//
// The running maximum m is kept per query row (column l%16, equal in the four
// lane groups) and only raised when a score clears it by kRescaleSlack, as in
// the vector kernel; the sums l stay per lane until the end.
#pragma once
#include "attention_core.hpp"

namespace da {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

template <typename T>
struct MatrixOps;
template <>
struct MatrixOps<BF16> {
  static __device__ __forceinline__ f32x4 k32(const u32x4 &a, const u32x4 &b, const f32x4 &c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 k16(const i16x4 &a, const u32x2 &b, const f32x4 &c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, __builtin_bit_cast(i16x4, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) { return pack_bf16(lo, hi); }
};
template <>
struct MatrixOps<F16> {
  static __device__ __forceinline__ f32x4 k32(const u32x4 &a, const u32x4 &b, const f32x4 &c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 k16(const i16x4 &a, const u32x2 &b, const f32x4 &c) {
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4, a),
                                                 __builtin_bit_cast(f16x4, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) { return pack_f16(lo, hi); }
};

constexpr int kTileTokens = 16;

// Shapes this pass takes; the launch code falls back to the vector kernel otherwise.
inline bool tile_pass_supported(int dtype, int head_dim, int rep, bool paged_overlap,
                                int page_size) {
  if (dtype != DA_BF16 && dtype != DA_F16) return false;
  if (head_dim != 64 && head_dim != 128 && head_dim != 256) return false;
  if (rep > 16) return false;
  // a tile must lie inside one page for the "slot is being rewritten" test
  return !paged_overlap || page_size % kTileTokens == 0;
}

template <int kD, int kRows>
struct TileShared {
  static constexpr int kLdsRow = kD * 2 + 32;  // bytes; the pad spreads 4 token rows over 32 banks
  static constexpr int kTileBytes = kAttnWaves * kTileTokens * kLdsRow;
  static constexpr int kMergeBytes = kAttnWaves * kRows * (kD + 2) * 4;
  static constexpr int kBytes = kTileBytes > kMergeBytes ? kTileBytes : kMergeBytes;
};

// Prefix and local chunks only (the pass over the miss list stays with the
// vector kernel).  kRows: query rows kept at the end (4, 8 or 16 >= rep).
// kStreamLoads: K and V are read with streaming loads, which leave what the caches
// hold alone.  The pass itself is slower with them (128K shape: 29.4 instead of 26.4 us)
// but the launches after it find their data where it was; for a pass whose
// duration hides behind something else.
template <typename T, int kD, int kRows, bool kStreamLoads = false>
__device__ __forceinline__ void attention_tile_block(const AttnArgs &a, const int block_x,
                                                     const int h) {
  using Ops = MatrixOps<T>;
  using Sh = TileShared<kD, kRows>;
  constexpr int kSteps = kD / 32;                 // MFMAs of the first product; K loads per lane
  constexpr int kBlocks = kD / 16;                // MFMAs of the second product
  constexpr int kRowLanes = kD / 8;               // lanes that cover a V row with 16-byte loads
  constexpr int kRowsPerLoad = 64 / kRowLanes;
  constexpr int kVLoads = kTileTokens / kRowsPerLoad;
  constexpr int kLdsRow = Sh::kLdsRow;
  constexpr int kRoundTokens = kAttnWaves * kTileTokens;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int g = lane >> 4;
  const int c = lane & 15;
  const int chunk_id = a.chunk_base + block_x;

  const int kind = chunk_id < a.n_pchunks ? 0 : 1;
  const LocalLen ll = local_len(a);
  const int64_t c_len = ll.c_len;
  int64_t seg_len, t_begin;
  if (kind == 0) {
    seg_len = a.p_len;
    t_begin = (int64_t)chunk_id * a.chunk;
  } else {
    seg_len = c_len + (ll.has_new ? 1 : 0);
    t_begin = (int64_t)(chunk_id - a.n_pchunks) * a.chunk;
  }
  if (t_begin >= seg_len) return;  // the merge kernel skips this chunk as well
  const int64_t t_end = t_begin + a.chunk < seg_len ? t_begin + a.chunk : seg_len;

  const char *kbase, *vbase;
  int64_t tok_stride_b;
  if (kind == 1) {
    kbase = a.ck + h * a.c_head_stride * T::kBytes;
    vbase = a.cv + h * a.c_head_stride * T::kBytes;
    tok_stride_b = a.c_tok_stride * T::kBytes;
  } else {
    kbase = a.pk + h * a.p_head_stride * T::kBytes;
    vbase = a.pv + h * a.p_head_stride * T::kBytes;
    tok_stride_b = a.p_tok_stride * T::kBytes;
  }
  const char *newk = nullptr, *newv = nullptr;
  if (kind == 1 && ll.has_new) {
    newk = a.new_k + h * a.new_head_stride * T::kBytes;
    newv = a.new_v + h * a.new_head_stride * T::kBytes;
  }
  const bool skip_fresh = kind == 0 && a.slot_epoch != nullptr;
  const int32_t epoch_now = skip_fresh ? *a.epoch : 0;
  const int32_t *slot_epoch = skip_fresh ? a.slot_epoch + h * a.slot_epoch_head_stride : nullptr;

  __shared__ __align__(16) char smem[Sh::kBytes];
  char *vt = smem + wave * (kTileTokens * kLdsRow);

  // Q^T as the B operand: lane (g, c) holds row c, dims 32*s + 8*g .. +7; rows past
  // the group are zero.
  u32x4 qv[kSteps];
  {
    const int rr = c < a.rep ? c : a.rep - 1;
    const char *qp = a.q + ((int64_t)(h * a.rep + rr) * a.q_head_stride) * T::kBytes + g * 16;
#pragma unroll
    for (int s = 0; s < kSteps; ++s) {
      qv[s] = load16(qp + s * 64);
      if (c >= a.rep) qv[s] = u32x4{0, 0, 0, 0};
    }
  }

  float m = kMinusHuge, l = 0.f;
  f32x4 acc[kBlocks];
#pragma unroll
  for (int b = 0; b < kBlocks; ++b) acc[b] = f32x4{0.f, 0.f, 0.f, 0.f};

  // Loads of one tile: always the same count, on clamped addresses past the chunk
  // end, so that the waits between fetch and use stay partial.
  auto fetch = [&](int64_t tile, u32x4 *kk, u32x4 *vv, int32_t &ep) {
    const bool live = tile < t_end;
    {
      const int64_t tok = tile + c;
      const int64_t tk = (live && tok < t_end) ? tok : t_begin;
      const char *kp = (newk != nullptr && tk == c_len) ? newk : kbase + tk * tok_stride_b;
#pragma unroll
      for (int s = 0; s < kSteps; ++s)
        kk[s] = kStreamLoads ? load16_stream(kp + s * 64 + g * 16) : load16(kp + s * 64 + g * 16);
    }
#pragma unroll
    for (int j = 0; j < kVLoads; ++j) {
      const int64_t tok = tile + lane / kRowLanes + j * kRowsPerLoad;
      const int64_t tk = (live && tok < t_end) ? tok : t_begin;
      const char *vp = (newv != nullptr && tk == c_len) ? newv : vbase + tk * tok_stride_b;
      vv[j] = kStreamLoads ? load16_stream(vp + (lane % kRowLanes) * 16)
                           : load16(vp + (lane % kRowLanes) * 16);
    }
    if (skip_fresh) {
      const int64_t tk = live ? tile : t_begin;
      ep = slot_epoch[a.page_shift >= 0 ? tk >> a.page_shift : tk / a.page_size];
    }
  };

  auto consume = [&](int64_t tile, const u32x4 *kk, u32x4 *vv, int32_t ep) {
    int64_t left = t_end - tile;
    // a slot that is being rewritten right now is left to the pass over the miss list
    if (skip_fresh && ep == epoch_now) left = 0;
    if (left <= 0) return;
    const int n_valid = left < kTileTokens ? (int)left : kTileTokens;

    f32x4 st = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < kSteps; ++s) st = Ops::k32(kk[s], qv[s], st);
    float sv[4];
    float smax = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      sv[i] = (4 * g + i < n_valid) ? st[i] * a.scale_log2 : -INFINITY;
      smax = fmaxf(smax, sv[i]);
    }
    if (__any(smax > m + kRescaleSlack)) {  // rare
      float mx = fmaxf(m, smax);
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float alpha = fast_exp2(m - mx);
      m = mx;
      l *= alpha;
#pragma unroll
      for (int b = 0; b < kBlocks; ++b) acc[b] *= alpha;
    }
    float p[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      p[i] = fast_exp2(sv[i] - m);
      l += p[i];
    }
    const u32x2 pt = u32x2{Ops::pack(p[0], p[1]), Ops::pack(p[2], p[3])};

    // V rows to LDS as loaded; rows past the end are memory nobody vouches for
    // (torn values, NaN): zeroed, so that 0 * NaN cannot arise
#pragma unroll
    for (int j = 0; j < kVLoads; ++j) {
      const int row = lane / kRowLanes + j * kRowsPerLoad;
      if (row >= n_valid) vv[j] = u32x4{0, 0, 0, 0};
      *(u32x4 *)(vt + row * kLdsRow + (lane % kRowLanes) * 16) = vv[j];
    }
    __builtin_amdgcn_wave_barrier();
    const char *tr = vt + (4 * g + (c >> 2)) * kLdsRow + (c & 3) * 8;
#pragma unroll
    for (int b = 0; b < kBlocks; ++b) {
      const i16x4 va = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (i16x4 __attribute__((address_space(3))) *)(tr + b * 32));
      acc[b] = Ops::k16(va, pt, acc[b]);
    }
    __builtin_amdgcn_wave_barrier();
  };

  {
    u32x4 ka[kSteps], va[kVLoads], kb[kSteps], vb[kVLoads];
    int32_t ea = 0, eb = 0;
    int64_t tile = t_begin + wave * kTileTokens;
    fetch(tile, ka, va, ea);
    for (; tile < t_end; tile += 2 * kRoundTokens) {
      fetch(tile + kRoundTokens, kb, vb, eb);
      consume(tile, ka, va, ea);
      fetch(tile + 2 * kRoundTokens, ka, va, ea);
      consume(tile + kRoundTokens, kb, vb, eb);
    }
  }

  // The append: the block whose chunk holds row c_len copies the new token in
  // (every read of that row above went to new_k / new_v instead).
  if (newk != nullptr && c_len >= t_begin && c_len < t_end && threadIdx.x < 2 * kRowLanes) {
    const int part = threadIdx.x % kRowLanes;
    const bool is_v = threadIdx.x >= kRowLanes;
    char *dst = (is_v ? a.cv : a.ck) + (h * a.c_head_stride + c_len * a.c_tok_stride) * T::kBytes;
    store16(dst + part * 16, load16((is_v ? newv : newk) + part * 16));
  }

  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);

  // Merge the four waves through LDS (the tile buffers are dead by now).
  __syncthreads();
  float *sm_m = (float *)smem;                        // [wave][kRows]
  float *sm_l = sm_m + kAttnWaves * kRows;            // [wave][kRows]
  float *sm_acc = sm_l + kAttnWaves * kRows;          // [wave][kRows][kD]
  if (c < kRows) {
    if (g == 0) {
      sm_m[wave * kRows + c] = m;
      sm_l[wave * kRows + c] = l;
    }
#pragma unroll
    for (int b = 0; b < kBlocks; ++b) {
#pragma unroll
      for (int i = 0; i < 4; ++i) sm_acc[(wave * kRows + c) * kD + 16 * b + 4 * g + i] = acc[b][i];
    }
  }
  __syncthreads();
  for (int item = threadIdx.x; item < kRows * kD; item += kAttnThreads) {
    const int r = item / kD, d = item % kD;
    if (r >= a.rep) continue;
    float mn = sm_m[r];
#pragma unroll
    for (int w = 1; w < kAttnWaves; ++w) mn = fmaxf(mn, sm_m[w * kRows + r]);
    float lt = 0.f, at = 0.f;
#pragma unroll
    for (int w = 0; w < kAttnWaves; ++w) {
      const float wgt = fast_exp2(sm_m[w * kRows + r] - mn);
      lt += sm_l[w * kRows + r] * wgt;
      at += sm_acc[(w * kRows + r) * kD + d] * wgt;
    }
    const int64_t hq = (int64_t)h * a.rep + r;
    const int64_t slot = (int64_t)chunk_id * a.n_q_heads + hq;
    a.part_acc[slot * kD + d] = at;
    if (d == 0) {
      a.part_ml[slot * 2] = mn;
      a.part_ml[slot * 2 + 1] = lt;
    }
  }
}

template <typename T, int kD, int kRows>
__global__ void __launch_bounds__(kAttnThreads)
decode_attention_tile_kernel(const AttnArgs a) {
  attention_tile_block<T, kD, kRows>(a, blockIdx.x, blockIdx.y);
}

}  // namespace da
