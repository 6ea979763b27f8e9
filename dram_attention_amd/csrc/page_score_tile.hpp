// Page scorer for bf16 summaries whose bounds are ordered (min <= max in every
// channel, as da_page_minmax writes them): the form the decode step runs.
//
//   score[n,h,l] = sum_d rnd(max(q*min, q*max)) = sum_d rnd(q * (q >= 0 ? max : min))
//
// Bound: HBM, H*L*2*D*2 bytes read once for all query rows of the head.  The
// plain vector form needs ~2.5 vector instructions per (channel, query row)
// product pair and is bound by instruction issue at half the memory rate; this
// form needs one per product plus a sixth of one:
//   - min and max words are interleaved once per page slice (v_perm_b32: a word
//     (max_d, min_d) per channel, shared by all query rows), and the query is
//     split by sign into (q+, q-) words with q+ = q where q >= 0 else 0 and
//     q- = q - q+.  One v_dot2_f32_bf16 then gives max_d*q+ + min_d*q-, which
//     is q * (q >= 0 ? max : min) with an added +-0: a bf16 x bf16 product is
//     exact in fp32, so this equals the fp32 multiply of the unpacked operands
//     (checked on the hardware for every pair of bf16 values, denormals
//     included).  Operands that are not finite: 0 * inf = NaN arises from the
//     bound that should not count, and the plain form takes the maximum of
//     two products as fmax does (a NaN product loses against the other one,
//     as in the reference's tl.maximum), where this form has only their sum.
//     Both differences can only turn a score into NaN, never into another
//     number, so a NaN score is recomputed the plain way;
//   - two products are rounded by one v_cvt_pk_bf16_f32, and the packed words
//     ARE the A operand of v_mfma_f32_16x16x32_bf16: the matrix core adds up the
//     8 products of a lane and the 4 lanes that share a row in fp32, which takes
//     the place of the cross-lane reduction.  The B operand is an indicator
//     (ones in one column, zeros elsewhere) that routes the sums of (query row
//     r, step t) into column 4r + t of an accumulator shared by 16 products, so
//     the results of four steps come out next to each other, ready to store.
//
// Lane l of a wave: row i = l % 16, k-block kb = l / 16.  Row i stands for
// (page pi = i / kQ, part = i % kQ) and the lane reads 16-byte chunk part + kQ*kb
// of that page's rows (kQ = row bytes / 64): four adjacent lanes read 64
// contiguous bytes, the wave 16/kQ whole rows per load.  After the products of
// four steps, lane (kb, c) holds in its four accumulator registers rows
// 4*kb .. 4*kb+3 of column c = 4*r + t: the kQ parts of a page are summed in the
// lane and the lane stores the score of query row r for the page of step t (four
// adjacent lanes: four consecutive pages).  A wave scores kSteps * 16/kQ pages
// per round with all of the round's loads in flight at once.
//
#pragma once

#include "common.hpp"

namespace da {

typedef float score_f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 score_bf16x8 __attribute__((ext_vector_type(8)));
typedef short score_i16x2 __attribute__((ext_vector_type(2)));

// The products of one 16-byte slice (4 channel pairs = 8 channels) with one query
// row, as a block of hand-placed instructions: lo[e] = max*q+ + min*q- of the even
// channel of pair e, hi[e] of the odd one, each one v_dot2_f32_bf16 in the
// three-operand encoding with a literal zero addend (the compiler's own choice,
// the accumulating two-operand form, costs a register clear per product).
// Inline asm is invisible to the compiler's hazard tracking, so the block keeps
// two rules by construction:
//   - a dot product's result may be read by another kind of vector instruction
//     only three issue slots later: the block ends with s_nop 2, and everything
//     that reads lo/hi comes after the block;
//   - a vector instruction must not write a register that a matrix instruction
//     in flight still reads as its addend or is about to write: the block
//     writes ONLY read-write operands, variables that stay live for the whole
//     kernel, which the register allocator therefore never hands to an MFMA.
__device__ __forceinline__ void slice_products(uint32_t (&lo)[4], uint32_t (&hi)[4],
                                               const u32x4 &even, const u32x4 &odd,
                                               const uint32_t (&q_even)[4],
                                               const uint32_t (&q_odd)[4]) {
  asm("v_dot2_f32_bf16 %0, %8, %16, 0\n\t"
      "v_dot2_f32_bf16 %4, %12, %20, 0\n\t"
      "v_dot2_f32_bf16 %1, %9, %17, 0\n\t"
      "v_dot2_f32_bf16 %5, %13, %21, 0\n\t"
      "v_dot2_f32_bf16 %2, %10, %18, 0\n\t"
      "v_dot2_f32_bf16 %6, %14, %22, 0\n\t"
      "v_dot2_f32_bf16 %3, %11, %19, 0\n\t"
      "v_dot2_f32_bf16 %7, %15, %23, 0\n\t"
      "s_nop 2"
      : "+v"(lo[0]), "+v"(lo[1]), "+v"(lo[2]), "+v"(lo[3]), "+v"(hi[0]), "+v"(hi[1]),
        "+v"(hi[2]), "+v"(hi[3])
      : "v"(even[0]), "v"(even[1]), "v"(even[2]), "v"(even[3]), "v"(odd[0]), "v"(odd[1]),
        "v"(odd[2]), "v"(odd[3]), "v"(q_even[0]), "v"(q_even[1]), "v"(q_even[2]),
        "v"(q_even[3]), "v"(q_odd[0]), "v"(q_odd[1]), "v"(q_odd[2]), "v"(q_odd[3]));
}

// The plain statement of one score (any non-finite operand behaves as in the
// vector kernel); used for the rare entries the fast form cannot vouch for.
__device__ inline float page_score_exact_bf16(const char *q_row, const char *mn, const char *mx,
                                              int head_dim) {
  float a = 0.f;
  for (int d = 0; d < head_dim; ++d) {
    const float qv = load_elem<BF16>(q_row, d);
    a += round_bf16(fmaxf(qv * load_elem<BF16>(mn, d), qv * load_elem<BF16>(mx, d)));
  }
  return a;
}

template <int kQ, int kRows, int kSteps, bool kMulti>
__global__ void __launch_bounds__(256, 2)
page_score_tile_kernel(const char *__restrict__ q, int64_t q_row_stride, int64_t q_head_stride,
                       const char *__restrict__ mm, int n_rows, int64_t n_pages,
                       float *__restrict__ out, int64_t out_row_stride, int64_t out_head_stride,
                       int round_out, int rounds) {
  static_assert(kQ == 1 || kQ == 2 || kQ == 4, "rows of 64, 128 or 256 bytes");
  static_assert(kRows == 4 || kRows == 8, "4 or 8 query rows per block");
  static_assert(kSteps % 4 == 0, "an accumulator collects four steps");
  constexpr int kRpa = kRows == 4 ? 4 : 2;  // query rows per accumulator
  constexpr int kAcc = kRows / kRpa;
  constexpr int kP = 16 / kQ;               // pages per step
  constexpr int kRowBytes = 64 * kQ;
  constexpr int kWavePages = kSteps * kP;   // pages per wave and round
  constexpr int kHeadDim = kRowBytes / 2;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int kb = lane >> 4;
  const int j = lane & 15;
  const int pi = j / kQ;
  const int part = j % kQ;
  const int chunk = part + kQ * kb;
  const int h = blockIdx.y;
  const int row0 = blockIdx.z * kRows;

  // The only registers the inline asm ever writes (see slice_products), claimed
  // before anything else so that they are never shared with an MFMA operand.
  uint32_t t_lo[4], t_hi[4];
#pragma unroll
  for (int e = 0; e < 4; ++e)
    asm volatile("v_mov_b32 %0, 0\n\tv_mov_b32 %1, 0" : "=v"(t_lo[e]), "=v"(t_hi[e]));

  // the query words of this lane's 8 channels, requested first and unpacked only
  // after the first round's page loads have gone out (loads complete in order)
  u32x4 qw[kRows];
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const int n = row0 + r < n_rows ? row0 + r : n_rows - 1;
    qw[r] = load16(q + (n * q_row_stride + h * q_head_stride + (int64_t)chunk * 8) * 2);
  }
  // query operands: per channel pair the words (q+, q-) of its even and of its odd
  // channel, q+ = q where its sign bit is clear else 0, q- = q - q+
  uint32_t q_even[kRows][4], q_odd[kRows][4];
  auto unpack_query = [&]() {
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint32_t word = qw[r][e];
        // each half: all ones when its sign bit is set (packed arithmetic shift)
        const uint32_t neg_mask = __builtin_bit_cast(uint32_t, __builtin_bit_cast(score_i16x2, word) >> 15);
        const uint32_t pos = word & ~neg_mask, neg = word & neg_mask;
        q_even[r][e] = __builtin_amdgcn_perm(neg, pos, 0x05040100u);   // (pos.lo, neg.lo)
        q_odd[r][e] = __builtin_amdgcn_perm(neg, pos, 0x07060302u);    // (pos.hi, neg.hi)
      }
    }
  };
  // indicator operands: column c of the product, as B, receives the row sums
  score_bf16x8 route[kRpa * 4];
#pragma unroll
  for (int c = 0; c < kRpa * 4; ++c) {
    const uint32_t w = j == c ? 0x3f803f80u : 0u;
    route[c] = __builtin_bit_cast(score_bf16x8, u32x4{w, w, w, w});
  }

  const int64_t wave_id = (int64_t)blockIdx.x * 4 + wave;
  const int64_t n_waves = (int64_t)gridDim.x * 4;
  const char *head_base = mm + (int64_t)h * n_pages * 2 * kRowBytes;

  // page of (round, step, row) and the loads of a round (addresses clamped
  // into the head: scores of pages beyond the end are not stored)
  auto first_page = [&](int round) { return ((int64_t)round * n_waves + wave_id) * kWavePages; };
  const uint32_t last_page = (uint32_t)(n_pages - 1);   // page ids fit 31 bits (checked by the launcher)
  const char *lane_base = head_base + chunk * 16;
  auto issue = [&](int round, u32x4 *vmin, u32x4 *vmax) {
    const int64_t first = first_page(round) + (int64_t)pi * kSteps;
    const uint32_t base = first < n_pages ? (uint32_t)first : last_page;
#pragma unroll
    for (int s = 0; s < kSteps; ++s) {
      const uint32_t p = base + s < last_page ? base + s : last_page;
      const char *src = lane_base + (uint64_t)p * (2 * kRowBytes);
      vmin[s] = load16(src);
      vmax[s] = load16(src + kRowBytes);
    }
  };
  auto compute = [&](int round, const u32x4 *vmin, const u32x4 *vmax) {
#pragma unroll
    for (int s4 = 0; s4 < kSteps; s4 += 4) {
      score_f32x4 acc[kAcc];
#pragma unroll
      for (int a = 0; a < kAcc; ++a) acc[a] = score_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int s = s4 + t;
        // (max_d, min_d) words of the even and of the odd channel of every pair
        u32x4 even, odd;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          even[e] = __builtin_amdgcn_perm(vmin[s][e], vmax[s][e], 0x05040100u);
          odd[e] = __builtin_amdgcn_perm(vmin[s][e], vmax[s][e], 0x07060302u);
        }
#pragma unroll
        for (int r = 0; r < kRows; ++r) {
          slice_products(t_lo, t_hi, even, odd, q_even[r], q_odd[r]);
          u32x4 b;
#pragma unroll
          for (int e = 0; e < 4; ++e) b[e] = pack_bf16(as_f32(t_lo[e]), as_f32(t_hi[e]));
          acc[r / kRpa] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              __builtin_bit_cast(score_bf16x8, b), route[4 * (r % kRpa) + t], acc[r / kRpa], 0, 0, 0);
        }
      }
      // lane (kb, c): rows 4*kb + reg of column c = 4*r + t, i.e. the parts of
      // 4/kQ pages for query row r (of each accumulator) and step t
      const int r_local = j >> 2, t = j & 3;
      if (r_local < kRpa) {
#pragma unroll
        for (int a = 0; a < kAcc; ++a) {
          const int row = row0 + a * kRpa + r_local;
#pragma unroll
          for (int u = 0; u < 4 / kQ; ++u) {
            float v = acc[a][u * kQ];
#pragma unroll
            for (int w = 1; w < kQ; ++w) v += acc[a][u * kQ + w];
            const int64_t p = first_page(round) + (int64_t)((4 * kb) / kQ + u) * kSteps + s4 + t;
            if (row < n_rows && p < n_pages) {
              if (__builtin_expect(v != v, 0)) {   // see the note on operands that are not finite
                const char *pg = head_base + p * 2 * kRowBytes;
                v = page_score_exact_bf16(q + (row * q_row_stride + h * q_head_stride) * 2, pg,
                                          pg + kRowBytes, kHeadDim);
              }
              if (round_out) v = round_bf16(v);
              out[row * out_row_stride + h * out_head_stride + p] = v;
            }
          }
        }
      }
    }
  };

  if constexpr (!kMulti) {
    if (first_page(0) >= n_pages) return;
    u32x4 vmin[kSteps], vmax[kSteps];
    issue(0, vmin, vmax);
    __builtin_amdgcn_sched_barrier(0);   // all of the round's loads go out before anything waits
    unpack_query();
    compute(0, vmin, vmax);
  } else {
    // two register sets: the next round's loads are in flight while this one is scored
    u32x4 amin[kSteps], amax[kSteps], bmin[kSteps], bmax[kSteps];
    issue(0, amin, amax);
    __builtin_amdgcn_sched_barrier(0);
    unpack_query();
    for (int round = 0; round < rounds; round += 2) {
      issue(round + 1, bmin, bmax);   // clamped: harmless when there is no such round
      compute(round, amin, amax);
      issue(round + 2, amin, amax);
      if (round + 1 < rounds) compute(round + 1, bmin, bmax);
    }
  }
}

// Whether the tile kernel takes the shape, and its launch.
inline bool page_score_tile_supported(int head_dim, int64_t n_pages, int64_t out_row_stride,
                                      int64_t out_head_stride, const void *out, const void *q,
                                      const void *mm, int64_t q_row_stride, int64_t q_head_stride) {
  return (head_dim == 32 || head_dim == 64 || head_dim == 128) && n_pages >= 1 &&
         n_pages < ((int64_t)1 << 31) - 64 &&
         (uintptr_t)q % 16 == 0 && (uintptr_t)mm % 16 == 0 && q_row_stride % 8 == 0 &&
         q_head_stride % 8 == 0;
}

template <int kQ, int kRows>
static void launch_page_score_tile(const void *q, int64_t qrs, int64_t qhs, const void *mm,
                                   int n_rows, int n_heads, int64_t n_pages, float *out,
                                   int64_t ors, int64_t ohs, int round_out, hipStream_t s) {
  constexpr int kP = 16 / kQ;
  const unsigned z = (unsigned)ceil_div(n_rows, kRows);
  // One round per wave while that gives at most ~4 blocks per CU; the rounds of
  // larger inputs are shared out over ~1024 blocks.  Small inputs take the
  // shorter step count so that the grid still covers the chip.
  const int64_t total_pages = n_pages * n_heads;
  const int64_t target_blocks = 1024;
  auto blocks_for = [&](int steps) { return ceil_div(n_pages, (int64_t)4 * steps * kP); };
#define DA_TILE_LAUNCH(steps, multi, grid_x, rounds)                                            \
  hipLaunchKernelGGL((page_score_tile_kernel<kQ, kRows, steps, multi>),                         \
                     dim3((unsigned)(grid_x), n_heads, z), dim3(256), 0, s, (const char *)q, qrs, \
                     qhs, (const char *)mm, n_rows, n_pages, out, ors, ohs, round_out, rounds)
  // 8 steps per round need 64 registers of page data next to the query operands:
  // with 8 query rows that no longer fits, so those take 4 steps per round.
  constexpr bool kLong = kRows == 4;
  if (!kLong || total_pages * 2 <= (int64_t)4 * 8 * kP * 512) {
    if (blocks_for(4) * n_heads <= 2 * target_blocks) {         // one round of 4 steps
      DA_TILE_LAUNCH(4, false, blocks_for(4), 1);
      return;
    }
  } else if (blocks_for(8) * n_heads <= target_blocks) {         // one round of 8 steps
    if constexpr (kLong) DA_TILE_LAUNCH(8, false, blocks_for(8), 1);
    return;
  }
  {
    int64_t gx = target_blocks / n_heads;
    if (gx < 1) gx = 1;
    const int64_t wave_rounds = ceil_div(n_pages, (int64_t)4 * kP);   // per head, 4 steps each
    const int rounds = (int)ceil_div(wave_rounds, gx * 4);
    gx = ceil_div(wave_rounds, (int64_t)rounds * 4);
    DA_TILE_LAUNCH(4, true, gx, rounds);
  }
#undef DA_TILE_LAUNCH
}

}  // namespace da
