// Causal attention over the whole prompt (the prefill stage): tiled flash
// attention on the matrix cores.  Counterpart of
// flash_attn_func(xq, xk, xv, causal=True) in dram_attention/dram_attention.py:136
// of the reference.
//
// Bound: MFMA.  4*S*S*D*Hq/2 flops (the causal half of two S x S x D products
// per query head); K and V are re-read once per block of query rows, nearly always
// from the L2 of the die the workgroup runs on (its neighbours there walk the same keys).
//
// Work split: a 512-thread workgroup, one per CU, owns kHeads query heads of one kv
// head (the GQA group, or a part of it) times 256/kHeads consecutive query rows;
// each of its eight waves owns 32 query rows of one head (two waves per SIMD: the
// registers of a wave allow no more, and with eight waves on one tile instead of two
// workgroups of four on two the CU loads half as many tile rows).  All waves walk the
// same keys, so one tile of K and V in LDS serves the whole group.  Per tile
// of 64 keys a wave computes, with 32x32x16 MFMAs,
//   S^T (keys x rows)  = K (keys x D) * Q^T (D x rows)        D/16 per 32 keys
//   O^T (D x rows)    += V^T (D x keys) * P^T (keys x rows)   D/32 per 16 keys
// S is computed transposed so that the accumulator layout of the first product
// (lane l: row l%32, keys 8j + 4(l/32) + i in register 4j + i) is, two register
// groups at a time, the B-operand layout of the second (lane l: row l%32, eight
// k indices): exp2(S^T - m) rounded to the value type feeds the second product
// without a shuffle.  The k index of that product then runs over the keys in the
// order (4g..4g+3, 8+4g..8+4g+3), g = l/32, and the A operand V^T follows it: two
// transposing LDS loads (ds_read_b64_tr_b16) of four keys each per MFMA.
// Q^T stays in registers for the whole pass; K rows are the A operand of the
// first product straight from the LDS tile (one 16-byte read per MFMA).
//
// The next tile's K/V rows travel from global memory straight into the other LDS
// buffer (loads that write LDS, no registers in between) while the current tile is
// computed: one barrier per tile.  Softmax state per query row: a running reference m that
// is only raised when a score clears it by kRescaleSlack (as in the decode
// kernels), per-lane partial sums, everything in the log2 domain.
// Workgroups take the longest rows first; which kv head a workgroup works on follows the
// die it runs on where the heads deal out evenly over the dies (see the kernel).
#include <type_traits>

#include "attention_core.hpp"

namespace da {

typedef float pf_f32x16 __attribute__((ext_vector_type(16)));
typedef short pf_i16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 pf_bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 pf_f16x8 __attribute__((ext_vector_type(8)));

template <typename T>
struct PrefillOps;
template <>
struct PrefillOps<BF16> {
  static __device__ __forceinline__ pf_f32x16 mma(const u32x4 &a, const u32x4 &b,
                                                  const pf_f32x16 &c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(pf_bf16x8, a),
                                                   __builtin_bit_cast(pf_bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) { return pack_bf16(lo, hi); }
};
template <>
struct PrefillOps<F16> {
  static __device__ __forceinline__ pf_f32x16 mma(const u32x4 &a, const u32x4 &b,
                                                  const pf_f32x16 &c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(pf_f16x8, a),
                                                  __builtin_bit_cast(pf_f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) { return pack_f16(lo, hi); }
};

struct PrefillArgs {
  const char *q, *k, *v;
  char *out;
  float *lse;  // (Hq, S) natural log, or null
  int64_t q_tok_stride, q_head_stride;  // elements
  int64_t k_tok_stride, k_head_stride;
  int64_t v_tok_stride, v_head_stride;
  int64_t o_tok_stride, o_head_stride;
  int64_t seq_len;
  int rep;          // query heads per kv head
  int n_groups;     // workgroups that share a kv head's rows: rep / kHeads
  int64_t n_row_blocks;
  int heads_per_xcd;  // kv heads per die when they deal out evenly, else 0
  float scale_log2;
};

constexpr int kPfThreads = 512;
constexpr int kPfWaves = 8;
constexpr int kPfKeys = 64;  // keys per tile
constexpr int kXcds = 8;     // dies (XCDs) of the part; consecutive workgroup ids go to consecutive dies

// LDS layout of a tile.  K and V rows arrive by loads that write LDS directly
// (global_load_lds_dwordx4: no staging registers, no LDS store instructions): a wave
// instruction deposits its 64 lanes' 16-byte chunks at 64 consecutive places, one block
// of 1024 bytes = kRows rows.  Which chunk a lane fetches is free, so the chunks of a
// block are placed with their column index XORed by a function of the row: the 16
// lanes that read one column of 16 rows (K rows as MFMA operands), and the 8 rows x 64
// bytes of a transposing read of V, then fall on distinct banks; 16 bytes of padding
// per block shift consecutive blocks by one bank group.
template <int kD>
struct PrefillShared {
  static constexpr int kRowBytes = kD * 2;
  static constexpr int kRows = 1024 / kRowBytes;          // rows per block: 4 (D 128) or 8 (D 64)
  static constexpr int kChunks = kRowBytes / 16;          // 16-byte chunks per row
  static constexpr int kBlock = 1024 + 16;                // bytes from block to block
  static constexpr int kBlocks = kPfKeys / kRows;         // blocks per tile (K, and V)
  static constexpr int kKBytes = kBlocks * kBlock;
  static constexpr int kBufBytes = 2 * kKBytes;           // K tile, then V tile
  static constexpr int kOutRow = kD * 2 + 16;             // epilogue staging
  static constexpr int kOutBytes = kPfWaves * 32 * kOutRow;
  static constexpr int kBytes = 2 * kBufBytes > kOutBytes ? 2 * kBufBytes : kOutBytes;
  // column swizzle of row rr of a block (a multiple of the chunk index's high bits)
  static __host__ __device__ constexpr int swizzle(int rr) { return kD == 128 ? 4 * rr : 2 * (rr >> 1); }
  // byte offset of chunk cc of row r of a tile
  static __device__ __forceinline__ int at(int r, int cc) {
    return (r / kRows) * kBlock + (r % kRows) * kRowBytes + ((cc ^ swizzle(r % kRows)) * 16);
  }
};

template <typename T, int kD, int kHeads>
__global__ void __launch_bounds__(kPfThreads, 1)
prefill_attention_kernel(const PrefillArgs a) {
  using Ops = PrefillOps<T>;
  using Sh = PrefillShared<kD>;
  static_assert(kD == 64 || kD == 128, "head sizes of 64 and 128");
  static_assert(kHeads == 1 || kHeads == 2 || kHeads == 4, "1, 2 or 4 query heads per workgroup");
  constexpr int kRowBlocks = kPfWaves / kHeads;       // 32-row blocks per workgroup
  constexpr int kBlockRows = 32 * kRowBlocks;
  constexpr int kQSteps = kD / 16;                    // MFMAs of S^T per 32 keys
  constexpr int kCBlocks = kD / 32;                   // 32-channel blocks of O^T
  constexpr int kRowChunks = kD / 8;                  // 16-byte chunks per K/V row
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int g = lane >> 5;
  const int c = lane & 31;

  // workgroup -> (kv head, row block, head group), long rows first.  Workgroups are dealt
  // to the chip's kXcds dies in turn and every die has a cache of its own: with a multiple
  // of kXcds kv heads, workgroup b works on a head that is b's die's alone (b % kXcds,
  // + kXcds, ...), so that a die's cache holds the keys and values of one head at a time
  // and no two dies fetch the same rows.  Otherwise: kv head by kv head.
  const int64_t per_head = a.n_row_blocks * a.n_groups;
  int hk;
  int64_t rem;
  if (a.heads_per_xcd > 0) {
    const int64_t j = blockIdx.x / kXcds;               // this die's j-th workgroup
    hk = (int)(blockIdx.x % kXcds) + kXcds * (int)(j / per_head);
    rem = j % per_head;
  } else {
    hk = (int)(blockIdx.x / per_head);
    rem = blockIdx.x % per_head;
  }
  const int64_t rb = a.n_row_blocks - 1 - rem / a.n_groups;
  const int hg = (int)(rem % a.n_groups);
  const int hq = hk * a.rep + hg * kHeads + wave % kHeads;
  const int64_t S = a.seq_len;
  const int64_t m0 = rb * kBlockRows;                       // first row of the workgroup
  const int64_t row0 = m0 + (wave / kHeads) * 32;           // first row of this wave
  const int64_t my_row = row0 + c;
  const int64_t last_key = (m0 + kBlockRows < S ? m0 + kBlockRows : S) - 1;  // last key any wave needs
  const int n_tiles = (int)(last_key / kPfKeys) + 1;
  // keys beyond this wave's last row are masked for all of its rows
  const int64_t wave_last_key = row0 + 31 < S ? row0 + 31 : S - 1;

  __shared__ __align__(16) char smem[Sh::kBytes];

  // Q^T as the B operand: lane (g, c) holds row c, channels 16*s + 8*g .. +7
  u32x4 qf[kQSteps];
  {
    const int64_t r = my_row < S ? my_row : S - 1;
    const char *qp = a.q + (r * a.q_tok_stride + (int64_t)hq * a.q_head_stride) * T::kBytes + g * 16;
#pragma unroll
    for (int s = 0; s < kQSteps; ++s) qf[s] = load16(qp + s * 32);
  }

  const char *kbase = a.k + (int64_t)hk * a.k_head_stride * T::kBytes;
  const char *vbase = a.v + (int64_t)hk * a.v_head_stride * T::kBytes;
  const int64_t k_tok_b = a.k_tok_stride * T::kBytes, v_tok_b = a.v_tok_stride * T::kBytes;

  // Tile loads.  Wave w brings blocks w, w + 4, ... of K and of V; lane L of the wave
  // owns place L of a block, i.e. row L / kChunks and the chunk whose swizzled column is
  // L % kChunks.  Offsets inside a tile fit 32 bits (checked by the launcher).
  constexpr int kBlocksPerWave = Sh::kBlocks / kPfWaves;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int ld_row = lane / Sh::kChunks;
  const int ld_col = (lane % Sh::kChunks) ^ Sh::swizzle(ld_row);
  const uint32_t k_rel = (uint32_t)(ld_row * k_tok_b) + ld_col * 16;
  const uint32_t v_rel = (uint32_t)(ld_row * v_tok_b) + ld_col * 16;
  typedef __attribute__((address_space(1))) const void *GlobalPtr;
  typedef __attribute__((address_space(3))) void *LdsPtr;
  auto fetch = [&](int tile, int buf) {
    const int64_t t0 = (int64_t)tile * kPfKeys;
    char *kt = smem + buf * Sh::kBufBytes;
    if (t0 + kPfKeys - 1 <= last_key) {             // a whole tile: one base, constant offsets
      const char *kt0 = kbase + t0 * k_tok_b, *vt0 = vbase + t0 * v_tok_b;
#pragma unroll
      for (int u = 0; u < kBlocksPerWave; ++u) {
        const int blk = wave_u + u * kPfWaves;
        __builtin_amdgcn_global_load_lds(
            (GlobalPtr)(kt0 + (int64_t)blk * Sh::kRows * k_tok_b + k_rel),
            (LdsPtr)(kt + blk * Sh::kBlock), 16, 0, 0);
        __builtin_amdgcn_global_load_lds(
            (GlobalPtr)(vt0 + (int64_t)blk * Sh::kRows * v_tok_b + v_rel),
            (LdsPtr)(kt + Sh::kKBytes + blk * Sh::kBlock), 16, 0, 0);
      }
    } else {                                        // the ragged last tile: rows clamped into range
#pragma unroll
      for (int u = 0; u < kBlocksPerWave; ++u) {
        const int blk = wave_u + u * kPfWaves;
        int64_t tok = t0 + blk * Sh::kRows + ld_row;
        if (tok > last_key) tok = last_key;         // in bounds; such keys are masked
        __builtin_amdgcn_global_load_lds((GlobalPtr)(kbase + tok * k_tok_b + ld_col * 16),
                                         (LdsPtr)(kt + blk * Sh::kBlock), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((GlobalPtr)(vbase + tok * v_tok_b + ld_col * 16),
                                         (LdsPtr)(kt + Sh::kKBytes + blk * Sh::kBlock), 16, 0, 0);
      }
    }
  };

  // LDS addresses of this lane's operands inside a tile.  K, as the A operand of S^T:
  // row c of a half, chunk 2s + g.  V, for the transposing load: lane i of a 16-lane
  // group addresses key t0 + i/4, channels c0 + 4*(i%4) .. +3 and receives channel
  // c0 + i of keys t0..t0+3; t0 = 4g (+8, +16 per group of keys), c0 = 32b + 16*((lane/16)%2).
  int k_at[kQSteps], v_at[kCBlocks];
#pragma unroll
  for (int s2 = 0; s2 < kQSteps; ++s2) k_at[s2] = Sh::at(c, 2 * s2 + g);
  {
    const int i16 = lane & 15;
#pragma unroll
    for (int b = 0; b < kCBlocks; ++b)
      v_at[b] = Sh::kKBytes + Sh::at(4 * g + (i16 >> 2), 4 * b + 2 * ((lane >> 4) & 1) + ((i16 & 3) >> 1)) +
                (i16 & 1) * 8;
  }
  constexpr int kHalfStep = (32 / Sh::kRows) * Sh::kBlock;   // 32 rows further down a tile
  constexpr int kKeys16 = (16 / Sh::kRows) * Sh::kBlock;     // 16 rows
  constexpr int kKeys8 = (8 / Sh::kRows) * Sh::kBlock;       // 8 rows

  float m = kMinusHuge, l = 0.f;
  pf_f32x16 acc[kCBlocks];
#pragma unroll
  for (int b = 0; b < kCBlocks; ++b)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[b][i] = 0.f;

  // One tile of 64 keys from LDS buffer `buf`; kMask: keys above a row are dropped.
  auto compute = [&](int tile, int buf, auto mask_tag) {
    constexpr bool kMask = decltype(mask_tag)::value;
    const char *kt = smem + buf * Sh::kBufBytes;
    pf_f32x16 st[2];
    // (raised priority while a wave issues MFMAs: they go ahead of the vector work of the
    // other wave on this SIMD, which fills the gaps; worth 0-2 % from run to run)
    __builtin_amdgcn_s_setprio(3);
#pragma unroll
    for (int half = 0; half < 2; ++half) {
#pragma unroll
      for (int i = 0; i < 16; ++i) st[half][i] = 0.f;
#pragma unroll
      for (int s = 0; s < kQSteps; ++s)
        st[half] = Ops::mma(*(const u32x4 *)(kt + k_at[s] + half * kHalfStep), qf[s], st[half]);
    }
    __builtin_amdgcn_s_setprio(0);
    // register 4j + i of half `half`: key tile*64 + half*32 + 8j + 4g + i
    float smax = -INFINITY;
    if constexpr (kMask) {
      const int lim = (int)(my_row - ((int64_t)tile * kPfKeys + 4 * g));  // key offset <= lim stays
#pragma unroll
      for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (half * 32 + 8 * j + i > lim) st[half][4 * j + i] = -INFINITY;
    }
#pragma unroll
    for (int half = 0; half < 2; ++half)
#pragma unroll
      for (int i = 0; i < 16; ++i) smax = fmaxf(smax, st[half][i]);
    smax *= a.scale_log2;   // the scale is positive: max and scaling commute
    if (__any(smax > m + kRescaleSlack)) {  // rare after the first tiles
      float mx = fmaxf(m, smax);
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float alpha = fast_exp2(m - mx);
      m = mx;
      l *= alpha;
#pragma unroll
      for (int b = 0; b < kCBlocks; ++b)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[b][i] *= alpha;
    }
    u32x4 pt[4];  // P^T operands: [half*2 + jj], keys half*32 + 16*jj + (4g..4g+3, 8+4g..8+4g+3)
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      float p[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        p[i] = fast_exp2(fmaf(st[half][i], a.scale_log2, -m));
        l += p[i];
      }
#pragma unroll
      for (int jj = 0; jj < 2; ++jj)
        pt[half * 2 + jj] = u32x4{Ops::pack(p[8 * jj], p[8 * jj + 1]), Ops::pack(p[8 * jj + 2], p[8 * jj + 3]),
                                  Ops::pack(p[8 * jj + 4], p[8 * jj + 5]), Ops::pack(p[8 * jj + 6], p[8 * jj + 7])};
    }
    __builtin_amdgcn_s_setprio(3);
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {   // 16 keys each
#pragma unroll
      for (int b = 0; b < kCBlocks; ++b) {
        const char *p0 = kt + v_at[b] + kk * kKeys16;
        const pf_i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (pf_i16x4 __attribute__((address_space(3))) *)(p0));
        const pf_i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (pf_i16x4 __attribute__((address_space(3))) *)(p0 + kKeys8));
        const u32x4 va = __builtin_bit_cast(u32x4, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        acc[b] = Ops::mma(va, pt[kk], acc[b]);
      }
    }
    __builtin_amdgcn_s_setprio(0);
  };

  fetch(0, 0);
  // The query rows have arrived before the loop starts (they were requested ahead of
  // tile 0): inside the loop nothing then waits for a load except the tile's own.
#pragma unroll
  for (int s = 0; s < kQSteps; ++s) asm volatile("" : "+v"(qf[s]));
  __syncthreads();                                  // (waits for this wave's tile loads first)
  for (int tile = 0; tile < n_tiles; ++tile) {
    const int buf = tile & 1;
    // the other buffer was last read before the barrier that ended the previous round
    if (tile + 1 < n_tiles) fetch(tile + 1, buf ^ 1);
    const int64_t t0 = (int64_t)tile * kPfKeys;
    if (t0 <= wave_last_key) {                     // else: every key of the tile is masked for this wave
      if (t0 + kPfKeys - 1 > row0) compute(tile, buf, std::true_type{});
      else compute(tile, buf, std::false_type{});
    }
    __syncthreads();                                // tile + 1 has landed, and everyone is done with `buf`
  }

  // ---- epilogue: normalise, transpose through LDS, store rows of 16-byte lanes
  l += __shfl_xor(l, 32, 64);
  const float inv = l > 0.f ? 1.f / l : 0.f;
  char *ot = smem + wave * 32 * Sh::kOutRow;     // (the last barrier retired every read of the tiles)
#pragma unroll
  for (int b = 0; b < kCBlocks; ++b)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t w0 = Ops::pack(acc[b][4 * j] * inv, acc[b][4 * j + 1] * inv);
      const uint32_t w1 = Ops::pack(acc[b][4 * j + 2] * inv, acc[b][4 * j + 3] * inv);
      *(uint2 *)(ot + c * Sh::kOutRow + (32 * b + 8 * j + 4 * g) * 2) = make_uint2(w0, w1);
    }
  __builtin_amdgcn_wave_barrier();
  constexpr int kRowsPerPass = 64 / kRowChunks;
#pragma unroll
  for (int pass = 0; pass < 32 / kRowsPerPass; ++pass) {
    const int r = pass * kRowsPerPass + lane / kRowChunks;
    const int col = lane % kRowChunks;
    const int64_t row = row0 + r;
    if (row < S)
      store16(a.out + (row * a.o_tok_stride + (int64_t)hq * a.o_head_stride) * T::kBytes + col * 16,
              *(const u32x4 *)(ot + r * Sh::kOutRow + col * 16));
  }
  if (a.lse != nullptr && g == 0 && my_row < S)
    a.lse[(int64_t)hq * S + my_row] = l > 0.f ? (m + __builtin_amdgcn_logf(l)) * kLn2 : -INFINITY;
}

template <typename T, int kD>
static int launch_prefill(PrefillArgs a, int n_kv_heads, hipStream_t s) {
  const int heads = a.rep % 4 == 0 ? 4 : (a.rep % 2 == 0 ? 2 : 1);
  const int block_rows = 32 * (kPfWaves / heads);
  a.n_groups = a.rep / heads;
  a.n_row_blocks = ceil_div(a.seq_len, block_rows);
  a.heads_per_xcd = n_kv_heads % kXcds == 0 ? n_kv_heads / kXcds : 0;
  const int64_t blocks = a.n_row_blocks * a.n_groups * n_kv_heads;
  if (blocks > 0x7fffffff) return fail(DA_ENOTSUP, "da_prefill_attention: %lld workgroups", (long long)blocks);
  const dim3 grid((unsigned)blocks);
  if (heads == 4)
    hipLaunchKernelGGL((prefill_attention_kernel<T, kD, 4>), grid, dim3(kPfThreads), 0, s, a);
  else if (heads == 2)
    hipLaunchKernelGGL((prefill_attention_kernel<T, kD, 2>), grid, dim3(kPfThreads), 0, s, a);
  else
    hipLaunchKernelGGL((prefill_attention_kernel<T, kD, 1>), grid, dim3(kPfThreads), 0, s, a);
  return launch_status("da_prefill_attention");
}

}  // namespace da

extern "C" int da_prefill_attention(const void *q, int64_t q_tok_stride, int64_t q_head_stride,
                                    const void *k, int64_t k_tok_stride, int64_t k_head_stride,
                                    const void *v, int64_t v_tok_stride, int64_t v_head_stride,
                                    int64_t seq_len, int n_q_heads, int n_kv_heads, int head_dim,
                                    int dtype, float scale, void *out, int64_t o_tok_stride,
                                    int64_t o_head_stride, float *lse_out, void *stream) {
  using namespace da;
  DA_REQUIRE(n_q_heads > 0 && n_kv_heads > 0 && n_q_heads % n_kv_heads == 0,
             "da_prefill_attention: %d query heads do not split over %d kv heads", n_q_heads,
             n_kv_heads);
  DA_REQUIRE(seq_len >= 0, "da_prefill_attention: negative length");
  DA_REQUIRE(dtype == DA_F32 || dtype == DA_F16 || dtype == DA_BF16,
             "da_prefill_attention: unknown dtype %d", dtype);
  DA_REQUIRE(scale > 0.f, "da_prefill_attention: the softmax scale must be positive");
  if (seq_len == 0) return DA_OK;
  DA_REQUIRE(q && k && v && out, "da_prefill_attention: null pointer");
  if (dtype == DA_F32 || (head_dim != 64 && head_dim != 128))
    return fail(DA_ENOTSUP,
                "da_prefill_attention: bf16 or fp16 with head_dim 64 or 128 (got dtype %d, head_dim %d)",
                dtype, head_dim);
  DA_REQUIRE(q_tok_stride % 8 == 0 && q_head_stride % 8 == 0 && k_tok_stride % 8 == 0 &&
                 k_head_stride % 8 == 0 && v_tok_stride % 8 == 0 && v_head_stride % 8 == 0 &&
                 o_tok_stride % 8 == 0 && o_head_stride % 8 == 0 && (uintptr_t)q % 16 == 0 &&
                 (uintptr_t)k % 16 == 0 && (uintptr_t)v % 16 == 0 && (uintptr_t)out % 16 == 0,
             "da_prefill_attention: rows must be 16-byte aligned");
  if (k_tok_stride < 0 || v_tok_stride < 0 || k_tok_stride > (1 << 23) || v_tok_stride > (1 << 23))
    return fail(DA_ENOTSUP, "da_prefill_attention: key/value token strides of 0..2^23 elements");
  PrefillArgs a = {};
  a.q = (const char *)q;
  a.k = (const char *)k;
  a.v = (const char *)v;
  a.out = (char *)out;
  a.lse = lse_out;
  a.q_tok_stride = q_tok_stride;
  a.q_head_stride = q_head_stride;
  a.k_tok_stride = k_tok_stride;
  a.k_head_stride = k_head_stride;
  a.v_tok_stride = v_tok_stride;
  a.v_head_stride = v_head_stride;
  a.o_tok_stride = o_tok_stride;
  a.o_head_stride = o_head_stride;
  a.seq_len = seq_len;
  a.rep = n_q_heads / n_kv_heads;
  a.scale_log2 = scale * kLog2e;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == DA_BF16)
    return head_dim == 128 ? launch_prefill<BF16, 128>(a, n_kv_heads, s)
                           : launch_prefill<BF16, 64>(a, n_kv_heads, s);
  return head_dim == 128 ? launch_prefill<F16, 128>(a, n_kv_heads, s)
                         : launch_prefill<F16, 64>(a, n_kv_heads, s);
}
