// Shared helpers for the gfx950 kernels of libdramattn.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/dram_attention_amd.h"

namespace da {

// ---- error reporting -------------------------------------------------------

char *last_error_buffer();  // thread-local, 256 bytes (defined in api.hip)

inline int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(last_error_buffer(), 256, fmt, ap);
  va_end(ap);
  return code;
}

inline int launch_status(const char *what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail((int)e, "%s: %s", what, hipGetErrorString(e));
  return DA_OK;
}

#define DA_REQUIRE(cond, ...) \
  do {                        \
    if (!(cond)) return ::da::fail(DA_EINVAL, __VA_ARGS__); \
  } while (0)

inline bool is_pow2(int64_t v) { return v > 0 && (v & (v - 1)) == 0; }
inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline int elem_size(int dtype) { return dtype == DA_F32 ? 4 : 2; }

// ---- element types ---------------------------------------------------------

struct F32 {
  static constexpr int kBytes = 4;
  static constexpr int kVec = 4;  // elements per 16-byte lane load
};
struct F16 {
  static constexpr int kBytes = 2;
  static constexpr int kVec = 8;
};
struct BF16 {
  static constexpr int kBytes = 2;
  static constexpr int kVec = 8;
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

// Reinterpreting helpers take their operand BY VALUE: __builtin_bit_cast applied
// directly to a vector subscript (v[i]) reads element 0 with this compiler.
__device__ __forceinline__ float as_f32(uint32_t w) { return __builtin_bit_cast(float, w); }
__device__ __forceinline__ bf16x2 as_bf16x2(uint32_t w) { return __builtin_bit_cast(bf16x2, w); }
__device__ __forceinline__ f16x2 as_f16x2(uint32_t w) { return __builtin_bit_cast(f16x2, w); }

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) {
  return __builtin_bit_cast(float, bits16 << 16);
}
// Two bf16 packed in one dword: element 0 in the low half.
__device__ __forceinline__ float bf16_lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) {
  return __builtin_bit_cast(float, w & 0xffff0000u);
}
__device__ __forceinline__ float f16_lo(uint32_t w) {
  return (float)__builtin_bit_cast(f16x2, w)[0];
}
__device__ __forceinline__ float f16_hi(uint32_t w) {
  return (float)__builtin_bit_cast(f16x2, w)[1];
}
// Round-to-nearest-even to bf16 and back (one v_cvt_pk_bf16_f32 on gfx950).
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  bf16x2 r;
  r[0] = (__bf16)lo;
  r[1] = (__bf16)hi;
  return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ uint32_t pack_f16(float lo, float hi) {
  f16x2 r;
  r[0] = (_Float16)lo;
  r[1] = (_Float16)hi;
  return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ float round_bf16(float x) {
  return (float)(__bf16)x;
}
__device__ __forceinline__ float round_f16(float x) { return (float)(_Float16)x; }

template <typename T>
__device__ __forceinline__ float round_to(float x);
template <>
__device__ __forceinline__ float round_to<F32>(float x) { return x; }
template <>
__device__ __forceinline__ float round_to<F16>(float x) { return round_f16(x); }
template <>
__device__ __forceinline__ float round_to<BF16>(float x) { return round_bf16(x); }

// Scalar element load / store by index (generic, slow paths).
template <typename T>
__device__ __forceinline__ float load_elem(const void *base, int64_t i);
template <>
__device__ __forceinline__ float load_elem<F32>(const void *base, int64_t i) {
  return ((const float *)base)[i];
}
template <>
__device__ __forceinline__ float load_elem<F16>(const void *base, int64_t i) {
  return (float)((const _Float16 *)base)[i];
}
template <>
__device__ __forceinline__ float load_elem<BF16>(const void *base, int64_t i) {
  return bf16_bits_to_f32(((const uint16_t *)base)[i]);
}
template <typename T>
__device__ __forceinline__ void store_elem(void *base, int64_t i, float v);
template <>
__device__ __forceinline__ void store_elem<F32>(void *base, int64_t i, float v) {
  ((float *)base)[i] = v;
}
template <>
__device__ __forceinline__ void store_elem<F16>(void *base, int64_t i, float v) {
  ((_Float16 *)base)[i] = (_Float16)v;
}
template <>
__device__ __forceinline__ void store_elem<BF16>(void *base, int64_t i, float v) {
  ((__bf16 *)base)[i] = (__bf16)v;
}

// Unpack one 16-byte lane load into kVec floats.
template <typename T>
__device__ __forceinline__ void unpack(const u32x4 &v, float *f);
template <>
__device__ __forceinline__ void unpack<F32>(const u32x4 &v, float *f) {
#pragma unroll
  for (int i = 0; i < 4; ++i) f[i] = as_f32(v[i]);
}
template <>
__device__ __forceinline__ void unpack<F16>(const u32x4 &v, float *f) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = f16_lo(v[i]);
    f[2 * i + 1] = f16_hi(v[i]);
  }
}
template <>
__device__ __forceinline__ void unpack<BF16>(const u32x4 &v, float *f) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = bf16_lo(v[i]);
    f[2 * i + 1] = bf16_hi(v[i]);
  }
}

__device__ __forceinline__ u32x4 load16(const void *p) { return *(const u32x4 *)p; }
// The same load marked as streaming: the data will not be read again soon.
__device__ __forceinline__ u32x4 load16_stream(const void *p) {
  return __builtin_nontemporal_load((const u32x4 *)p);
}
__device__ __forceinline__ void store16(void *p, const u32x4 &v) { *(u32x4 *)p = v; }
__device__ __forceinline__ void store16_stream(void *p, const u32x4 &v) {
  __builtin_nontemporal_store(v, (u32x4 *)p);
}

// Sum over groups of `width` adjacent lanes (width a power of two <= 64);
// every lane of a group ends with the group's total.
// The first four folding steps stay inside a 16-lane row and ride on the
// adder as DPP operand swizzles (quad permutes, then half-row and row
// mirrors, which pair up lanes that already hold equal partial sums).
template <int kCtrl>
__device__ __forceinline__ float dpp_swizzle(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), kCtrl, 0xf, 0xf, false));
}
template <int kWidth>
__device__ __forceinline__ float group_sum(float v) {
  if (kWidth >= 2) v += dpp_swizzle<0xB1>(v);   // quad_perm [1,0,3,2]
  if (kWidth >= 4) v += dpp_swizzle<0x4E>(v);   // quad_perm [2,3,0,1]
  if (kWidth >= 8) v += dpp_swizzle<0x141>(v);  // row_half_mirror
  if (kWidth >= 16) v += dpp_swizzle<0x140>(v); // row_mirror
  if (kWidth >= 32) v += __shfl_xor(v, 16, 64);
  if (kWidth >= 64) v += __shfl_xor(v, 32, 64);
  return v;
}
template <int kWidth>
__device__ __forceinline__ float group_max(float v) {
#pragma unroll
  for (int m = kWidth / 2; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, 64));
  return v;
}

// Order-preserving map float -> uint32 (larger float <=> larger key).
// -0.0 and +0.0 map to the same key; every NaN maps above +inf.
__device__ __forceinline__ uint32_t float_order_key(float x) {
  if (x != x) return 0xffffffffu;
  uint32_t b = __builtin_bit_cast(uint32_t, x);
  if (b == 0x80000000u) b = 0u;
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

}  // namespace da
