// Shared device helpers for the gfx950 kernels (wave64, MFMA, bf16/f16 bit tricks).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/sana_hip.h"

namespace sana {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef short s16x2_t __attribute__((ext_vector_type(2)));

struct BF16 {};  // tag types for the 16-bit io dtypes
struct F16 {};

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }
__device__ __forceinline__ float bf16_lo(uint32_t packed) { return __uint_as_float(packed << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t packed) { return __uint_as_float(packed & 0xffff0000u); }

// round-to-nearest-even fp32 -> bf16 bits (NaN stays NaN)
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  __bf16 b = (__bf16)f;
  return (uint32_t)__builtin_bit_cast(uint16_t, b);
}
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  // one v_cvt_pk_bf16_f32 (round-to-nearest-even on both halves)
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
__device__ __forceinline__ float round_bf16(float f) { return bf16_bits_to_f32(f32_to_bf16_bits(f)); }

__device__ __forceinline__ float f16_bits_to_f32(uint32_t bits16) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)bits16);
}
__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
  _Float16 h = (_Float16)f;
  return (uint32_t)__builtin_bit_cast(uint16_t, h);
}
__device__ __forceinline__ uint32_t pack_f16(float lo, float hi) {
  return f32_to_f16_bits(lo) | (f32_to_f16_bits(hi) << 16);
}

// Conversions of the two 16-bit io dtypes by tag (T = BF16 or F16): pack two floats with round-to-nearest-even (one
// v_cvt_pk_bf16_f32 for bf16; two conversions and a pack for f16, which has no packed round-to-nearest conversion),
// unpack either half of a packed pair, round through the dtype.
template <typename T> inline constexpr bool is_f16 = false;
template <> inline constexpr bool is_f16<F16> = true;
template <typename T> __device__ __forceinline__ uint32_t pk16(float lo, float hi) {
  if constexpr (is_f16<T>) return pack_f16(lo, hi);
  else return pack_bf16(lo, hi);
}
template <typename T> __device__ __forceinline__ float lo16(uint32_t p) {
  if constexpr (is_f16<T>) return f16_bits_to_f32(p & 0xffffu);
  else return bf16_lo(p);
}
template <typename T> __device__ __forceinline__ float hi16(uint32_t p) {
  if constexpr (is_f16<T>) return f16_bits_to_f32(p >> 16);
  else return bf16_hi(p);
}
template <typename T> __device__ __forceinline__ float rnd16(float f) {
  // (through the bit pattern: a float -> _Float16 -> float cast pair alone may be evaluated in excess precision,
  // i.e. not round at all)
  if constexpr (is_f16<T>) return f16_bits_to_f32(f32_to_f16_bits(f));
  else return round_bf16(f);
}

// ReLU on two packed 16-bit floats (bf16 or f16: both sign-magnitude, so a
// signed-integer max against 0 clears negatives and -0).
__device__ __forceinline__ uint32_t relu_pk16(uint32_t x) {
  s16x2_t v = __builtin_bit_cast(s16x2_t, x);
  s16x2_t z = {0, 0};
  return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(v, z));
}
__device__ __forceinline__ u32x4_t relu_pk16(u32x4_t x) {
  u32x4_t r;
  r.x = relu_pk16(x.x);
  r.y = relu_pk16(x.y);
  r.z = relu_pk16(x.z);
  r.w = relu_pk16(x.w);
  return r;
}

template <typename T>
__device__ __forceinline__ f32x16_t mfma_32x32x16(u32x4_t a, u32x4_t b, f32x16_t c);
template <>
__device__ __forceinline__ f32x16_t mfma_32x32x16<BF16>(u32x4_t a, u32x4_t b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}
template <>
__device__ __forceinline__ f32x16_t mfma_32x32x16<F16>(u32x4_t a, u32x4_t b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
}
__device__ __forceinline__ f32x4_t mfma_16x16x32_bf16(u32x4_t a, u32x4_t b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

// acc + lo(x) + hi(x) for two packed 16-bit floats: one dot2 against (1, 1), fp32 accumulate
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
template <typename T>
__device__ __forceinline__ float add_pk16(uint32_t x, float acc);
template <>
__device__ __forceinline__ float add_pk16<BF16>(uint32_t x, float acc) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, x), __builtin_bit_cast(bf16x2_t, 0x3f803f80u), acc,
                                         false);
}
template <>
__device__ __forceinline__ float add_pk16<F16>(uint32_t x, float acc) {
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, x), __builtin_bit_cast(f16x2_t, 0x3c003c00u), acc, false);
}

__device__ __forceinline__ float silu_f32(float g) {
  // g * sigmoid(g) = g / (1 + exp(-g)); exp via the hardware exp2
  return g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504088896341f * g));
}

// Streaming accesses.  The non-temporal hint keeps data that is touched once from displacing reusable lines in the
// L2 and spares the write path its allocate traffic: a 2-reads-1-write stream of 552 MB runs at 6.6 TB/s with the
// hint on loads and stores and at 5.8 TB/s without on MI355X.  Whether a kernel of the block should use it depends
// on its neighbours: an output that the next kernel reads is better left cacheable (the 256 MB Infinity Cache
// then serves that read), and inputs a producer has just written are found there.  Each kernel therefore names
// its own policy (the SANA_*_NT_* knobs of its source file); these helpers only carry it out.
template <bool NT, typename V>
__device__ __forceinline__ V load_stream(const V* p) {
  if constexpr (NT) return __builtin_nontemporal_load(p);
  else return *p;
}
template <bool NT, typename V>
__device__ __forceinline__ void store_stream(V v, V* p) {
  if constexpr (NT) __builtin_nontemporal_store(v, p);
  else *p = v;
}
template <bool NT>
__device__ __forceinline__ void store_stream(float2 v, float2* p) {
  store_stream<NT>(f32x2_t{v.x, v.y}, reinterpret_cast<f32x2_t*>(p));
}
constexpr int kBufferNt = 2;  // cache-policy operand of the buffer load / store intrinsics: bit 1 = non-temporal

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace sana
