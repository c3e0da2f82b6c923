// LayerNorm (no affine) fused with the adaLN-single modulation, for gfx950:
//
//   out[b, n, :] = LN(x[b, n, :]) * (1 + scale[b, :]) + shift[b, :]
//
// HBM bound: one read and one write of the activation (2 * M * C * 2 bytes).  A second form takes the
// residual sum in front of the norm along: sum = x + y is computed, stored and normalised in one pass
// (2 reads + 2 writes instead of the 3 + 2 of a separate add).
// One wave per token row; the row lives in registers as raw 16-byte chunks
// (lane l holds chunks l, l+64, ...), so it is read from memory once: mean and
// the centred variance are two register passes with wave reductions, the third
// pass normalises, modulates and stores.  The four roundings of the stock op
// chain (layer_norm -> 1+scale -> product -> +shift, each a bf16 tensor) are
// reproduced in registers.
#include "common.h"

// No implicit fused multiply-adds in this file: the epilogues reproduce the stock op chain's roundings (product
// rounded to the io dtype, THEN the sum), and for fp16 -- which has native arithmetic -- the compiler would otherwise
// contract "round(g * y) + r" into one v_fma_f16 and drop the product's rounding.  Wanted fmas are written as fmaf.
#pragma clang fp contract(off)

#ifndef SANA_LN_NT_LOAD
#define SANA_LN_NT_LOAD 0
#endif
#ifndef SANA_LN_NT_STORE
#define SANA_LN_NT_STORE 0
#endif

namespace sana {
namespace {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// NCH: 16-byte chunks per lane (C <= 512 * NCH).  ADD: the row is x + y (rounded to bf16, as the stock add
// stores it) and is written to `sum` as well: the residual update in front of the norm, in the same pass.
template <int NCH, bool ADD, typename T>
__global__ __launch_bounds__(256) void ln_modulate_kernel(const uint16_t* __restrict__ x,
                                                          const uint16_t* __restrict__ y,
                                                          const uint16_t* __restrict__ scale,
                                                          const uint16_t* __restrict__ shift,
                                                          uint16_t* __restrict__ sum,
                                                          uint16_t* __restrict__ out, int64_t M, int C,
                                                          int64_t ldx, int64_t ldy, int64_t lds, int64_t ldo,
                                                          int rows_per_mod, int64_t mod_stride, float eps) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + wave;
  if (row >= M) return;  // no barriers in this kernel
  const int nchunks = C >> 3;
  const uint16_t* xr = x + row * ldx;
  u32x4_t raw[NCH];
  const u32x4_t zero4 = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int ch = lane + 64 * i;
    raw[i] = ch < nchunks ? load_stream<SANA_LN_NT_LOAD != 0>(reinterpret_cast<const u32x4_t*>(xr + 8 * ch)) : zero4;
  }
  if (ADD) {
    const uint16_t* yr = y + row * ldy;
    uint16_t* sr = sum + row * lds;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int ch = lane + 64 * i;
      if (ch < nchunks) {
        const u32x4_t b = load_stream<SANA_LN_NT_LOAD != 0>(reinterpret_cast<const u32x4_t*>(yr + 8 * ch));
#pragma unroll
        for (int e = 0; e < 4; ++e)
          raw[i][e] = pk16<T>(lo16<T>(raw[i][e]) + lo16<T>(b[e]), hi16<T>(raw[i][e]) + hi16<T>(b[e]));
        store_stream<SANA_LN_NT_STORE != 0>(raw[i], reinterpret_cast<u32x4_t*>(sr + 8 * ch));
      }
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; ++i)
#pragma unroll
    for (int e = 0; e < 4; ++e) s += lo16<T>(raw[i][e]) + hi16<T>(raw[i][e]);
  const float mean = wave_sum(s) / (float)C;
  float v = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    if (lane + 64 * i < nchunks) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float a = lo16<T>(raw[i][e]) - mean, b = hi16<T>(raw[i][e]) - mean;
        v = fmaf(a, a, v);
        v = fmaf(b, b, v);
      }
    }
  }
  const float rstd = rsqrtf(wave_sum(v) / (float)C + eps);
  const int64_t mod = (row / rows_per_mod) * mod_stride;
  uint16_t* orow = out + row * ldo;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int ch = lane + 64 * i;
    if (ch < nchunks) {
      const u32x4_t sc = *reinterpret_cast<const u32x4_t*>(scale + mod + 8 * ch);
      const u32x4_t sh = *reinterpret_cast<const u32x4_t*>(shift + mod + 8 * ch);
      u32x4_t o;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint32_t ln = pk16<T>((lo16<T>(raw[i][e]) - mean) * rstd, (hi16<T>(raw[i][e]) - mean) * rstd);
        const uint32_t s1 = pk16<T>(1.0f + lo16<T>(sc[e]), 1.0f + hi16<T>(sc[e]));
        const uint32_t t = pk16<T>(lo16<T>(ln) * lo16<T>(s1), hi16<T>(ln) * hi16<T>(s1));
        o[e] = pk16<T>(lo16<T>(t) + lo16<T>(sh[e]), hi16<T>(t) + hi16<T>(sh[e]));
      }
      store_stream<SANA_LN_NT_STORE != 0>(o, reinterpret_cast<u32x4_t*>(orow + 8 * ch));
    }
  }
}

// out = res + gate[row / rows_per_gate] * y with the two roundings of the stock op pair (product, then sum):
// the gated residual update behind a module whose last op is not one of this library's GEMMs.  One thread per
// 8 channels; three streams (y, res, out), HBM bound.
template <typename T>
__global__ __launch_bounds__(256) void gate_residual_kernel(const uint16_t* __restrict__ y,
                                                            const uint16_t* __restrict__ gate,
                                                            const uint16_t* __restrict__ res,
                                                            uint16_t* __restrict__ out, int64_t M, int C, int64_t ldy,
                                                            int64_t ldr, int64_t ldo, int rows_per_gate,
                                                            int64_t gate_stride) {
  const int chunks = C >> 3;
  const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (id >= M * chunks) return;
  const int64_t m = id / chunks;
  const int n = (int)(id - m * chunks) * 8;
  const u32x4_t yv = load_stream<SANA_LN_NT_LOAD != 0>(reinterpret_cast<const u32x4_t*>(y + m * ldy + n));
  const u32x4_t rv = load_stream<SANA_LN_NT_LOAD != 0>(reinterpret_cast<const u32x4_t*>(res + m * ldr + n));
  const u32x4_t gv = *reinterpret_cast<const u32x4_t*>(gate + (m / rows_per_gate) * gate_stride + n);
  u32x4_t o;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const uint32_t t = pk16<T>(lo16<T>(gv[e]) * lo16<T>(yv[e]), hi16<T>(gv[e]) * hi16<T>(yv[e]));
    o[e] = pk16<T>(lo16<T>(rv[e]) + lo16<T>(t), hi16<T>(rv[e]) + hi16<T>(t));
  }
  store_stream<SANA_LN_NT_STORE != 0>(o, reinterpret_cast<u32x4_t*>(out + m * ldo + n));
}

}  // namespace
}  // namespace sana

using namespace sana;

template <bool ADD>
static int ln_impl(const void* x, const void* y, const void* scale, const void* shift, void* sum, void* out, int64_t M,
                   int C, int64_t ldx, int64_t ldy, int64_t lds, int64_t ldo, int rows_per_mod, int64_t mod_stride,
                   float eps, int io_dtype, void* stream) {
  if (!x || !scale || !shift || !out || M <= 0 || C <= 0 || rows_per_mod <= 0) return SANA_ERR_ARG;
  if (ADD && (!y || !sum)) return SANA_ERR_ARG;
  if (io_dtype != SANA_DT_BF16 && io_dtype != SANA_DT_F16) return SANA_ERR_DTYPE;
  if (C % 8 || C > 8192) return SANA_ERR_SHAPE;
  if (ldx < C || ldo < C || mod_stride < 0 || (ADD && (ldy < C || lds < C))) return SANA_ERR_ARG;
  if (ldx % 8 || ldo % 8 || mod_stride % 8 || !aligned16(x) || !aligned16(out) || !aligned16(scale) ||
      !aligned16(shift))
    return SANA_ERR_ALIGN;
  if (ADD && (ldy % 8 || lds % 8 || !aligned16(y) || !aligned16(sum))) return SANA_ERR_ALIGN;
  if ((M + 3) / 4 > 0x7fffffff) return SANA_ERR_SHAPE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid((unsigned)((M + 3) / 4)), block(256);
  const uint16_t* xp = static_cast<const uint16_t*>(x);
  const uint16_t* yp = static_cast<const uint16_t*>(y);
  const uint16_t* sc = static_cast<const uint16_t*>(scale);
  const uint16_t* sh = static_cast<const uint16_t*>(shift);
  uint16_t* sp = static_cast<uint16_t*>(sum);
  uint16_t* op = static_cast<uint16_t*>(out);
  const int nch = (C / 8 + 63) / 64;
#define SANA_LN(NCH)                                                                                          \
  do {                                                                                                        \
    if (io_dtype == SANA_DT_F16)                                                                              \
      hipLaunchKernelGGL((ln_modulate_kernel<NCH, ADD, F16>), grid, block, 0, s, xp, yp, sc, sh, sp, op, M, C, \
                         ldx, ldy, lds, ldo, rows_per_mod, mod_stride, eps);                                  \
    else                                                                                                      \
      hipLaunchKernelGGL((ln_modulate_kernel<NCH, ADD, BF16>), grid, block, 0, s, xp, yp, sc, sh, sp, op, M, C, \
                         ldx, ldy, lds, ldo, rows_per_mod, mod_stride, eps);                                  \
  } while (0)
  if (nch <= 2) SANA_LN(2);
  else if (nch <= 3) SANA_LN(3);
  else if (nch <= 5) SANA_LN(5);
  else if (nch <= 8) SANA_LN(8);
  else SANA_LN(16);
#undef SANA_LN
  return hipGetLastError() == hipSuccess ? SANA_OK : SANA_ERR_LAUNCH;
}

extern "C" __attribute__((visibility("default"))) int sana_hip_layernorm_modulate(
    const void* x, const void* scale, const void* shift, void* out, int64_t M, int C, int64_t ldx, int64_t ldo,
    int rows_per_mod, int64_t mod_stride, float eps, int io_dtype, void* stream) {
  return ln_impl<false>(x, nullptr, scale, shift, nullptr, out, M, C, ldx, 0, 0, ldo, rows_per_mod, mod_stride, eps,
                        io_dtype, stream);
}

extern "C" __attribute__((visibility("default"))) int sana_hip_add_layernorm_modulate(
    const void* x, const void* y, const void* scale, const void* shift, void* sum, void* out, int64_t M, int C,
    int64_t ldx, int64_t ldy, int64_t lds, int64_t ldo, int rows_per_mod, int64_t mod_stride, float eps, int io_dtype,
    void* stream) {
  return ln_impl<true>(x, y, scale, shift, sum, out, M, C, ldx, ldy, lds, ldo, rows_per_mod, mod_stride, eps, io_dtype,
                       stream);
}

extern "C" __attribute__((visibility("default"))) int sana_hip_gate_residual(
    const void* y, const void* gate, const void* residual, void* out, int64_t M, int C, int64_t ldy, int64_t ldr,
    int64_t ldo, int rows_per_gate, int64_t gate_stride, int io_dtype, void* stream) {
  if (!y || !gate || !residual || !out || M <= 0 || C <= 0 || rows_per_gate <= 0) return SANA_ERR_ARG;
  if (io_dtype != SANA_DT_BF16 && io_dtype != SANA_DT_F16) return SANA_ERR_DTYPE;
  if (C % 8) return SANA_ERR_SHAPE;
  if (ldy < C || ldr < C || ldo < C || gate_stride < 0) return SANA_ERR_ARG;
  if (ldy % 8 || ldr % 8 || ldo % 8 || gate_stride % 8 || !aligned16(y) || !aligned16(gate) || !aligned16(residual) ||
      !aligned16(out))
    return SANA_ERR_ALIGN;
  const int64_t threads = M * (C / 8);
  if ((threads + 255) / 256 > 0x7fffffff) return SANA_ERR_SHAPE;
  const dim3 grid((unsigned)((threads + 255) / 256)), block(256);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (io_dtype == SANA_DT_F16)
    hipLaunchKernelGGL(gate_residual_kernel<F16>, grid, block, 0, s, static_cast<const uint16_t*>(y),
                       static_cast<const uint16_t*>(gate), static_cast<const uint16_t*>(residual),
                       static_cast<uint16_t*>(out), M, C, ldy, ldr, ldo, rows_per_gate, gate_stride);
  else
    hipLaunchKernelGGL(gate_residual_kernel<BF16>, grid, block, 0, s, static_cast<const uint16_t*>(y),
                       static_cast<const uint16_t*>(gate), static_cast<const uint16_t*>(residual),
                       static_cast<uint16_t*>(out), M, C, ldy, ldr, ldo, rows_per_gate, gate_stride);
  return hipGetLastError() == hipSuccess ? SANA_OK : SANA_ERR_LAUNCH;
}
