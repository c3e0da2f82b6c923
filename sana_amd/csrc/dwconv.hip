// Depthwise 3x3 (zero pad 1) + bias + SiLU gate, channels-last, for gfx950.
//
//   u [BT][H][W][2*Ch] -> y [BT][H][W][Ch],  y[c] = t[c] * silu(t[Ch+c]),
//   t[c] = bias[c] + sum_taps u[..][c] * w[c][tap]
//
// HBM-bound (no reuse across channels; 9-fold reuse across pixels).  Lanes run
// along the channel axis: a lane owns the channel pair (c, c+1) of the first
// half and (Ch+c, Ch+c+1) of the gate half, so a wave reads 256 contiguous
// bytes per pixel and half.  A wave walks DOWN a strip of TW output columns
// holding a rolling 3 x (TW+2) pixel window in fp32 registers: every input
// element is loaded once per strip (plus the two halo columns) and converted
// once; the next row's loads are in flight while the current row is computed.
// The four waves of a workgroup take four adjacent strips so that the halo
// columns hit in the CU's vector L1.
#include <type_traits>

#include "common.h"

#ifndef SANA_DW_MINWAVES
#define SANA_DW_MINWAVES 6144  // split rows into bands until the launch has at least this many waves
#endif
#ifndef SANA_DW_TW
#define SANA_DW_TW 4  // output columns per wave strip (tuning knob: register window is 3 x (TW+2) pixels)
#endif

namespace sana {
namespace {

template <typename T>
struct Pair;  // two adjacent channels
template <>
struct Pair<BF16> {
  typedef uint32_t raw;
  static __device__ __forceinline__ raw load(const void* p, int64_t elem) {
    return *reinterpret_cast<const uint32_t*>(static_cast<const uint16_t*>(p) + elem);
  }
  static __device__ __forceinline__ float lo(raw r) { return bf16_lo(r); }
  static __device__ __forceinline__ float hi(raw r) { return bf16_hi(r); }
  static __device__ __forceinline__ float one(const void* p, int64_t elem) {
    return bf16_bits_to_f32(static_cast<const uint16_t*>(p)[elem]);
  }
  static __device__ __forceinline__ raw pack(float a, float b) { return pack_bf16(a, b); }
  static __device__ __forceinline__ void rnd2(float a, float b, float& ra, float& rb) {
    const raw r = pack_bf16(a, b);  // one packed convert rounds both
    ra = lo(r);
    rb = hi(r);
  }
};
template <>
struct Pair<F16> {
  typedef uint32_t raw;
  static __device__ __forceinline__ raw load(const void* p, int64_t elem) {
    return *reinterpret_cast<const uint32_t*>(static_cast<const uint16_t*>(p) + elem);
  }
  static __device__ __forceinline__ float lo(raw r) { return f16_bits_to_f32(r & 0xffffu); }
  static __device__ __forceinline__ float hi(raw r) { return f16_bits_to_f32(r >> 16); }
  static __device__ __forceinline__ float one(const void* p, int64_t elem) {
    return f16_bits_to_f32(static_cast<const uint16_t*>(p)[elem]);
  }
  static __device__ __forceinline__ raw pack(float a, float b) { return pack_f16(a, b); }
  static __device__ __forceinline__ void rnd2(float a, float b, float& ra, float& rb) {
    const raw r = pack_f16(a, b);
    ra = lo(r);
    rb = hi(r);
  }
};
template <>
struct Pair<float> {
  typedef float2 raw;
  static __device__ __forceinline__ raw load(const void* p, int64_t elem) {
    return *reinterpret_cast<const float2*>(static_cast<const float*>(p) + elem);
  }
  static __device__ __forceinline__ float lo(raw r) { return r.x; }
  static __device__ __forceinline__ float hi(raw r) { return r.y; }
  static __device__ __forceinline__ float one(const void* p, int64_t elem) { return static_cast<const float*>(p)[elem]; }
  static __device__ __forceinline__ raw pack(float a, float b) { return make_float2(a, b); }
  static __device__ __forceinline__ void rnd2(float a, float b, float& ra, float& rb) {
    ra = a;
    rb = b;
  }
};

// grid: x = channel slabs of 128 (fastest: neighbouring workgroups read neighbouring 256-byte
// pieces of the same pixels), y = x-groups (4 strips) * row bands, z = BT; block 256.  Remapping
// workgroups so that halo neighbours share an XCD's L2 lowers the HBM fetch size (measured 1.56x ->
// 1.25x of the algorithmic bytes) but runs slower: the kernel is co-limited by the vector ALU.
//
// Everything except the channel offset of a lane is wave-uniform, so pixel addresses are formed on
// the scalar unit (uniform 64-bit base + one constant 32-bit lane offset) and image-border handling
// is a uniform branch: rows whose whole (TW+2)-pixel footprint is inside the image take a path with
// no per-element selects.
template <typename T, int TW, bool ROUND>
__global__ __launch_bounds__(256) void dwconv_gate_kernel(const void* __restrict__ u, const void* __restrict__ w,
                                                          const void* __restrict__ bias, void* __restrict__ y,
                                                          int H, int W, int Ch, int R, int xgroups) {
  typedef Pair<T> P;
  typedef typename P::raw raw_t;
  constexpr int ESZ = sizeof(raw_t) / 2;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  // Workgroup ids are dealt round-robin to the 8 XCDs (own L2 each).  Position p in a grid row goes to
  // XCD p % 8; give each XCD a run of CONSECUTIVE slabs: the gate half of a pixel starts Ch*2 bytes in,
  // which is not a multiple of 128 in general, so neighbouring slabs share a 128-byte line there and
  // now meet in one L2 instead of fetching it from HBM twice.
  int slab;
  {
    const int nsl = gridDim.x, q = nsl >> 3, r = nsl & 7, k = blockIdx.x & 7, j = blockIdx.x >> 3;
    slab = (k < r ? k * (q + 1) : r * (q + 1) + (k - r) * q) + j;
  }
  const int bt = blockIdx.z;
  const int xg = blockIdx.y % xgroups, band = blockIdx.y / xgroups;
  const int c = slab * 128 + 2 * lane;
  const int x0 = (xg * 4 + wave) * TW;
  if (c >= Ch || x0 >= W) return;  // no barriers in this kernel
  const int y0 = band * R, y1 = min(H, y0 + R);
  const int64_t C2 = 2 * (int64_t)Ch;
  const int64_t img = (int64_t)bt * H * W;
  const uint32_t lane_b = (uint32_t)(2 * lane) * ESZ;  // the only per-lane part of an address
  const char* ub = static_cast<const char*>(u) + (int64_t)slab * 128 * ESZ;
  char* yb = static_cast<char*>(y) + (int64_t)slab * 128 * ESZ;
  const int64_t g_off = (int64_t)Ch * ESZ;  // gate half of a pixel

  // filter taps and bias for the four channels of this lane: [a0, a1, g0, g1]
  float wt[4][9], bs[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int ch = c + (q & 1) + (q >> 1) * Ch;
#pragma unroll
    for (int t = 0; t < 9; ++t) wt[q][t] = P::one(w, (int64_t)ch * 9 + t);
    bs[q] = bias ? P::one(bias, ch) : 0.f;
  }

  float win[3][TW + 2][4];
  raw_t ra[TW + 2], rg[TW + 2];
  bool rowok = false;
  const bool cols_inside = x0 >= 1 && x0 + TW <= W - 1;  // footprint columns x0-1 .. x0+TW all in the image

  // loads always hit a valid (clamped) address; out-of-image taps are zeroed at commit
  auto issue = [&](int yy) {
    rowok = yy >= 0 && yy < H && yy <= y1;  // rows past the band's lower halo are never used
    const int yc = min(max(yy, 0), H - 1);
    const char* rowp = ub + (img + (int64_t)yc * W) * C2 * ESZ;
#pragma unroll
    for (int i = 0; i < TW + 2; ++i) {
      const int xc = min(max(x0 - 1 + i, 0), W - 1);
      const char* pix = rowp + (int64_t)xc * C2 * ESZ;
      ra[i] = *reinterpret_cast<const raw_t*>(pix + lane_b);
      rg[i] = *reinterpret_cast<const raw_t*>(pix + g_off + lane_b);
    }
  };
  auto commit = [&](float (&row)[TW + 2][4]) {
    if (rowok && cols_inside) {
#pragma unroll
      for (int i = 0; i < TW + 2; ++i) {
        row[i][0] = P::lo(ra[i]);
        row[i][1] = P::hi(ra[i]);
        row[i][2] = P::lo(rg[i]);
        row[i][3] = P::hi(rg[i]);
      }
    } else {
#pragma unroll
      for (int i = 0; i < TW + 2; ++i) {
        const bool ok = rowok && (x0 - 1 + i >= 0) && (x0 - 1 + i < W);
        row[i][0] = ok ? P::lo(ra[i]) : 0.f;
        row[i][1] = ok ? P::hi(ra[i]) : 0.f;
        row[i][2] = ok ? P::lo(rg[i]) : 0.f;
        row[i][3] = ok ? P::hi(rg[i]) : 0.f;
      }
    }
  };
  auto compute = [&](int yo, const float (&top)[TW + 2][4], const float (&mid)[TW + 2][4],
                     const float (&bot)[TW + 2][4]) {
    char* orow = yb + (img + (int64_t)yo * W + x0) * Ch * ESZ;
#pragma unroll
    for (int x = 0; x < TW; ++x) {
      if (x0 + x >= W) break;
      float acc[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float a = bs[q];
#pragma unroll
        for (int dx = 0; dx < 3; ++dx) {
          a = fmaf(top[x + dx][q], wt[q][dx], a);
          a = fmaf(mid[x + dx][q], wt[q][3 + dx], a);
          a = fmaf(bot[x + dx][q], wt[q][6 + dx], a);
        }
        acc[q] = a;
      }
      float o0, o1;
      if (ROUND) {
        // the reference rounds after the conv, after SiLU and after the product
        float a0, a1, g0, g1, s0, s1;
        P::rnd2(acc[0], acc[1], a0, a1);
        P::rnd2(acc[2], acc[3], g0, g1);
        P::rnd2(silu_f32(g0), silu_f32(g1), s0, s1);
        o0 = a0 * s0;
        o1 = a1 * s1;
      } else {
        o0 = acc[0] * silu_f32(acc[2]);
        o1 = acc[1] * silu_f32(acc[3]);
      }
      *reinterpret_cast<raw_t*>(orow + (int64_t)x * Ch * ESZ + lane_b) = P::pack(o0, o1);
    }
  };

  // prologue: rows y0-1 and y0 in the window, row y0+1 in flight
  issue(y0 - 1);
  commit(win[0]);
  issue(y0);
  commit(win[1]);
  issue(y0 + 1);
  for (int yo = y0; yo < y1; yo += 3) {
    // sub-step s: window rows (top, mid, bot) = win[s], win[s+1], win[s+2] (mod 3)
    commit(win[2]);
    issue(yo + 2);
    compute(yo, win[0], win[1], win[2]);
    if (yo + 1 >= y1) break;
    commit(win[0]);
    issue(yo + 3);
    compute(yo + 1, win[1], win[2], win[0]);
    if (yo + 2 >= y1) break;
    commit(win[1]);
    issue(yo + 4);
    compute(yo + 2, win[2], win[0], win[1]);
  }
}

// ----------------------------------------------------------------------------
// 16-bit io: the taps run on packed dot products.  The window keeps, per row, channel and column j,
// the PAIR (x[j], x[j+1]) as two 16-bit values in one register (built with one byte-permute from the
// loaded channel-pair words of pixels j and j+1), and a 3-tap row is
//   dot2(pair[j], (w0, w1)) + dot2(pair[j+2], (w2, 0))
// with fp32 accumulation: 6 instructions per output channel instead of 9 FMAs, and no unpacking of
// the inputs at all (products of 16-bit values are exact in fp32).
// ----------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ float dot2_16(uint32_t a, uint32_t b, float c);
template <>
__device__ __forceinline__ float dot2_16<BF16>(uint32_t a, uint32_t b, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), c, false);
}
template <>
__device__ __forceinline__ float dot2_16<F16>(uint32_t a, uint32_t b, float c) {
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, a), __builtin_bit_cast(f16x2_t, b), c, false);
}

template <typename T, int TW, bool ROUND>
__global__ __launch_bounds__(256) void dwconv_gate16_kernel(const void* __restrict__ u, const void* __restrict__ w,
                                                            const void* __restrict__ bias, void* __restrict__ y,
                                                            int H, int W, int Ch, int R, int xgroups) {
  typedef Pair<T> P;
  constexpr int ESZ = 2;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  // Workgroups go round-robin to the 8 XCDs (own L2 each) in launch order, x fastest.  All slabs of a
  // tile are launched together, so the eight XCDs read the same pixels at the same time -- whole
  // contiguous 2*Ch-element pixel rows, which is what DRAM pages like -- and WHICH slab a workgroup
  // takes is chosen from the XCD it landed on: slab m*q + j for the j-th workgroup of XCD m in this
  // grid row (q = slabs / 8), the slabs left over going to whoever has a (q+1)-th workgroup.  A slab
  // below 8*q is then always served by the same L2, which is where neighbouring tiles find their
  // shared halo rows and columns.  (Giving each XCD its own slabs AND its own run of neighbouring
  // tiles lowers the fetch size further but was measured slower: it breaks up the pixel rows.)
  int slab;
  {
    const int nsl = gridDim.x, q = nsl >> 3;
    const int xcd = (blockIdx.x + nsl * (blockIdx.y + gridDim.y * blockIdx.z)) & 7, j = blockIdx.x >> 3;
    slab = j < q ? xcd * q + j : 8 * q + (blockIdx.x & 7);
  }
  const int bt = blockIdx.z;
  const int xg = blockIdx.y % xgroups, band = blockIdx.y / xgroups;
  const int c = slab * 128 + 2 * lane;
  const int x0 = (xg * 4 + wave) * TW;
  if (c >= Ch || x0 >= W) return;  // no barriers in this kernel
  const int y0 = band * R, y1 = min(H, y0 + R);
  const int64_t C2 = 2 * (int64_t)Ch;
  const int64_t img = (int64_t)bt * H * W;
  const uint32_t lane_b = (uint32_t)(2 * lane) * ESZ;
  const char* ub = static_cast<const char*>(u) + (int64_t)slab * 128 * ESZ;
  char* yb = static_cast<char*>(y) + (int64_t)slab * 128 * ESZ;
  const int64_t g_off = (int64_t)Ch * ESZ;

  // taps of the four channels of this lane [a0, a1, g0, g1], per filter row: (w0, w1) and (w2, 0) packed
  uint32_t w01[4][3], w2z[4][3];
  float bs[4];
  const uint16_t* wp = static_cast<const uint16_t*>(w);
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int64_t ch = c + (q & 1) + (q >> 1) * Ch;
#pragma unroll
    for (int r = 0; r < 3; ++r) {
      w01[q][r] = (uint32_t)wp[ch * 9 + 3 * r] | ((uint32_t)wp[ch * 9 + 3 * r + 1] << 16);
      w2z[q][r] = (uint32_t)wp[ch * 9 + 3 * r + 2];
    }
    bs[q] = bias ? P::one(bias, ch) : 0.f;
  }

  uint32_t win[3][TW + 2][4];  // [row][column j][channel]: (x[j], x[j+1]); the last column pairs with 0
  uint32_t ra[TW + 2], rg[TW + 2];
  bool rowok = false;
  const bool cols_inside = x0 >= 1 && x0 + TW <= W - 1;

  // Buffer loads: the image (this slab's view of it) is one buffer resource in scalar registers, a pixel
  // is a scalar byte offset and the lane's channel pair the vector offset, so no vector ALU work goes
  // into addresses.  One image is below 2 GiB (the host checks).  Addresses are always valid
  // (clamped); the resource's own range check is left wide open.
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(ub + img * C2 * ESZ), 0, -1, 0x00020000);
  const int pix_b = (int)(C2 * ESZ), g_off32 = (int)g_off;
  int coff[TW + 2];  // byte offsets of the (clamped) footprint columns inside a row: scalar registers
#pragma unroll
  for (int i = 0; i < TW + 2; ++i) coff[i] = min(max(x0 - 1 + i, 0), W - 1) * pix_b;
  auto issue = [&](int yy) {
    rowok = yy >= 0 && yy < H && yy <= y1;  // rows past the band's lower halo are never used
    const int rowb = min(max(yy, 0), H - 1) * W * pix_b;
#pragma unroll
    for (int i = 0; i < TW + 2; ++i) {
      ra[i] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)lane_b, rowb + coff[i], 0);
      rg[i] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)lane_b, rowb + coff[i] + g_off32, 0);
    }
  };
  auto commit = [&](uint32_t (&row)[TW + 2][4]) {
    if (!(rowok && cols_inside)) {  // out-of-image taps are zero
#pragma unroll
      for (int i = 0; i < TW + 2; ++i) {
        const bool ok = rowok && (x0 - 1 + i >= 0) && (x0 - 1 + i < W);
        ra[i] = ok ? ra[i] : 0u;
        rg[i] = ok ? rg[i] : 0u;
      }
    }
#pragma unroll
    for (int i = 0; i < TW + 2; ++i) {
      const uint32_t na = i + 1 < TW + 2 ? ra[i + 1] : 0u, ng = i + 1 < TW + 2 ? rg[i + 1] : 0u;
      row[i][0] = __builtin_amdgcn_perm(na, ra[i], 0x05040100u);  // low halves: channel c of pixels i, i+1
      row[i][1] = __builtin_amdgcn_perm(na, ra[i], 0x07060302u);  // high halves: channel c+1
      row[i][2] = __builtin_amdgcn_perm(ng, rg[i], 0x05040100u);
      row[i][3] = __builtin_amdgcn_perm(ng, rg[i], 0x07060302u);
    }
  };
  auto compute = [&](int yo, const uint32_t (&top)[TW + 2][4], const uint32_t (&mid)[TW + 2][4],
                     const uint32_t (&bot)[TW + 2][4]) {
    char* orow = yb + (img + (int64_t)yo * W + x0) * Ch * ESZ;
#pragma unroll
    for (int x = 0; x < TW; ++x) {
      if (x0 + x >= W) break;
      float acc[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float a = bs[q];
        a = dot2_16<T>(top[x][q], w01[q][0], a);
        a = dot2_16<T>(top[x + 2][q], w2z[q][0], a);
        a = dot2_16<T>(mid[x][q], w01[q][1], a);
        a = dot2_16<T>(mid[x + 2][q], w2z[q][1], a);
        a = dot2_16<T>(bot[x][q], w01[q][2], a);
        a = dot2_16<T>(bot[x + 2][q], w2z[q][2], a);
        acc[q] = a;
      }
      float o0, o1;
      if (ROUND) {
        float a0, a1, g0, g1, s0, s1;
        P::rnd2(acc[0], acc[1], a0, a1);
        P::rnd2(acc[2], acc[3], g0, g1);
        P::rnd2(silu_f32(g0), silu_f32(g1), s0, s1);
        o0 = a0 * s0;
        o1 = a1 * s1;
      } else {
        o0 = acc[0] * silu_f32(acc[2]);
        o1 = acc[1] * silu_f32(acc[3]);
      }
      *reinterpret_cast<uint32_t*>(orow + (int64_t)x * Ch * ESZ + lane_b) = P::pack(o0, o1);
    }
  };

  issue(y0 - 1);
  commit(win[0]);
  issue(y0);
  commit(win[1]);
  issue(y0 + 1);
  for (int yo = y0; yo < y1; yo += 3) {
    commit(win[2]);
    issue(yo + 2);
    compute(yo, win[0], win[1], win[2]);
    if (yo + 1 >= y1) break;
    commit(win[0]);
    issue(yo + 3);
    compute(yo + 1, win[1], win[2], win[0]);
    if (yo + 2 >= y1) break;
    commit(win[1]);
    issue(yo + 4);
    compute(yo + 2, win[2], win[0], win[1]);
  }
}

template <typename T, int TW>
int launch(const void* u, const void* w, const void* bias, void* y, int BT, int H, int W, int Ch, int round_ref,
           hipStream_t s) {
  const int slabs = (Ch + 127) / 128;
  const int xgroups = (W + 4 * TW - 1) / (4 * TW);
  // pick the band height so that the launch has enough waves to fill 256 CUs,
  // but keep bands >= 4 rows (two halo rows are re-read per band)
  int R = H;
  const int64_t strips = (int64_t)slabs * ((W + TW - 1) / TW) * BT;
  while (R > 4 && strips * ((H + R - 1) / R) < SANA_DW_MINWAVES) R = (R + 1) / 2;
  const int bands = (H + R - 1) / R;
  if ((int64_t)xgroups * bands > 65535 || BT > 65535) return SANA_ERR_SHAPE;
  dim3 grid(slabs, xgroups * bands, BT);
  // the 16-bit kernel addresses pixels of one image with 32-bit offsets
  const bool small_image = (int64_t)H * W * 2 * Ch * 2 < ((int64_t)1 << 31);
  bool launched = false;
  if constexpr (!std::is_same<T, float>::value) {
    if (small_image) {
      if (round_ref)
        hipLaunchKernelGGL((dwconv_gate16_kernel<T, TW, true>), grid, dim3(256), 0, s, u, w, bias, y, H, W, Ch, R, xgroups);
      else
        hipLaunchKernelGGL((dwconv_gate16_kernel<T, TW, false>), grid, dim3(256), 0, s, u, w, bias, y, H, W, Ch, R, xgroups);
      launched = true;
    }
  }
  if (!launched) {
    if (round_ref)
      hipLaunchKernelGGL((dwconv_gate_kernel<T, TW, true>), grid, dim3(256), 0, s, u, w, bias, y, H, W, Ch, R, xgroups);
    else
      hipLaunchKernelGGL((dwconv_gate_kernel<T, TW, false>), grid, dim3(256), 0, s, u, w, bias, y, H, W, Ch, R, xgroups);
  }
  return hipGetLastError() == hipSuccess ? SANA_OK : SANA_ERR_LAUNCH;
}

}  // namespace
}  // namespace sana

using namespace sana;

extern "C" __attribute__((visibility("default"))) int sana_hip_dwconv3x3_silu_gate(
    const void* u, const void* w, const void* bias, void* y, int BT, int H, int W, int Ch, int round_like_reference,
    int io_dtype, void* stream) {
  if (!u || !w || !y || BT <= 0 || H <= 0 || W <= 0 || Ch <= 0) return SANA_ERR_ARG;
  if (Ch & 1) return SANA_ERR_SHAPE;  // a lane owns a channel pair
  const int esz = io_dtype == SANA_DT_F32 ? 4 : 2;
  const uintptr_t mask = 2 * esz - 1;
  if ((reinterpret_cast<uintptr_t>(u) & mask) || (reinterpret_cast<uintptr_t>(y) & mask)) return SANA_ERR_ALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  constexpr int TW = SANA_DW_TW;
  switch (io_dtype) {
    case SANA_DT_BF16: return launch<BF16, TW>(u, w, bias, y, BT, H, W, Ch, round_like_reference, s);
    case SANA_DT_F16: return launch<F16, TW>(u, w, bias, y, BT, H, W, Ch, round_like_reference, s);
    case SANA_DT_F32: return launch<float, TW>(u, w, bias, y, BT, H, W, Ch, round_like_reference, s);
    default: return SANA_ERR_DTYPE;
  }
}
