// Depthwise 3x3 (zero pad 1) + bias + SiLU gate, channels-last, for gfx950.
//
//   u [BT][H][W][2*Ch] -> y [BT][H][W][Ch],  y[c] = t[c] * silu(t[Ch+c]),
//   t[c] = bias[c] + sum_taps u[..][c] * w[c][tap]
//
// HBM-bound (no reuse across channels; 9-fold reuse across pixels).  Lanes run along the channel axis: a
// lane owns the channel pair (c, c+1) of the first half and (Ch+c, Ch+c+1) of the gate half, so a wave
// covers 256 contiguous bytes per pixel and half, and walks DOWN a strip of 4 output columns with a rolling
// 3-row window in registers: a row of the strip enters the window once, the next rows are in flight while
// the current one is computed.
//   16-bit io (bf16 / f16, Ch % 8 == 0): dwconv_gate16_lds_kernel -- the rows of a workgroup's strip
//     (16 columns + 2 halo columns) are staged through LDS by direct global -> LDS loads, the taps run
//     on packed dot products.
//   fp32 io, and 16-bit io where that kernel does not apply: dwconv_gate_kernel -- every wave loads its
//     own 6-column footprint into an fp32 register window (the four waves of a workgroup take adjacent
//     strips, so the shared halo columns hit in the vector L1).
#include <algorithm>
#include <type_traits>

#include "common.h"

#ifndef SANA_DW_MINWAVES
#define SANA_DW_MINWAVES 6144  // register-window kernel: split rows into bands until the launch has this many waves
#endif
#ifndef SANA_DW_LDS_MINWG
#define SANA_DW_LDS_MINWG 1536  // LDS kernel: split rows into bands until the launch has this many workgroups
#endif
#ifndef SANA_DW_NT_STORE
#define SANA_DW_NT_STORE 0  // non-temporal output stores: faster alone (-5 %), slower for the block (the next GEMM reads y)
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
      store_stream<SANA_DW_NT_STORE != 0>(P::pack(o0, o1), reinterpret_cast<raw_t*>(orow + (int64_t)x * Ch * ESZ + lane_b));
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
// 16-bit io: the taps run on packed dot products.  The register window keeps, per row, channel and column j,
// the PAIR (x[j], x[j+1]) as two 16-bit values in one register (built with one byte-permute from the
// loaded channel-pair words of pixels j and j+1), and a 3-tap row is
//   dot2(pair[j], (w0, w1)) + dot2(pair[j+1], (0, w2))
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

// The same with the sum written to a fresh register (the three-operand encoding): the chain's first product takes
// the bias as its addend without a copy.  (The compiler picks the two-operand form, whose accumulator is also its
// destination, and then copies the bias in front of every chain.)
template <typename T>
__device__ __forceinline__ float dot2_16_from(uint32_t a, uint32_t b, float c);
template <>
__device__ __forceinline__ float dot2_16_from<BF16>(uint32_t a, uint32_t b, float c) {
  float d;
  asm("v_dot2_f32_bf16 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
  return d;
}
template <>
__device__ __forceinline__ float dot2_16_from<F16>(uint32_t a, uint32_t b, float c) {
  float d;
  asm("v_dot2_f32_f16 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
  return d;
}

// ----------------------------------------------------------------------------
// 16-bit io, halo-tiled through LDS.  A workgroup owns a strip of 16 output columns x one slab of 128
// channel pairs and walks down its band of rows.  Rows travel global -> LDS by direct loads (no registers:
// `buffer_load_dwordx4 ... lds`, 16 bytes per lane, whole 256-byte channel runs of a pixel), two rows per
// group, a ring of two groups: while the waves compute from one group the next is in flight, so the bytes
// in flight per compute unit do not depend on registers (4 workgroups x 2 rows x 9 KB).  Every input row of
// the strip -- 16 columns plus one halo column either side -- is read from L2 once per workgroup; each wave
// takes the 6 footprint columns of its 4 output columns from LDS into the same rolling register window of
// (x[j], x[j+1]) pairs as the kernel above.  Pixels and rows outside the image never need a branch or a
// select: their lanes load through an offset outside the buffer resource, which writes zeros to LDS.
// A row in LDS is [18 pixels][first half: 256 B | gate half: 256 B]; one load instruction fills 1 KB = two
// pixels.  The 18 instructions of a group are dealt to the four waves five each (two pieces are written
// twice, with the same data), so every wave can wait on its own counter with a constant.
// ----------------------------------------------------------------------------
constexpr int DWL_PIXB = 512, DWL_RING = 4;

template <typename T, bool ROUND, int NW>
__global__ __launch_bounds__(64 * NW, 16 / NW) void dwconv_gate16_lds_kernel(const void* __restrict__ u, const void* __restrict__ w,
                                                                   const void* __restrict__ bias, void* __restrict__ y,
                                                                   int H, int W, int Ch, int R, int xgroups) {
  typedef Pair<T> P;
  constexpr int ESZ = 2, TW = 4, SW = TW * NW, FP = SW + 2, DWL_ROWB = FP * DWL_PIXB, NPIECE = FP / 2;
  __shared__ __attribute__((aligned(1024))) unsigned char ring[DWL_RING * DWL_ROWB];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  // Workgroups go round-robin to the 8 XCDs (own L2 each) in launch order, x fastest.  All slabs of a strip
  // are launched together, so the eight XCDs read the same pixels at the same time -- whole contiguous
  // 2*Ch-element pixel rows, which is what DRAM pages like -- and WHICH slab a workgroup takes follows from
  // the XCD it landed on: slab m*q + j for the j-th workgroup of XCD m in this grid row (q = slabs / 8), the
  // slabs left over going to whoever has a (q+1)-th workgroup.  A slab below 8*q is then always served by
  // the same L2, which is where neighbouring strips find their shared halo columns.
  int slab;
  {
    const int nsl = gridDim.x, q = nsl >> 3;
    const int xcd = (blockIdx.x + nsl * (blockIdx.y + gridDim.y * blockIdx.z)) & 7, j = blockIdx.x >> 3;
    slab = j < q ? xcd * q + j : 8 * q + (blockIdx.x & 7);
  }
  const int bt = blockIdx.z;
  const int xg = blockIdx.y % xgroups, band = blockIdx.y / xgroups;
  const int x0wg = xg * SW, x0 = x0wg + wave * TW;
  const int y0 = band * R, y1 = min(H, y0 + R);
  const int c = slab * 128 + 2 * lane;
  const bool lane_ok = c < Ch;      // this lane's channel pair exists
  const bool wave_ok = x0 < W;      // this wave has output columns (all waves load and meet at the barriers)
  const int64_t C2 = 2 * (int64_t)Ch;
  const int64_t img = (int64_t)bt * H * W;
  const uint32_t lane_b = (uint32_t)(2 * lane) * ESZ;

  uint32_t w01[4][3], wz2[4][3];
  float bs[4];
  const uint16_t* wp = static_cast<const uint16_t*>(w);
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int64_t ch = (lane_ok ? c : 0) + (q & 1) + (q >> 1) * Ch;
#pragma unroll
    for (int r = 0; r < 3; ++r) {
      w01[q][r] = (uint32_t)wp[ch * 9 + 3 * r] | ((uint32_t)wp[ch * 9 + 3 * r + 1] << 16);
      wz2[q][r] = (uint32_t)wp[ch * 9 + 3 * r + 2] << 16;
    }
    bs[q] = bias ? P::one(bias, ch) : 0.f;
  }

  // ---- global -> LDS.  Lane l of a load instruction: pixel parity l / 32, half (l / 16) % 2, 16-byte chunk l % 16.
  const int pix_b = (int)(C2 * ESZ);
  const __amdgpu_buffer_rsrc_t rsrc_u = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(static_cast<const char*>(u) + img * C2 * ESZ), 0, H * W * pix_b, 0x00020000);
  const int oob = (int)0x80000000u;
  const int d_chan = slab * 128 + (lane & 15) * 8;                       // first channel of the chunk inside its half
  const int d_chb = ((((lane >> 4) & 1) ? Ch : 0) + d_chan) * ESZ;
  const int d_col0 = x0wg - 1 + (lane >> 5);                             // footprint column of piece 0
  const bool d_ok = d_chan < Ch;                                         // Ch % 8 == 0: a chunk is in or out
  auto issue_group = [&](int g) {   // rows 2g, 2g+1 of the band's row stream: image rows y0 - 1 + 2g (+1)
#pragma unroll
    for (int k = 0; k < (2 * NPIECE + NW - 1) / NW; ++k) {
      const int j = wave + NW * k;
      if (j >= 2 * NPIECE) break;                                         // wave-uniform
      const int r = j >= NPIECE ? 1 : 0, i = j - NPIECE * r;
      const int t = 2 * g + r, yy = y0 - 1 + t;
      const bool row_ok = yy >= 0 && yy < H;
      const int col = d_col0 + 2 * i;
      const int voff = (d_ok && row_ok && col >= 0 && col < W) ? col * pix_b + d_chb : oob;
      unsigned char* dst = ring + (t & (DWL_RING - 1)) * DWL_ROWB + i * 1024;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_u, (__attribute__((address_space(3))) void*)dst, 16, voff,
                                               row_ok ? yy * W * pix_b : 0, 0, 0);
    }
  };

  uint32_t win[3][TW + 1][4];
  // the output image from this slab's first channel on: offsets past its end (and the 2^31 of a masked lane) are dropped
  const int opix_b = (int)(Ch * ESZ);
  const __amdgpu_buffer_rsrc_t rsrc_y = __builtin_amdgcn_make_buffer_rsrc(
      static_cast<char*>(y) + (int64_t)slab * 128 * ESZ + img * Ch * ESZ, 0, H * W * opix_b - slab * 128 * ESZ, 0x00020000);
  const unsigned char* my = ring + (4 * wave) * DWL_PIXB + lane_b;        // this wave's first footprint pixel, this lane's pair
  // The ring is read with asm loads: to the compiler an ordinary LDS read may alias the LDS-writing global loads
  // still in flight (the next group's), and it would wait for ALL of them (vmcnt(0)) in front of the first read --
  // which empties the ring at every group.  Which loads must have landed is this kernel's own business (the counted
  // waits and barriers of the main loop); the wait for the reads themselves is tied to their results below.
  const uint32_t my_lds = (uint32_t)(size_t)(__attribute__((address_space(3))) const unsigned char*)my;
  auto take_row = [&](int slot, uint32_t (&row)[TW + 1][4]) {
    uint32_t ra[TW + 2], rg[TW + 2];
    const uint32_t base = my_lds + slot * DWL_ROWB;
#pragma unroll
    for (int i = 0; i < TW + 2; ++i) {
      asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(ra[i]) : "v"(base), "n"(i * DWL_PIXB));
      asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(rg[i]) : "v"(base), "n"(i * DWL_PIXB + 256));
    }
    static_assert(TW + 2 == 6, "the wait below names the six pixels of a row");
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(ra[0]), "+v"(ra[1]), "+v"(ra[2]), "+v"(ra[3]), "+v"(ra[4]), "+v"(ra[5]), "+v"(rg[0]), "+v"(rg[1]),
                   "+v"(rg[2]), "+v"(rg[3]), "+v"(rg[4]), "+v"(rg[5]));
#pragma unroll
    for (int i = 0; i < TW + 1; ++i) {
      row[i][0] = __builtin_amdgcn_perm(ra[i + 1], ra[i], 0x05040100u);
      row[i][1] = __builtin_amdgcn_perm(ra[i + 1], ra[i], 0x07060302u);
      row[i][2] = __builtin_amdgcn_perm(rg[i + 1], rg[i], 0x05040100u);
      row[i][3] = __builtin_amdgcn_perm(rg[i + 1], rg[i], 0x07060302u);
    }
  };
  auto compute = [&](int yo, const uint32_t (&top)[TW + 1][4], const uint32_t (&mid)[TW + 1][4],
                     const uint32_t (&bot)[TW + 1][4]) {
    const int orow = (yo * W + x0) * opix_b;
#pragma unroll
    for (int x = 0; x < TW; ++x) {
      float acc[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float a = dot2_16_from<T>(top[x][q], w01[q][0], bs[q]);
        a = dot2_16<T>(top[x + 1][q], wz2[q][0], a);
        a = dot2_16<T>(mid[x][q], w01[q][1], a);
        a = dot2_16<T>(mid[x + 1][q], wz2[q][1], a);
        a = dot2_16<T>(bot[x][q], w01[q][2], a);
        a = dot2_16<T>(bot[x + 1][q], wz2[q][2], a);
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
      // lanes without a channel pair and columns past the image store through an offset outside the resource
      __builtin_amdgcn_raw_buffer_store_b32(P::pack(o0, o1), rsrc_y,
                                            (lane_ok && x0 + x < W) ? (int)lane_b : oob,
                                            orow + x * opix_b, SANA_DW_NT_STORE ? kBufferNt : 0);
    }
  };

  const int NT = y1 - y0 + 2, NGRP = (NT + 1) >> 1;
  issue_group(0);
  if (NGRP > 1) issue_group(1);
  for (int g0 = 0; g0 < NGRP; g0 += 3) {
#pragma unroll
    for (int gg = 0; gg < 3; ++gg) {
      const int g = g0 + gg;
      if (g >= NGRP) break;  // uniform over the workgroup
      // this wave's pieces of group g have landed: all but the pieces of group g + 1 it issued since
      constexpr int PMAX = (2 * NPIECE + NW - 1) / NW, NFULL = 2 * NPIECE - (PMAX - 1) * NW;  // waves < NFULL issue PMAX
      if (g + 1 >= NGRP) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      else if (wave < NFULL) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(PMAX) : "memory");
      else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(PMAX - 1) : "memory");
      __builtin_amdgcn_s_barrier();                                        // and so have everyone else's (no fence: the
                                                                           // next group's loads stay in flight)
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        const int t = 2 * g + r;
        if (t < NT) {
          const int s3 = (2 * gg + r) % 3;  // static: the loop is unrolled over three groups = six rows
          take_row(t & (DWL_RING - 1), win[s3]);
          if (t >= 2 && wave_ok) compute(y0 + t - 2, win[(s3 + 1) % 3], win[(s3 + 2) % 3], win[s3]);
        }
      }
      __builtin_amdgcn_s_barrier();  // every wave has taken the group's rows (its reads are waited for): the slots may be refilled
      if (g + 2 < NGRP) issue_group(g + 2);
    }
  }
}

template <typename T>
int launch(const void* u, const void* w, const void* bias, void* y, int BT, int H, int W, int Ch, int round_ref,
           hipStream_t s) {
  const int slabs = (Ch + 127) / 128;
  if (BT > 65535) return SANA_ERR_SHAPE;
  // 16-bit io: the LDS kernel (32-bit byte offsets inside one image, 16-byte channel chunks)
  if constexpr (!std::is_same<T, float>::value) {
    if ((int64_t)H * W * 2 * Ch * 2 < ((int64_t)1 << 31) && Ch % 8 == 0) {
      // Bands of rows so that the launch has at least SANA_DW_LDS_MINWG workgroups (four fit a compute unit).
      // Two halo rows are re-read per band: no band shorter than 8 rows, or than 4 where even that leaves
      // the chip short of work (single small images).
      constexpr int NW = 4;
      const int xg = (W + 4 * NW - 1) / (4 * NW);
      const int64_t base = (int64_t)slabs * xg * BT;
      const int min_rows = base * ((H + 7) / 8) >= 512 ? 8 : 4;
      int nb = (int)((SANA_DW_LDS_MINWG + base - 1) / base);
      nb = std::max(1, std::min(nb, (H + min_rows - 1) / min_rows));
      const int R = (H + nb - 1) / nb, bands = (H + R - 1) / R;
      if ((int64_t)xg * bands <= 65535) {
        dim3 grid(slabs, xg * bands, BT);
        if (round_ref)
          hipLaunchKernelGGL((dwconv_gate16_lds_kernel<T, true, NW>), grid, dim3(64 * NW), 0, s, u, w, bias, y, H, W, Ch, R, xg);
        else
          hipLaunchKernelGGL((dwconv_gate16_lds_kernel<T, false, NW>), grid, dim3(64 * NW), 0, s, u, w, bias, y, H, W, Ch, R, xg);
        return hipGetLastError() == hipSuccess ? SANA_OK : SANA_ERR_LAUNCH;
      }
    }
  }
  // register-window kernel: pick the band height so that the launch has enough waves to fill 256 CUs,
  // but keep bands >= 4 rows
  constexpr int TW = 4;
  const int xgroups = (W + 4 * TW - 1) / (4 * TW);
  int R = H;
  const int64_t strips = (int64_t)slabs * ((W + TW - 1) / TW) * BT;
  while (R > 4 && strips * ((H + R - 1) / R) < SANA_DW_MINWAVES) R = (R + 1) / 2;
  const int bands = (H + R - 1) / R;
  if ((int64_t)xgroups * bands > 65535) return SANA_ERR_SHAPE;
  dim3 grid(slabs, xgroups * bands, BT);
  if (round_ref)
    hipLaunchKernelGGL((dwconv_gate_kernel<T, TW, true>), grid, dim3(256), 0, s, u, w, bias, y, H, W, Ch, R, xgroups);
  else
    hipLaunchKernelGGL((dwconv_gate_kernel<T, TW, false>), grid, dim3(256), 0, s, u, w, bias, y, H, W, Ch, R, xgroups);
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
  switch (io_dtype) {
    case SANA_DT_BF16: return launch<BF16>(u, w, bias, y, BT, H, W, Ch, round_like_reference, s);
    case SANA_DT_F16: return launch<F16>(u, w, bias, y, BT, H, W, Ch, round_like_reference, s);
    case SANA_DT_F32: return launch<float>(u, w, bias, y, BT, H, W, Ch, round_like_reference, s);
    default: return SANA_ERR_DTYPE;
  }
}
