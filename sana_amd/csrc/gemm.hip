// bf16 MFMA GEMM for gfx950:  C[M][N] = epilogue(A[M][K] . W[N][K]^T)
// with an int8-weight (W8A16) variant dequantised on the way into LDS.
//
// Both operands are K-contiguous, which is exactly the MFMA operand layout (a
// lane holds 8 consecutive k of one row), so nothing is transposed.  The MFMA
// "row" operand is the WEIGHT tile and the "column" operand the ACTIVATION
// tile: a lane of the accumulator then owns one token (column) and a few output
// channels (rows).  Weight rows are permuted on their way into LDS so that the
// channels a lane owns are contiguous in C (the pipelined kernel: 8*NI channels
// from 2*NI MFMA tiles of 16; the compiler-scheduled one: 16 channels per 32x32 tile).
//
// Workgroup tile 256 (tokens) x 256 (channels) x 64 (k), four waves in 2x2,
// each 128x128 (256 fp32 accumulators).  The pipelined kernel multiplies with
// v_mfma_f32_16x16x32_bf16: on this chip the matrix pipes are power-limited, and
// with random bf16 operands a loop of nothing but 32x32x16 MFMAs settles at 1.64 GHz
// (0.69 of the 2.5 PFLOP/s peak) where the same flops as 16x16x32 run at 1.9-2.0 GHz.
// LDS is double buffered (2 x 64 KB); 16-byte chunks are XOR-swizzled by (row / 2) % 8 so
// that ds_read_b128 / ds_write_b128 are bank-conflict free.  Workgroup ids are
// remapped so that each XCD (own L2) works on a compact group of tiles.
#include <algorithm>

#include "common.h"

// No implicit fused multiply-adds in this file: the epilogues reproduce the stock op chain's roundings (product
// rounded to the io dtype, THEN the sum), and for fp16 -- which has native arithmetic -- the compiler would otherwise
// contract "round(g * y) + r" into one v_fma_f16 and drop the product's rounding.  Wanted fmas are written as fmaf.
#pragma clang fp contract(off)

// Tuning knobs: non-temporal hint on the output stores (one bit per epilogue kind: 1 none, 2 bias, 4 bias + SiLU,
// 8 gated residual; measured on the 20-block step, all four on is best: 2.307 ms per block against 2.319-2.324 with
// the gated-residual or the plain outputs cacheable and 2.332 with none) / on the residual loads of the pipelined
// kernel's epilogue.
#ifndef SANA_GEMM_NT_STORE
#define SANA_GEMM_NT_STORE 15
#endif
#ifndef SANA_GEMM_NT_RES
#define SANA_GEMM_NT_RES 0
#endif

namespace sana {
namespace {

constexpr int BT = 256;   // tokens (rows of A / C) per workgroup
constexpr int BC = 256;   // output channels (rows of W) per workgroup
constexpr int BK = 64;
constexpr int ROW_BYTES = BK * 2;            // 128
constexpr int TILE_BYTES = 256 * ROW_BYTES;  // 32 KB per operand per stage

// LDS reads of 16 bytes are served 16 lanes (256 bytes = all 64 banks) per clock, so 16 consecutive
// rows of one k chunk must land in 16 different 16-byte bank groups: rows alternate between the two
// halves of the bank space (128-byte rows), and the chunk index is XORed with (row / 2) % 8.
__device__ __forceinline__ int swz_key(int row) { return (row >> 1) & 7; }
__device__ __forceinline__ int swz(int row, int chunk) { return row * ROW_BYTES + ((chunk ^ swz_key(row)) << 4); }

// LDS row of weight row n (within the 256-row tile): permute inside each 32-row block
__device__ __forceinline__ int wrow_to_lds(int n) {
  const int blk = n & ~31, r = n & 31;
  return blk + 8 * ((r >> 2) & 3) + 4 * (r >> 4) + (r & 3);
}

// The GEMMs exist for the two 16-bit io dtypes, T = BF16 (also the int8-weight and the fused-state variants) or F16:
// same loops, the MFMA of the dtype, and the dtype's own conversions in the epilogues (one v_cvt_pk_bf16_f32 per pair
// for bf16; two conversions and a pack for f16, which has no packed round-to-nearest conversion).
// acc += W fragment (16 channels x 32 k) . A fragment (32 k x 16 tokens), as an asm statement so that the
// accumulator is one AGPR quad in and out: given the builtin, whose destination may differ from its addend, the
// register allocator rotates accumulators through other registers across the loop edge (dozens of copies and
// their wait states per k-tile in some instances).
template <typename T>
__device__ __forceinline__ void mfma_acc(f32x4_t& c, u32x4_t a, u32x4_t b) {
  if constexpr (is_f16<T>) asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  else asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}

__device__ __forceinline__ uint32_t dequant2(uint32_t q4, int which, float s, float off) {
  // two int8 (bytes 2*which, 2*which+1 of q4, already biased by +128) -> packed bf16(q*s)
  // (the compiler turns these byte extracts into v_cvt_f32_ubyteN)
  const float f0 = (float)((q4 >> (16 * which)) & 0xffu);
  const float f1 = (float)((q4 >> (16 * which + 8)) & 0xffu);
  // (q+128)*s - 128*s == q*s exactly before the single fp32 rounding
  return pack_bf16(fmaf(f0, s, off), fmaf(f1, s, off));
}

// int8 weight [N][K] + per-row scale -> bf16 [N][K], with the rounding of dequant2: the expansion the GEMM's
// int8 path performs on its way to LDS, as a streaming kernel of its own (16 values per thread).
__global__ __launch_bounds__(256) void dequant_w8_kernel(const int8_t* __restrict__ wq, const float* __restrict__ scale,
                                                         uint16_t* __restrict__ out, int N, int K, int64_t ldw,
                                                         int64_t ldo) {
  const int pieces = K >> 4;
  const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (id >= (int64_t)N * pieces) return;
  const int n = (int)(id / pieces), p = (int)(id - (int64_t)n * pieces);
  u32x4_t q = *reinterpret_cast<const u32x4_t*>(wq + n * ldw + 16 * p);
  const float s = scale[n], off = -128.f * s;
  u32x4_t lo, hi;
  q.x ^= 0x80808080u, q.y ^= 0x80808080u, q.z ^= 0x80808080u, q.w ^= 0x80808080u;
  lo.x = dequant2(q.x, 0, s, off), lo.y = dequant2(q.x, 1, s, off);
  lo.z = dequant2(q.y, 0, s, off), lo.w = dequant2(q.y, 1, s, off);
  hi.x = dequant2(q.z, 0, s, off), hi.y = dequant2(q.z, 1, s, off);
  hi.z = dequant2(q.w, 0, s, off), hi.w = dequant2(q.w, 1, s, off);
  uint16_t* o = out + n * ldo + 16 * p;
  *reinterpret_cast<u32x4_t*>(o) = lo;
  *reinterpret_cast<u32x4_t*>(o + 8) = hi;
}

// Epilogue operands.  SANA_EPI_GATE_RES: C = res + gate[row / rows_per_gate] * (acc + bias), i.e. the
// gated residual update of the block (x + gate * module(x)), with the reference's three roundings
// (linear output, gate product, residual sum) reproduced in registers.
struct EpiArgs {
  const uint16_t* bias;  // [N] or null
  const uint16_t* gate;  // [*, N] rows gate_stride apart, one row per rows_per_gate rows of C
  const uint16_t* res;   // [M, N] with row stride ldr
  int64_t ldr, gate_stride;
  int rows_per_gate;
  // SANA_EPI_QKV_STATE only: per-token-tile partial states, [B * heads][tiles_per_batch][33 * 32] fp32
  float* part;
  int q_cols, q_pad, heads, tiles_per_batch;  // q_cols = C (columns of the q region), q_pad = C rounded up to the tile
};
#define SANA_EPI_GATE_RES 3
// (not part of the C ABI's epilogue codes) qkv projection of the linear attention with the k / v column tiles
// contracted over their tokens in the epilogue instead of stored: see state_tile16
#define SANA_EPI_QKV_STATE 4

// Virtual concatenation of the A operand along k: columns [t*kc, (t+1)*kc) of the GEMM's A are columns
// [0, kc) of the matrix whose row m is row m + t*stride of the buffer (a convolution over rows as one GEMM,
// without materialising its im2col matrix).  rows = rows of the buffer that exist, counted from A: reads
// past them return zero (the convolution's zero padding on that side).
struct Taps {
  int kc;          // columns per tap, a multiple of the k-tile
  int64_t stride;  // rows between taps
  int64_t rows;
  // split-k launches (SPLIT, never together with taps): grid row z works on k-tiles
  // [z*split_tiles + min(z, split_rem), ...) -- split_tiles of them, one more for z < split_rem
  int split_tiles, split_rem;
  // taps only, may be null: one byte per block of `stride` output rows; non-zero = the LAST tap reads zeros for
  // these rows (a chunk boundary behind the block: the convolution's zero padding inside the buffer)
  const unsigned char* zero_last;
};

// 8 outputs of one row: accumulator (+bias) -> io dtype, per the epilogue kind (everything except
// the gated residual, which needs the row's residual and gate and is applied at store time).
template <int EPI, typename T = BF16>
__device__ __forceinline__ u32x4_t epi_pack8(const float* a, const float* bv) {
  float v[8];
#pragma unroll
  for (int r = 0; r < 8; ++r) v[r] = EPI != SANA_EPI_NONE ? a[r] + bv[r] : a[r];
  u32x4_t o;
  o.x = pk16<T>(v[0], v[1]);
  o.y = pk16<T>(v[2], v[3]);
  o.z = pk16<T>(v[4], v[5]);
  o.w = pk16<T>(v[6], v[7]);
  if (EPI == SANA_EPI_BIAS_SILU) {
    // The reference rounds the linear output to bf16 before the activation.  x * rcp(1 + 2^(-x log2 e)),
    // written stage by stage over the eight values (and pinned that way): one value at a time is a
    // chain of dependent instructions with two slow transcendentals, which a lone wave per SIMD
    // cannot hide.
    float x[8], t[8];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      x[2 * p] = lo16<T>(o[p]);
      x[2 * p + 1] = hi16<T>(o[p]);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int r = 0; r < 8; ++r) t[r] = -1.44269504088896341f * x[r];
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int r = 0; r < 8; ++r) t[r] = __builtin_amdgcn_exp2f(t[r]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int r = 0; r < 8; ++r) t[r] = 1.0f + t[r];
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int r = 0; r < 8; ++r) t[r] = __builtin_amdgcn_rcpf(t[r]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int r = 0; r < 8; ++r) x[r] *= t[r];
    __builtin_amdgcn_sched_barrier(0);
    o.x = pk16<T>(x[0], x[1]);
    o.y = pk16<T>(x[2], x[3]);
    o.z = pk16<T>(x[4], x[5]);
    o.w = pk16<T>(x[6], x[7]);
  }
  return o;
}
template <typename T = BF16>
__device__ __forceinline__ uint32_t gate_res2(uint32_t y, uint32_t g, uint32_t r) {
  const float t0 = rnd16<T>(lo16<T>(g) * lo16<T>(y)), t1 = rnd16<T>(hi16<T>(g) * hi16<T>(y));
  return pk16<T>(lo16<T>(r) + t0, hi16<T>(r) + t1);
}
// y: 8 linear outputs (already rounded to bf16), g / r: the gate and residual values of the same 8 columns
template <typename T = BF16>
__device__ __forceinline__ u32x4_t gate_res8v(u32x4_t y, u32x4_t g, u32x4_t r) {
  u32x4_t o;
  o.x = gate_res2<T>(y.x, g.x, r.x);
  o.y = gate_res2<T>(y.y, g.y, r.y);
  o.z = gate_res2<T>(y.z, g.z, r.z);
  o.w = gate_res2<T>(y.w, g.w, r.w);
  return o;
}
// the same with the gate values already unpacked (they are the same for every row a lane handles)
template <typename T = BF16>
__device__ __forceinline__ u32x4_t gate_res8f(u32x4_t y, const float* g, u32x4_t r) {
  u32x4_t o;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const uint32_t t = pk16<T>(g[2 * e] * lo16<T>(y[e]), g[2 * e + 1] * hi16<T>(y[e]));  // one convert rounds both
    o[e] = pk16<T>(lo16<T>(r[e]) + lo16<T>(t), hi16<T>(r[e]) + hi16<T>(t));
  }
  return o;
}
// y: 8 linear outputs (already rounded to bf16) of row m, columns n..n+7
template <typename T = BF16>
__device__ __forceinline__ u32x4_t gate_res8(u32x4_t y, const EpiArgs& e, int m, int n) {
  const u32x4_t g = *reinterpret_cast<const u32x4_t*>(e.gate + (int64_t)(m / e.rows_per_gate) * e.gate_stride + n);
  const u32x4_t r = *reinterpret_cast<const u32x4_t*>(e.res + (int64_t)m * e.ldr + n);
  u32x4_t o;
  o.x = gate_res2<T>(y.x, g.x, r.x);
  o.y = gate_res2<T>(y.y, g.y, r.y);
  o.z = gate_res2<T>(y.z, g.z, r.z);
  o.w = gate_res2<T>(y.w, g.w, r.w);
  return o;
}

// Compiler-scheduled kernel, any K % 8 == 0 (int8: K % 16 == 0).  Workgroup tile 64*TT tokens x 64*TC channels,
// four waves in 2x2, each TT x TC MFMA tiles.  <4, 4>: the 256 x 256 tile of the pipelined kernel, for the K
// values that one does not take.  <2, 2>: 128 x 128 with 64 accumulators and 64 KB of LDS, two workgroups per
// CU -- a quarter of the work per k-tile, so a much shorter latency chain for shapes whose 256-wide grid would
// leave the chip mostly idle (a few hundred to a few thousand tokens); its k-tiles are requested three ahead
// (three register sets in rotation), because with so little math per k-tile the chain is otherwise one global
// load latency per k-tile.  Every output sums its k products in the same order in all of these kernels, so
// they agree bit for bit.
template <bool W8, int EPI, int TT = 4, int TC = 4, typename T = BF16>
__global__ __launch_bounds__(256, (TT * TC <= 4 ? 2 : 1)) void gemm_kernel(const uint16_t* __restrict__ A, const void* __restrict__ Wv,
                                                   const float* __restrict__ scale, const EpiArgs ep,
                                                   uint16_t* __restrict__ C,
                                                   int M, int N, int K, int64_t lda, int64_t ldw, int64_t ldc,
                                                   int tiles_t, int tiles_c) {
  constexpr int BT = 64 * TT, BC = 64 * TC;              // shadow the file-scope 256 x 256
  constexpr int A_BYTES = BT * ROW_BYTES, STAGE_BYTES = (BT + BC) * ROW_BYTES;
  __shared__ __attribute__((aligned(16))) unsigned char smem[2 * STAGE_BYTES];  // [stage][A | W]
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;

  // ---- workgroup -> tile, XCD aware: ids are dealt round-robin to the 8 XCDs, so
  // give XCD x the x-th contiguous eighth of the (grouped) tile order.
  const int total = tiles_t * tiles_c;
  int pid = blockIdx.x;
  {
    const int xcd = pid & 7, local = pid >> 3;
    const int base = total >> 3, rem = total & 7;
    pid = xcd * base + min(xcd, rem) + local;  // ids with id%8 == x: base + (x < rem) of them
  }
  constexpr int GROUP = 8;  // token tiles per group
  const int group_sz = GROUP * tiles_c;
  const int gid = pid / group_sz;
  const int first_t = gid * GROUP;
  const int gt = min(tiles_t - first_t, GROUP);
  const int tile_t = first_t + (pid % group_sz) % gt;
  const int tile_c = (pid % group_sz) / gt;
  const int m0 = tile_t * BT, n0 = tile_c * BC;

  // ---- global -> register staging
  // A tile: BT rows x 8 chunks(16 B); thread -> chunk tid%8, rows tid/8 + 32*i
  const int a_chunk = tid & 7, a_row = tid >> 3;
  constexpr int NA = 2 * TT, NW = W8 ? TC : 2 * TC;
  constexpr int DEPTH = TT * TC <= 4 ? 3 : 1;  // k-tiles in flight in registers
  u32x4_t ra[DEPTH][NA];
  // W tile bf16: same shape.  W8: BC rows x 4 chunks of 16 int8; thread -> chunk tid%4, rows tid/4 + 64*i
  u32x4_t rw[DEPTH][NW];
  const int w_chunk = W8 ? (tid & 3) : (tid & 7), w_row = W8 ? (tid >> 2) : (tid >> 3);

  // Operand tiles are read with buffer loads, one resource per operand over the tile's valid rows (ending with
  // the last valid row's K-th element): rows past M / N fall outside it and read as zero, and a k chunk past K
  // gets an offset outside it -- no branches around the loads, so that several k-tiles can stay in flight.
  // (The whole offset is the vector offset: only that one is range-checked.)
  const int a_last = min(BT, M - m0) - 1, w_last = min(BC, N - n0) - 1;
  constexpr int WB = W8 ? 1 : 2;  // bytes per weight
  const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(A + (int64_t)m0 * lda), 0, (int)(((int64_t)a_last * lda + K) * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_w = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(static_cast<const char*>(Wv) + (int64_t)n0 * ldw * WB), 0,
      (int)(((int64_t)w_last * ldw + K) * WB), 0x00020000);
  const int idle_off = (int)0x80000000u;
  const int voff_a = (a_row * (int)lda + a_chunk * 8) * 2, step_a = 32 * (int)lda * 2;
  const int voff_w = (w_row * (int)ldw + w_chunk * (W8 ? 16 : 8)) * WB, step_w = (W8 ? 64 : 32) * (int)ldw * WB;
  auto load_tile = [&](int set, int k0) {  // k chunks past K load zeros
    const int off_a = k0 + a_chunk * 8 < K ? voff_a + k0 * 2 : idle_off;
    const int off_w = k0 + w_chunk * (W8 ? 16 : 8) < K ? voff_w + k0 * WB : idle_off;
#pragma unroll
    for (int i = 0; i < NA; ++i)
      ra[set][i] = __builtin_bit_cast(u32x4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, off_a + i * step_a, 0, 0));
#pragma unroll
    for (int i = 0; i < NW; ++i)
      rw[set][i] = __builtin_bit_cast(u32x4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, off_w + i * step_w, 0, 0));
  };
  float wscale[TC], woff[TC];
  if (W8) {
#pragma unroll
    for (int i = 0; i < TC; ++i) {
      const int n = n0 + w_row + 64 * i;
      wscale[i] = n < N ? scale[n] : 0.f;
      woff[i] = -128.f * wscale[i];
    }
  }
  auto store_tile = [&](int set, int stage) {
    unsigned char* sa = smem + stage * STAGE_BYTES;
    unsigned char* sw = sa + A_BYTES;
#pragma unroll
    for (int i = 0; i < NA; ++i) *reinterpret_cast<u32x4_t*>(sa + swz(a_row + 32 * i, a_chunk)) = ra[set][i];
    if (W8) {
#pragma unroll
      for (int i = 0; i < NW; ++i) {
        const int lrow = wrow_to_lds(w_row + 64 * i);
        u32x4_t q = rw[set][i];
        q.x ^= 0x80808080u;
        q.y ^= 0x80808080u;
        q.z ^= 0x80808080u;
        q.w ^= 0x80808080u;
        u32x4_t lo, hi;
        lo.x = dequant2(q.x, 0, wscale[i], woff[i]);
        lo.y = dequant2(q.x, 1, wscale[i], woff[i]);
        lo.z = dequant2(q.y, 0, wscale[i], woff[i]);
        lo.w = dequant2(q.y, 1, wscale[i], woff[i]);
        hi.x = dequant2(q.z, 0, wscale[i], woff[i]);
        hi.y = dequant2(q.z, 1, wscale[i], woff[i]);
        hi.z = dequant2(q.w, 0, wscale[i], woff[i]);
        hi.w = dequant2(q.w, 1, wscale[i], woff[i]);
        *reinterpret_cast<u32x4_t*>(sw + swz(lrow, 2 * w_chunk)) = lo;
        *reinterpret_cast<u32x4_t*>(sw + swz(lrow, 2 * w_chunk + 1)) = hi;
      }
    } else {
#pragma unroll
      for (int i = 0; i < NW; ++i)
        *reinterpret_cast<u32x4_t*>(sw + swz(wrow_to_lds(w_row + 32 * i), w_chunk)) = rw[set][i];
    }
  };

  // ---- MFMA tiling: wave (wc, wt) owns channels [wc*32*TC, +32*TC) x tokens [wt*32*TT, +32*TT)
  const int wc = wave & 1, wt = wave >> 1;
  const int fr = lane & 31, fg = lane >> 5;
  f32x16_t acc[TC][TT];
#pragma unroll
  for (int i = 0; i < TC; ++i)
#pragma unroll
    for (int j = 0; j < TT; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int KT = (K + BK - 1) / BK;
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) load_tile(d, d * BK);
  store_tile(0, 0);
  __syncthreads();
  // k-tile kt is multiplied from LDS stage kt % 2 while register set kt % DEPTH (which held it) is refilled with
  // k-tile kt + DEPTH and set (kt + 1) % DEPTH goes to the other stage; unrolled by DEPTH so the set is static.
  // The loop runs whole rounds of DEPTH: k-tiles past K are all zeros (they add nothing), and a body without
  // exits keeps the compiler's count of outstanding loads exact.
  for (int kt0 = 0; kt0 < KT; kt0 += DEPTH) {
#pragma unroll
   for (int d = 0; d < DEPTH; ++d) {
    const int kt = kt0 + d;
    const int cur = kt & 1;
    load_tile(d, (kt + DEPTH) * BK);
    const unsigned char* sa = smem + cur * STAGE_BYTES;
    const unsigned char* sw = sa + A_BYTES;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      u32x4_t fw[TC], fa[TT];
#pragma unroll
      for (int i = 0; i < TC; ++i)
        fw[i] = *reinterpret_cast<const u32x4_t*>(sw + swz(wc * 32 * TC + 32 * i + fr, 2 * ks + fg));
#pragma unroll
      for (int j = 0; j < TT; ++j)
        fa[j] = *reinterpret_cast<const u32x4_t*>(sa + swz(wt * 32 * TT + 32 * j + fr, 2 * ks + fg));
#pragma unroll
      for (int i = 0; i < TC; ++i)
#pragma unroll
        for (int j = 0; j < TT; ++j)
          acc[i][j] = mfma_32x32x16<T>(fw[i], fa[j], acc[i][j]);
    }
    store_tile((d + 1) % DEPTH, cur ^ 1);
    __syncthreads();
   }
  }

  // ---- epilogue.  acc[i][j][r]: token m0 + wt*32*TT + 32*j + lane%32,
  // channel n0 + wc*32*TC + 32*i + 16*(lane/32) + r
  constexpr bool HAS_BIAS = EPI != SANA_EPI_NONE;
#pragma unroll
  for (int i = 0; i < TC; ++i) {
    const int n = n0 + wc * 32 * TC + 32 * i + 16 * fg;
    float bv[16];
    if (HAS_BIAS) {
#pragma unroll
      for (int r = 0; r < 16; ++r) bv[r] = (ep.bias && n + r < N) ? lo16<T>(ep.bias[n + r]) : 0.f;
    }
#pragma unroll
    for (int j = 0; j < TT; ++j) {
      const int m = m0 + wt * 32 * TT + 32 * j + fr;
      if (m >= M) continue;
      uint16_t* cp = C + (int64_t)m * ldc + n;
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        if (n + 8 * half < N) {  // N % 8 == 0: a chunk is either fully inside or outside
          float a8[8];
#pragma unroll
          for (int r = 0; r < 8; ++r) a8[r] = acc[i][j][8 * half + r];
          u32x4_t o = epi_pack8<EPI == SANA_EPI_GATE_RES ? SANA_EPI_BIAS : EPI, T>(a8, bv + 8 * half);
          if (EPI == SANA_EPI_GATE_RES) o = gate_res8<T>(o, ep, m, n + 8 * half);
          *reinterpret_cast<u32x4_t*>(cp + 8 * half) = o;
        }
      }
    }
  }
}


// Epilogue of a k / v column tile of the fused qkv projection (SANA_EPI_QKV_STATE, 256-wide tiles only).  The tile's
// 256 weight rows are, per wave column wc, [K of head 4T+2wc | V of it | K of head 4T+2wc+1 | V of it] (32 rows
// each; the caller lays the weight out that way, see sana_hip_qkv_state_rows), so lane group g = lane / 16 of a wave
// holds, for its tokens lane % 16 + 16 j, all 32 channels of one of those four blocks.  Instead of storing k and v,
// the wave contracts them over its 128 tokens: S[dv][dk] += v[n][dv] * relu(k[n][dk]) and ksum[dk] += relu(k[n][dk])
// with v and k rounded to bf16 first (what the unfused path stores and reads back), products in fp32 on the MFMA.
// The contraction index of v_mfma_f32_16x16x32_bf16 is the token, and which token sits in which k slot is free as
// long as both operands agree: the 8 tokens a lane holds for one channel (j = 0 .. 7) ARE one operand fragment, it
// only sits in the wrong lane (the lane is the token group, the MFMA wants the channel there), so it takes one trip
// through the wave's LDS: written at [channel][token group ^ channel % 16] (16 bytes each, conflict-free both ways),
// read back as [channel = lane % 16][token group 4 m + lane / 16] for the m-th MFMA of a chain of four.  The two
// token halves of the workgroup are added through LDS and the sum goes to this token tile's slot of the partial
// states, which a second kernel adds up in tile order (deterministic, no atomics).
__device__ __forceinline__ void state_tile16(f32x4_t (&acc)[8][8], const u32x4_t (&bpk)[4], unsigned char* smem,
                                             const EpiArgs& ep, int m0, int n0) {
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int wc = wave & 1, wt = wave >> 1;
  const int fr = lane & 15, fg = lane >> 4;
  __syncthreads();  // every wave is done with the operand tiles
  unsigned char* stg = smem + wave * 32768;
  // relu for the k blocks (fg even) as a packed signed-integer max on the bf16 pairs; int16 minimum = no-op for v
  const uint32_t floor2 = (fg & 1) ? 0x80008000u : 0u;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint32_t bw0 = bpk[i >> 1][2 * (i & 1)], bw1 = bpk[i >> 1][2 * (i & 1) + 1];
    const float b4[4] = {bf16_lo(bw0), bf16_hi(bw0), bf16_lo(bw1), bf16_hi(bw1)};  // channels 4 i + r of the lane's 32
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      u32x4_t o;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint32_t pk = pack_bf16(acc[i][2 * e][r] + b4[r], acc[i][2 * e + 1][r] + b4[r]);
        o[e] = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(s16x2_t, pk),
                                                                    __builtin_bit_cast(s16x2_t, floor2)));
      }
      const int row = 32 * fg + 4 * i + r;
      *reinterpret_cast<u32x4_t*>(stg + row * 256 + ((fr ^ (row & 15)) << 4)) = o;
    }
  }
  // wave-private LDS is in order: the reads below see the writes above.  hh: the wave's two heads.  The products
  // are formed transposed (rows = dk, columns = dv), so that a lane ends with four consecutive dk of one dv:
  // 16-byte stores into the [dv][dk] state.
  f32x4_t S[2][2][2], Ks[2][2];  // S[hh][a][b]: dk 16 a + 4 fg + r, dv 16 b + fr;  Ks[hh][a]: dk 16 a + 4 fg + r
#pragma unroll
  for (int hh = 0; hh < 2; ++hh)
#pragma unroll
    for (int b = 0; b < 2; ++b) {
#pragma unroll
      for (int r = 0; r < 4; ++r) Ks[hh][b][r] = 0.f, S[hh][0][b][r] = 0.f, S[hh][1][b][r] = 0.f;
    }
  const u32x4_t ones = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
#pragma unroll
  for (int hh = 0; hh < 2; ++hh) {
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const int slot = ((4 * m + fg) ^ fr) << 4;
      u32x4_t kf[2], vf[2];
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        kf[b] = *reinterpret_cast<const u32x4_t*>(stg + (64 * hh + 16 * b + fr) * 256 + slot);
        vf[b] = *reinterpret_cast<const u32x4_t*>(stg + (64 * hh + 32 + 16 * b + fr) * 256 + slot);
      }
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        // (the builtin, not the main loop's asm statement: the compiler then places the wait states itself)
        S[hh][a][0] = mfma_16x16x32_bf16(kf[a], vf[0], S[hh][a][0]);
        S[hh][a][1] = mfma_16x16x32_bf16(kf[a], vf[1], S[hh][a][1]);
        Ks[hh][a] = mfma_16x16x32_bf16(kf[a], ones, Ks[hh][a]);
      }
    }
  }
  // add the two token halves: wave wt = 1 hands its 48 values per lane to wave wt = 0 of the same channel half
  f32x4_t* xch = reinterpret_cast<f32x4_t*>(stg) + lane;
  if (wt == 1) {
#pragma unroll
    for (int hh = 0; hh < 2; ++hh)
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        xch[((hh * 2 + a) * 3 + 0) * 64] = S[hh][a][0];
        xch[((hh * 2 + a) * 3 + 1) * 64] = S[hh][a][1];
        xch[((hh * 2 + a) * 3 + 2) * 64] = Ks[hh][a];
      }
  }
  __syncthreads();
  if (wt == 0) {
    const f32x4_t* oth = reinterpret_cast<const f32x4_t*>(smem + (wave + 2) * 32768) + lane;
    const int tile_kv = (n0 - ep.q_pad) >> 8;
    const int tile_m = m0 >> 8;
    const int bi = tile_m / ep.tiles_per_batch, split = tile_m - bi * ep.tiles_per_batch;
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      const int head = 4 * tile_kv + 2 * wc + hh;
      if (head < ep.heads) {
        float* o = ep.part + (((int64_t)bi * ep.heads + head) * ep.tiles_per_batch + split) * (33 * 32);
#pragma unroll
        for (int a = 0; a < 2; ++a) {
          const int dk0 = 16 * a + 4 * fg;
#pragma unroll
          for (int b = 0; b < 2; ++b)
            *reinterpret_cast<f32x4_t*>(o + (16 * b + fr) * 32 + dk0) = S[hh][a][b] + oth[((hh * 2 + a) * 3 + b) * 64];
          if (fr == 0) *reinterpret_cast<f32x4_t*>(o + 32 * 32 + dk0) = Ks[hh][a] + oth[((hh * 2 + a) * 3 + 2) * 64];
        }
      }
    }
  }
}

// Epilogue of the pipelined kernels.  acc[i][j][r] (MFMA 16x16 tiles: i = channel tile of the wave, j = token tile):
// token m0 + wt*128 + 16*j + lane%16, channel n0 + wc*32*NI + 8*NI*(lane/16) + 4*i + r.  bpk: the lane's 8*NI bias
// values, packed (the caller requests them ahead of its last k-tile so that their latency hides behind its MFMAs).
template <int EPI, int NI, bool SPLIT, typename T = BF16>
__device__ __forceinline__ void finish_tile16(f32x4_t (&acc)[2 * NI][8], const u32x4_t (&bpk)[NI], unsigned char* smem,
                                              const EpiArgs& ep, uint16_t* __restrict__ C, int M, int N, int64_t ldc,
                                              int m0, int n0) {
  constexpr int NWT = 2 * NI;
  constexpr bool HAS_BIAS = EPI != SANA_EPI_NONE;
  if constexpr (EPI == SANA_EPI_QKV_STATE) {
    static_assert(NI == 4 && !SPLIT && !is_f16<T>, "the fused qkv projection runs 256-wide bf16 tiles, unsplit");
    if (n0 >= ep.q_pad) {  // uniform per workgroup: a k / v tile
      state_tile16(acc, bpk, smem, ep, m0, n0);
      return;
    }
    N = ep.q_cols;  // a q tile: stored like any biased output, columns past C dropped
  }
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int wc = wave & 1, wt = wave >> 1;
  const int fr = lane & 15, fg = lane >> 4;
  const int o_chunk = lane & 15, o_rsub = lane >> 4;
  const int o_n = n0 + wc * 32 * NI + o_chunk * 8;
  const bool o_live = o_chunk < 4 * NI && o_n < N;  // a staged row holds 4*NI chunks (the row pitch stays 256 bytes)
  // ---- epilogue.  acc[i][j][r]: token m0 + wt*128 + 16*j + lane%16,
  // channel n0 + wc*32*NI + 8*NI*(lane/16) + 4*i + r.  The wave's sub-tile goes through its own 32 KB of
  // LDS ([128 tokens][256 bytes], 16-byte chunks XOR-swizzled by token % 16) and comes back
  // row-contiguous, so each store instruction writes four full 256-byte row segments.  It goes in four
  // groups of 32 tokens: the stores of one group drain while the next group's activations are computed.
  if (SPLIT) {
    // raw accumulators -> partial[z][M][N] (fp32, dense).  A lane owns 8*NI consecutive channels of one token per
    // token tile j, but one store instruction of that layout would write 64 separate 16-byte pieces (16 rows x 4
    // lane groups): measured, such an epilogue took as long as the 22 k-tiles in front of it.  So the sub-tile
    // goes through the wave's 32 KB of LDS, 64 tokens at a time ([64 tokens][128 channels] fp32, 16-byte chunks
    // XOR-swizzled by token % 16), and leaves as whole row segments: a store instruction writes two rows of 512
    // contiguous bytes.  Rows past M fall outside the buffer resource and are dropped; chunks past N get the idle
    // offset.
    __syncthreads();  // every wave is done with the operand tiles
    unsigned char* stg = smem + wave * 32768;
    const int prow0 = m0 + __builtin_amdgcn_readfirstlane(wt) * 128;
    const int prows = max(0, min(128, M - prow0));
    float* plane = reinterpret_cast<float*>(C) + ((int64_t)blockIdx.y * M + prow0) * N;
    const __amdgpu_buffer_rsrc_t rsrc_p =
        __builtin_amdgcn_make_buffer_rsrc(plane, 0, (int)((int64_t)prows * N * 4), 0x00020000);
    const int s_chunk = lane & 31, s_rsub = lane >> 5;               // store side: 32 chunks of 4 channels, 2 rows
    const int s_n = n0 + wc * 32 * NI + 4 * s_chunk;
    const bool s_live = s_chunk < 8 * NI && s_n < N;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) {
        const int tok = 16 * jj + fr;                                 // token of this half, 0 .. 63
#pragma unroll
        for (int i = 0; i < NWT; ++i) {
          const int chunk = 2 * NI * fg + i;                          // 4 channels each: 8*NI*fg + 4*i
          const u32x4_t o = {__float_as_uint(acc[i][4 * half + jj][0]), __float_as_uint(acc[i][4 * half + jj][1]),
                             __float_as_uint(acc[i][4 * half + jj][2]), __float_as_uint(acc[i][4 * half + jj][3])};
          *reinterpret_cast<u32x4_t*>(stg + tok * 512 + ((chunk ^ (tok & 15)) << 4)) = o;
        }
      }
      // wave-private LDS is in order: the reads below see the writes above
#pragma unroll
      for (int it = 0; it < 32; ++it) {
        const int row = 2 * it + s_rsub;                              // 0 .. 63
        const u32x4_t o = *reinterpret_cast<const u32x4_t*>(stg + row * 512 + ((s_chunk ^ (row & 15)) << 4));
        const int off = s_live ? ((64 * half + row) * N + s_n) * 4 : (int)0x80000000u;
        __builtin_amdgcn_raw_buffer_store_b128(o, rsrc_p, off, 0, 0);
      }
    }
    return;
  }
  __syncthreads();  // every wave is done with the operand tiles
  unsigned char* stg = smem + wave * 32768;
  // Global accesses of the epilogue are buffer loads / stores on the wave's 128 rows of C (and of the
  // residual): a row costs one vector add for its offset, rows past M and channel pieces past N fall
  // outside the resource (loads return zero, stores are dropped) -- no 64-bit address arithmetic, no
  // per-row predication.
  const int wrow0 = m0 + __builtin_amdgcn_readfirstlane(wt) * 128;  // first row of this wave (a scalar: it goes into resources)
  const int wrows = max(0, min(128, M - wrow0));          // its rows that exist
  const int idle_off = (int)0x80000000u;
  const __amdgpu_buffer_rsrc_t rsrc_c = __builtin_amdgcn_make_buffer_rsrc(
      C + (int64_t)wrow0 * ldc, 0, wrows ? (int)((((int64_t)wrows - 1) * ldc + N) * 2) : 0, 0x00020000);
  const int c_off0 = o_live ? (o_rsub * (int)ldc + o_n) * 2 : idle_off, c_step = 4 * (int)ldc * 2;
  // Gated residual: the residual rows this lane will add are requested now, a whole epilogue ahead
  // of their use (128 registers that the main loop no longer needs; asking for them before the last
  // k-tile makes the compiler spill).
  u32x4_t res[4][8];
  const bool gated = EPI == SANA_EPI_GATE_RES;
  const __amdgpu_buffer_rsrc_t rsrc_r = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(gated ? ep.res + (int64_t)wrow0 * ep.ldr : nullptr), 0,
      gated && wrows ? (int)((((int64_t)wrows - 1) * ep.ldr + N) * 2) : 0, 0x00020000);
  const int r_off0 = o_live ? (o_rsub * (int)ep.ldr + o_n) * 2 : idle_off, r_step = 4 * (int)ep.ldr * 2;
  if (EPI == SANA_EPI_GATE_RES) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int it = 0; it < 8; ++it)
        res[j][it] = __builtin_bit_cast(
            u32x4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc_r, r_off0 + (8 * j + it) * r_step, 0, SANA_GEMM_NT_RES ? kBufferNt : 0));
  }
  float bv[NI][8];
  if (HAS_BIAS) {
#pragma unroll
    for (int c = 0; c < NI; ++c)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        bv[c][2 * e] = lo16<T>(bpk[c][e]);
        bv[c][2 * e + 1] = hi16<T>(bpk[c][e]);
      }
  }
  // Software-pipelined over the four groups of 32 tokens: step s of phase j converts piece s of group j
  // (accumulators -> activation -> LDS) and stores row chunk s of group j - 1 (LDS -> gate / residual -> global).
  // Handing a 16-byte-per-lane store to the memory pipeline keeps it busy for ~130 clocks, during which the
  // wave can issue VALU work but not another store: one store between two pieces of arithmetic costs a
  // fraction of what eight stores in a row cost.
  auto convert_piece = [&](int jg, int p) {  // group jg of 32 tokens = token tiles 2*jg, 2*jg + 1; p = NI * (tile & 1) + c
    const int j = 2 * jg + p / NI, c = p % NI;  // c: the lane's c-th chunk of 8 channels = W tiles 2c, 2c + 1
    const int tok = 16 * j + fr;
    float a8[8];
#pragma unroll
    for (int r = 0; r < 4; ++r) a8[r] = acc[2 * c][j][r], a8[4 + r] = acc[2 * c + 1][j][r];
    const u32x4_t o = epi_pack8<(EPI == SANA_EPI_GATE_RES || EPI == SANA_EPI_QKV_STATE) ? SANA_EPI_BIAS : EPI, T>(a8, bv[c]);
    const int chunk = NI * fg + c;
    *reinterpret_cast<u32x4_t*>(stg + tok * 256 + ((chunk ^ (tok & 15)) << 4)) = o;
  };
  auto read_row = [&](int j, int it) {
    const int row = 32 * j + it * 4 + o_rsub;
    return *reinterpret_cast<const u32x4_t*>(stg + row * 256 + ((o_chunk ^ (row & 15)) << 4));
  };
#pragma unroll
  for (int j = 0; j <= 4; ++j) {
    const int js = j - 1;  // the group whose rows are stored in this phase
    // The lane's eight gate values, as floats.  One gate row serves the whole group of 32 tokens unless a
    // batch boundary runs through it: then the rows from m_switch on take the next gate row (gates are per
    // batch entry; entries shorter than 32 tokens take the slow way, a division per row).
    const int m_first = wrow0 + 32 * js;
    int m_switch = 0;
    bool two_gates = false;
    float gf[8] = {1.f, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f};  // no gate: 1.0, a plain residual add
    u32x4_t o_next = {0u, 0u, 0u, 0u};
    if (js >= 0) {
      if (EPI == SANA_EPI_GATE_RES) {
        const int g_first = m_first / ep.rows_per_gate;
        m_switch = (g_first + 1) * ep.rows_per_gate;
        two_gates = ep.gate && m_switch < min(m_first + 32, M);
        if (ep.gate && o_live && m_first < M) {
          const u32x4_t gate = *reinterpret_cast<const u32x4_t*>(ep.gate + (int64_t)g_first * ep.gate_stride + o_n);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            gf[2 * e] = lo16<T>(gate[e]);
            gf[2 * e + 1] = hi16<T>(gate[e]);
          }
        }
      }
      o_next = read_row(js, 0);  // wave-private LDS is in order: the group's writes are behind it
    }
#pragma unroll
    for (int st = 0; st < 8; ++st) {
      u32x4_t o = o_next;
      if (js >= 0 && st + 1 < 8) o_next = read_row(js, st + 1);
      __builtin_amdgcn_sched_barrier(0);
      if (j < 4 && st < 2 * NI) convert_piece(j, st);
      __builtin_amdgcn_sched_barrier(0);
      if (js >= 0) {
        if (EPI == SANA_EPI_GATE_RES) o = gate_res8f<T>(o, gf, res[js][st]);
        __builtin_amdgcn_raw_buffer_store_b128(o, rsrc_c, c_off0 + (8 * js + st) * c_step, 0, ((SANA_GEMM_NT_STORE >> EPI) & 1) ? kBufferNt : 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (js >= 0 && two_gates) {  // uniform, rare: rows behind the boundary are redone with their own gate row and stored again
#pragma unroll 1
      for (int it = 0; it < 8; ++it) {
        const int row = 32 * js + it * 4 + o_rsub, m = wrow0 + row;
        if (o_live && m >= m_switch && m < M) {
          const u32x4_t y = *reinterpret_cast<const u32x4_t*>(stg + row * 256 + ((o_chunk ^ (row & 15)) << 4));
          const u32x4_t r = __builtin_bit_cast(
              u32x4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc_r, r_off0 + (8 * js + it) * r_step, 0, 0));
          const u32x4_t g2 = *reinterpret_cast<const u32x4_t*>(
              ep.gate + (int64_t)(m / ep.rows_per_gate) * ep.gate_stride + o_n);
          __builtin_amdgcn_raw_buffer_store_b128(gate_res8v<T>(y, g2, r), rsrc_c, c_off0 + (8 * js + it) * c_step, 0, 0);
        }
      }
    }
  }
}

// ============================================================================
// Pipelined kernel (K % 32 == 0, K >= 64; bf16 and int8 weights): 256 threads, one
// wave per SIMD with the whole register file (256 accumulators + 256 VGPRs), each
// wave a sub-tile of 128 tokens x 32*NI channels = 2*NI x 8 MFMA tiles of 16x16
// (NI = 4: 128x128; NI = 3 narrows the workgroup's channel tile to 192 where that fills
// the last round of workgroups better, NI = 2 to 128 for few tokens and wide N, where the
// shorter k-tile and the larger grid shorten the latency chain).  With a single wave per SIMD nothing
// else hides a stalled memory instruction, so the main loop is one hand-ordered
// stream (pinned with sched_barrier): a k-tile is two k-steps of 32 = 2 * 16*NI MFMA
// slots of 16 cycles, and a lone wave issues about one other instruction per 5 cycles,
// so a slot carries at most a fragment read, a store or a load (bf16):
//   * k-step 0: the fragments of k-step 1, and all staging -- quad q (k-tile kt+1) is
//     stored into the other LDS stage and the same registers are re-loaded with
//     k-tile kt+2 one slot later, so every global load has a whole k-tile (about
//     1 us) to land and one 64-register set is enough;
//   * the only barrier sits right behind it, and the next tile's k-step-0 fragments
//     are read over the rest of k-step 1, which runs from the other fragment buffer
//     (int8 weights: 16 values per quad, converted two at a time in the MFMA slots
//     before they are stored, the quad reloaded after its last piece; their barrier
//     stays at the end of the k-tile).
// The MFMAs are asm statements with the accumulator tied in and out (see mfma_acc).
// Rows past M / N read as zero (buffer range check) and only feed outputs that are
// never stored; the last k-tile runs just the k-steps that exist.
// ============================================================================
// SPLIT (split-k, for shapes with too few tiles to fill the chip): grid row z multiplies its own range of
// k-tiles and stores the raw fp32 accumulators to C taken as float [gridDim.y][M][N]; splitk_epilogue_kernel
// adds the ranges up in order and applies the epilogue.
// TAPS: 0 = plain A operand, 1 = tap-concatenated A operand, 2 = the same with per-row-block zero_last flags.
template <bool W8, int EPI, int NI, int TAPS = 0, bool SPLIT = false, typename T = BF16>
__global__ __launch_bounds__(256) void gemm4_kernel(const uint16_t* __restrict__ A_, const void* __restrict__ Wv_,
                                                    const float* __restrict__ scale, const EpiArgs ep,
                                                    uint16_t* __restrict__ C, int M, int N, int K_, int64_t lda,
                                                    int64_t ldw, int64_t ldc, int tiles_t, int tiles_c,
                                                    const Taps tp) {
  __shared__ __attribute__((aligned(1024))) unsigned char smem[4 * TILE_BYTES];  // [stage][A | W]
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const uint16_t* A = A_;
  const void* Wv = Wv_;
  int K = K_;
  if (SPLIT) {  // this grid row's k range becomes "the" K of everything below
    const int z = blockIdx.y;
    const int kb = (z * tp.split_tiles + min(z, tp.split_rem)) * BK;
    const int kn = (tp.split_tiles + (z < tp.split_rem ? 1 : 0)) * BK;
    A += kb;
    Wv = static_cast<const char*>(Wv_) + (int64_t)kb * (W8 ? 1 : 2);
    K = min(K_ - kb, kn);
  }
  const int total = tiles_t * tiles_c;
  int pid = blockIdx.x;
  {
    const int xcd = pid & 7, local = pid >> 3;
    const int base = total >> 3, rem = total & 7;
    pid = xcd * base + min(xcd, rem) + local;
  }
  // tile rows per group: an XCD's 32 concurrent tiles are GROUP rows x 32/GROUP columns.  Measured: 4 is 1-2 % better
  // for the short-K wide-N shapes (qkv, inverted conv), 8 is 2-3 % better for the long-K point conv.
  const int GROUP = K >= 4096 ? 8 : 4;
  const int group_sz = GROUP * tiles_c;
  const int gid = pid / group_sz;
  const int first_t = gid * GROUP;
  const int gt = min(tiles_t - first_t, GROUP);
  const int tile_t = first_t + (pid % group_sz) % gt;
  const int tile_c = (pid % group_sz) / gt;
  constexpr int BCN = 64 * NI;  // channels per workgroup: two waves x NI MFMA tiles of 32
  const int m0 = tile_t * BT, n0 = tile_c * BCN;

  // global -> VGPR -> LDS: thread -> k chunk tid%8, rows tid/8 + 32*q, q < 8 for A and q < 2*NI for bf16 W.
  // int8 W: thread -> 16-value chunk tid%4, rows tid/4 + 64*q (q < NI); dequantised on the way to LDS.
  const int g_chunk = tid & 7, g_row = tid >> 3;
  const int a_last = min(BT, M - m0) - 1, w_last = min(BCN, N - n0) - 1;  // last valid row of each tile
  const uint32_t ulda = (uint32_t)lda, uldw = (uint32_t)ldw;
  const int a_dst0 = swz(g_row, g_chunk);               // rows +32*q keep the key: +4096 bytes each
  const int w_dst0 = TILE_BYTES + swz(g_row, g_chunk);  // LDS rows g_row + 32*q; the weight-row permutation is on the global side
  // LDS row L of a wave's block of 32*NI weight rows belongs to MFMA tile L / 16 as its row L % 16 = 4*g + r, and
  // holds channel 8*NI*g + 4*(L / 16) + r of the block: a lane's accumulators (tile i, registers r) are then the
  // 8*NI contiguous channels 8*NI*g + 4*i + r.  The thread's quad q (LDS rows g_row + 32*q) is channel
  // w_chan0 + 8*(q % NI) + 32*NI*(q / NI) of the tile.
  const int w_chan0 = 8 * NI * ((g_row >> 2) & 3) + 4 * (g_row >> 4) + (g_row & 3);
  constexpr int NWQ = W8 ? NI : 2 * NI;  // W quads per thread
  constexpr int NQ = 8 + NWQ;
  u32x4_t rs[NQ];  // the k-tile in flight: A quads 0..7, then the W quads
  const int q_chunk = tid & 3, q_row = tid >> 2;
  const int q_dst_lo = TILE_BYTES + swz(q_row, 2 * q_chunk);  // LDS rows q_row + 64*q: +8192 bytes, same key
  const int q_dst_hi = TILE_BYTES + swz(q_row, 2 * q_chunk + 1);
  float wscale[NI], woff[NI];
  int q_voff[NI];  // int8 quads: byte offset of the channel that LDS row q_row + 64*q holds
  if (W8) {
#pragma unroll
    for (int q = 0; q < NI; ++q) {
      const int L = q_row + 64 * q, blk = L / (32 * NI), l = L % (32 * NI);
      const int chan = blk * 32 * NI + 8 * NI * ((l >> 2) & 3) + 4 * (l >> 4) + (l & 3);
      q_voff[q] = chan * (int)ldw + 16 * q_chunk;
      wscale[q] = scale[n0 + min(chan, w_last)];
      woff[q] = -128.f * wscale[q];
    }
  }
  u32x4_t dq[2];  // dequantised halves of the int8 quad being converted

  const int wc = wave & 1, wt = wave >> 1;
  const int fr = lane & 15, fg = lane >> 4;
  const int x7 = swz_key(fr);
  const int w_off = TILE_BYTES + (wc * 32 * NI + fr) * ROW_BYTES, a_off = (wt * 128 + fr) * ROW_BYTES;
  constexpr int NWT = 2 * NI;  // MFMA tiles of 16 channels per wave (and 8 tiles of 16 tokens)
  f32x4_t acc[NWT][8];
#pragma unroll
  for (int i = 0; i < NWT; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;
  u32x4_t fw[2][NWT], fa[2][8];

#define SANA_G4_PIN() __builtin_amdgcn_sched_barrier(0)
  // Operand tiles are read with buffer loads: the tile's rows are one resource each for A and W (scalar
  // registers), the lane's (row, k chunk) is a constant vector offset, and the quad / k-tile part of the
  // address is scalar, so a load costs one vector add.  The resource ends with the last valid row's
  // K-th element: rows past M / N and anything past the end of the matrix read as zero instead of
  // faulting (k chunks past K inside the matrix read the next row: they are never multiplied).
  // (TAPS: the resource ends with the buffer's last existing row instead, so a tap that reaches past it is zero)
  const int64_t a_bytes = TAPS ? (tp.rows > m0 ? ((tp.rows - m0 - 1) * lda + tp.kc) * 2 : 0)
                               : ((int64_t)a_last * lda + K) * 2;
  const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(A + (int64_t)m0 * lda), 0, (int)a_bytes, 0x00020000);
  // byte offset of k-tile k0 inside a row of A (TAPS: tap k0 / kc starts tp.stride rows further down)
  const int tap_b = TAPS ? (int)(tp.stride * lda * 2) : 0;
  auto a_koff = [&](int k0) { return TAPS ? (k0 / tp.kc) * tap_b + (k0 % tp.kc) * 2 : k0 * 2; };
  int a_kb = 0, a_kin = 0;  // offset of the k-tile being requested, and its column inside the tap
  // rows of this thread (bit q: row g_row + 32*q) whose last tap is zero padding.  While the k-tile being
  // requested belongs to the last tap, those rows' vector offsets carry 2^31 -- outside the resource, so the
  // loads return zeros -- at no cost in the loop: the per-row offsets live in registers and change with the tap.
  uint32_t zlast = 0;
  int voffq[8];
  int a_tap = 0;
  const int last_tap = TAPS ? K / tp.kc - 1 : 0;
  if (TAPS == 2 && tp.zero_last) {
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const int r = m0 + (tid >> 3) + 32 * q;
      if (r < M && tp.zero_last[r / tp.stride]) zlast |= 1u << q;
    }
  }
  const int voff_a0 = ((tid >> 3) * (int)lda + 8 * (tid & 7)) * 2;  // the thread's (row, k chunk) inside the tile
  auto poison = [&](bool last) {
#pragma unroll
    for (int q = 0; q < 8; ++q) voffq[q] = voff_a0;
    if (TAPS == 2 && last) {
#pragma unroll
      for (int q = 0; q < 8; ++q) voffq[q] = voff_a0 + (((zlast >> q) & 1u) ? (int)0x80000000u : 0);
    }
  };
  poison(false);
  const __amdgpu_buffer_rsrc_t rsrc_w = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(static_cast<const char*>(Wv) + (int64_t)n0 * ldw * (W8 ? 1 : 2)), 0,
      (int)(((int64_t)w_last * ldw + K) * (W8 ? 1 : 2)), 0x00020000);
  const int voff_a = (g_row * (int)ulda + 8 * g_chunk) * 2;
  const int voff_w = (w_chan0 * (int)uldw + 8 * g_chunk) * 2;  // bf16 weights
  const int step_a = 32 * (int)ulda * 2, step_w1 = (int)uldw * 2;
  auto gload = [&](int q, int k0) {
    if (q < 8) {
      const int off = (TAPS == 2 ? voffq[q] : voff_a) + (q * step_a + (TAPS ? a_kb : k0 * 2));
      const auto v = __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, off, 0, 0);
      rs[q] = __builtin_bit_cast(u32x4_t, v);
    } else {
      const int wq = q - 8;
      const int off = W8 ? q_voff[wq] + k0 : voff_w + ((8 * (wq % NI) + 32 * NI * (wq / NI)) * step_w1 + k0 * 2);
      const auto v = __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, off, 0, 0);
      rs[q] = __builtin_bit_cast(u32x4_t, v);
    }
  };
  auto lstore = [&](int q, int stage) {  // A quads, bf16 W quads
    unsigned char* base = smem + stage * 2 * TILE_BYTES;
    if (q < 8) *reinterpret_cast<u32x4_t*>(base + a_dst0 + 4096 * q) = rs[q];
    else *reinterpret_cast<u32x4_t*>(base + w_dst0 + 4096 * (q - 8)) = rs[q];
  };
  // int8 quad wq (16 values), piece 0..7 = two values each: convert, and store a 16-byte half when complete
  auto dequant_piece = [&](int wq, int piece, int stage) {
    uint32_t word = rs[8 + wq][piece >> 1] ^ 0x80808080u;
    dq[piece >> 2][piece & 3] = dequant2(word, piece & 1, wscale[wq], woff[wq]);
    if ((piece & 3) == 3) {
      unsigned char* base = smem + stage * 2 * TILE_BYTES + 8192 * wq;
      *reinterpret_cast<u32x4_t*>(base + (piece < 4 ? q_dst_lo : q_dst_hi)) = dq[piece >> 2];
    }
  };
  constexpr int NFR = NWT + 8;  // fragment reads per k-step (of 32)
  // read r of a k-step, in the order the MFMAs need them: W tile 0, the eight A tiles, then W tiles 1 ..
  auto fread = [&](const unsigned char* st, int buf, int ks, int r) {
    const int col = ((4 * ks + fg) ^ x7) << 4;
    if (r == 0 || r > 8) {
      const int i = r == 0 ? 0 : r - 8;
      fw[buf][i] = *reinterpret_cast<const u32x4_t*>(st + w_off + i * 16 * ROW_BYTES + col);
    } else {
      fa[buf][r - 1] = *reinterpret_cast<const u32x4_t*>(st + a_off + (r - 1) * 16 * ROW_BYTES + col);
    }
  };
  // MFMA t of a k-step: weight tile t / 8, and the token tiles in alternating direction (0..7, 7..0, ..), so that
  // every MFMA differs from its predecessor in ONE operand -- at the end of a row of eight only the weight fragment
  // changes, not both.  Less switching on the operand buses: the power-limited clock settles ~1 % higher.
  auto mfma = [&](int buf, int t) {  // t < 8 * NWT
    const int i = t >> 3, j = (i & 1) ? 7 - (t & 7) : (t & 7);
    mfma_acc<T>(acc[i][j], fw[buf][i], fa[buf][j]);
  };

  const int KT = (K + BK - 1) / BK;
  // prologue: k-tile 0 -> stage 0, k-tile 1 in flight
#pragma unroll
  for (int q = 0; q < NQ; ++q) gload(q, 0);
  if (TAPS) {
    a_kb = a_koff(BK);
    if (TAPS == 2 && zlast) poison(BK / tp.kc == last_tap);
  }
#pragma unroll
  for (int q = 0; q < (W8 ? 8 : NQ); ++q) lstore(q, 0);
  if (W8) {
#pragma unroll
    for (int n = 0; n < 8 * NI; ++n) dequant_piece(n >> 3, n & 7, 0);
  }
#pragma unroll
  for (int q = 0; q < NQ; ++q) gload(q, BK);
  if (TAPS) {
    a_kb = a_koff(2 * BK);
    a_kin = (2 * BK) % tp.kc;
    a_tap = (2 * BK) / tp.kc;
    if (TAPS == 2 && zlast) poison(a_tap == last_tap);
  }
  __syncthreads();
#pragma unroll
  for (int q = 0; q < NFR; ++q) fread(smem, 0, 0, q);

  // Slots: a k-tile is two k-steps of 32 = 2 * SL MFMAs of 16 cycles each, and a lone wave issues about one
  // other instruction per 5 cycles, so no slot carries more than a fragment read or a store or a load.
  //  * k-step 0: the fragments of k-step 1 (read r at slot r*SL/NFR), and all staging -- quad q stored to the other
  //    LDS stage at slot 1 + q*QSTRIDE and re-loaded (k-tile kt+2) one slot later;
  //  * the barrier right behind it (slot SL + 2), and the next tile's k-step-0 fragments spread over the rest
  //    of k-step 1, which runs from the other fragment buffer.
  // int8 weights convert 8*NI pieces in the MFMA slots as well, so their barrier stays at the end of the k-tile.
  constexpr int SL = 8 * NWT, TS = 2 * SL;
  constexpr int BAR = W8 ? TS - NFR - 1 : SL + 2;
  constexpr int RSTR = W8 ? 1 : (TS - BAR - 1 - 8) / NFR;  // spacing of the reads behind the barrier
  constexpr int QSTRIDE = SL / NQ;                           // bf16: spacing of the staging quads
  constexpr int PSTR = (BAR - 4) / (8 * NI);                 // int8: piece n (two values) at slot 2 + n*PSTR
  static_assert(W8 || (QSTRIDE >= 2 && 1 + (NQ - 1) * QSTRIDE < BAR - 2 && RSTR >= 1 && BAR + 1 + (NFR - 1) * RSTR < TS),
                "staging does not fit in front of the barrier");
  static_assert(!W8 || (4 * 7 + 1 < BAR && PSTR >= 1), "staging does not fit in front of the barrier");
  // The MFMAs below are asm statements: the compiler neither knows that they read the accumulators through the
  // matrix pipe nor places the wait states such a read needs behind the VALU writes that zeroed them.  Pin the
  // order by hand: every accumulator passes through an empty asm statement (its zeroing is complete, in program
  // order, in front of it), then eight wait states, then the first MFMA -- whatever the compiler puts in between.
#pragma unroll
  for (int i = 0; i < NWT; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) asm volatile("" : "+a"(acc[i][j]));
  asm volatile("s_nop 7" ::: "memory");
  for (int kt = 0; kt < KT - 1; ++kt) {
    const int cur = kt & 1;
    const unsigned char* st = smem + cur * 2 * TILE_BYTES;
    const unsigned char* stn = smem + (cur ^ 1) * 2 * TILE_BYTES;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
      for (int t = 0; t < SL; ++t) {
        const int slot = ks * SL + t;
        mfma(ks, t);
        SANA_G4_PIN();
        if (ks == 0) {
          // read r of k-step 1 goes to slot (r * SL) / NFR of k-step 0
          if (((t * NFR + SL - 1) / SL) * SL / NFR == t && (t * NFR + SL - 1) / SL < NFR)
            fread(st, 1, 1, (t * NFR + SL - 1) / SL);
        }
        if (slot == BAR) {
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // own LDS stores done; no fence: loads stay in flight
          __builtin_amdgcn_s_barrier();
          asm volatile("" ::: "memory");
        } else if (slot > BAR && (slot - BAR - 1) % RSTR == 0 && (slot - BAR - 1) / RSTR < NFR) {
          fread(stn, 0, 0, (slot - BAR - 1) / RSTR);
        }
        if (!W8) {
          if (slot >= 1 && (slot - 1) % QSTRIDE == 0 && (slot - 1) / QSTRIDE < NQ) lstore((slot - 1) / QSTRIDE, cur ^ 1);
          if (slot >= 2 && (slot - 2) % QSTRIDE == 0 && (slot - 2) / QSTRIDE < NQ)
            gload((slot - 2) / QSTRIDE, (kt + 2) * BK);
        } else {
          // A quad q: store at slot 4q, reload at 4q+1.  int8 piece n at slot 2 + n*PSTR (its half is stored
          // with pieces 3 and 7), the quad is reloaded one slot after its last piece.
          if (slot % 4 == 0 && slot / 4 < 8) lstore(slot / 4, cur ^ 1);
          if (slot % 4 == 1 && slot / 4 < 8) gload(slot / 4, (kt + 2) * BK);
          if (slot >= 2 && (slot - 2) % PSTR == 0 && (slot - 2) / PSTR < 8 * NI)
            dequant_piece(((slot - 2) / PSTR) >> 3, ((slot - 2) / PSTR) & 7, cur ^ 1);
          if (slot >= 3 && (slot - 3) % PSTR == 0 && (slot - 3) / PSTR < 8 * NI && (((slot - 3) / PSTR) & 7) == 7)
            gload(8 + (((slot - 3) / PSTR) >> 3), (kt + 2) * BK);
        }
        SANA_G4_PIN();
      }
    }
    if (TAPS) {  // the next iteration requests k-tile kt + 3
      a_kin += BK;
      a_kb += BK * 2;
      if (a_kin >= tp.kc) {
        a_kin -= tp.kc;
        a_kb += tap_b - tp.kc * 2;
        ++a_tap;
        if (TAPS == 2 && zlast) poison(a_tap == last_tap);
      }
    }
  }
#undef SANA_G4_PIN
  // The lane's bias values (16 consecutive channels per MFMA tile, packed) are requested here, ahead of
  // the last k-tile, so that their latency hides behind its MFMAs.
  constexpr bool HAS_BIAS = EPI != SANA_EPI_NONE;
  u32x4_t bpk[NI];  // the lane's 8*NI contiguous channels, in chunks of 8
  if (HAS_BIAS) {
#pragma unroll
    for (int c = 0; c < NI; ++c) {
      const int n = n0 + wc * 32 * NI + 8 * NI * fg + 8 * c;  // N % 8 == 0: a chunk is in or out
      bpk[c] = (ep.bias && n < N) ? *reinterpret_cast<const u32x4_t*>(ep.bias + n) : u32x4_t{0u, 0u, 0u, 0u};
    }
  }
  {  // last k-tile: no successor, and K % 64 may leave one k-step of 32 instead of two
    const unsigned char* st = smem + ((KT - 1) & 1) * 2 * TILE_BYTES;
    const int steps = (K - (KT - 1) * BK) / 32;
    for (int ks = 0; ks < steps; ++ks) {
      const int col = ((4 * ks + fg) ^ x7) << 4;
      u32x4_t w8[NWT], a8[8];
#pragma unroll
      for (int i = 0; i < NWT; ++i) w8[i] = *reinterpret_cast<const u32x4_t*>(st + w_off + i * 16 * ROW_BYTES + col);
#pragma unroll
      for (int j = 0; j < 8; ++j) a8[j] = *reinterpret_cast<const u32x4_t*>(st + a_off + j * 16 * ROW_BYTES + col);
#pragma unroll
      for (int i = 0; i < NWT; ++i)
#pragma unroll
        for (int jj = 0; jj < 8; ++jj) {
          const int j = (i & 1) ? 7 - jj : jj;
          mfma_acc<T>(acc[i][j], w8[i], a8[j]);
        }
    }
    // the MFMAs are asm statements, so the compiler does not know that their results are in flight: wait out the
    // last ones before anything reads an accumulator
    asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" ::: "memory");
  }

  finish_tile16<EPI, NI, SPLIT, T>(acc, bpk, smem, ep, C, M, N, ldc, m0, n0);
}

// Second half of a split-k GEMM: partial[S][M][N] (fp32) -> C = epilogue(sum over the S k-ranges, added in
// order).  One thread per row and 8 channels; the same epilogue functions as the fused path.
template <int EPI, typename T = BF16>
__global__ __launch_bounds__(256) void splitk_epilogue_kernel(const float* __restrict__ partial, int S,
                                                               const EpiArgs ep, uint16_t* __restrict__ C, int M, int N,
                                                               int64_t ldc) {
  const int chunks = N >> 3;
  const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (id >= (int64_t)M * chunks) return;
  const int m = (int)(id / chunks), n = (int)(id - (int64_t)m * chunks) * 8;
  const f32x4_t* p = reinterpret_cast<const f32x4_t*>(partial + (int64_t)m * N + n);
  const int64_t plane = (int64_t)M * N / 4;
  f32x4_t lo = p[0], hi = p[1];
  for (int z = 1; z < S; ++z) {
    lo += p[z * plane];
    hi += p[z * plane + 1];
  }
  const float a[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  float bv[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (EPI != SANA_EPI_NONE && ep.bias) {
    const u32x4_t b = *reinterpret_cast<const u32x4_t*>(ep.bias + n);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      bv[2 * e] = lo16<T>(b[e]);
      bv[2 * e + 1] = hi16<T>(b[e]);
    }
  }
  u32x4_t o = epi_pack8<EPI == SANA_EPI_GATE_RES ? SANA_EPI_BIAS : EPI, T>(a, bv);
  if (EPI == SANA_EPI_GATE_RES) o = gate_res8<T>(o, ep, m, n);
  *reinterpret_cast<u32x4_t*>(C + (int64_t)m * ldc + n) = o;
}

// The library is built for one chip, MI355X: 256 compute units in 8 XCDs.  A constant (not a device query)
// keeps the library free of global state and makes the plans -- and sana_hip_gemm_workspace_bytes -- the same on
// every host, with or without a GPU.
constexpr int compute_units() { return 256; }

// Channel tile of the pipelined kernel (NI = 4: 256 channels, 3: 192).  One workgroup per compute unit at a
// time, so the grid runs in rounds: the tile whose rounds x tile size is smaller wins; the narrower tile
// re-reads a little more per MFMA, hence its 4 % handicap.
int pick_ni(int M, int N) {
  const int64_t cu = compute_units(), tiles_t = (M + BT - 1) / BT;
  const int64_t t256 = tiles_t * ((N + 255) / 256), t192 = tiles_t * ((N + 191) / 192);
  const double cost256 = (double)((t256 + cu - 1) / cu) * 4.0, cost192 = (double)((t192 + cu - 1) / cu) * 3.0 * 1.04;
  return cost192 < cost256 ? 3 : 4;
}

// Channels to cover with 256-wide tiles when the rest goes to 192-wide ones in a second launch, or 0 when one width
// for all of N is at least as good.  Costs in rounds of 256 workgroups: a 192-wide round counts 0.78 (3/4 of the
// math, 4 % more operand traffic per MFMA), the second launch 0.05; the mix must win by 2 %.
int mixed_split(int M, int N) {
  const int64_t cu = compute_units(), tiles_t = (M + BT - 1) / BT;
  auto rounds = [&](int64_t col_tiles) { return (double)((tiles_t * col_tiles + cu - 1) / cu); };
  const double pure = std::min(rounds((N + 255) / 256), 0.78 * rounds((N + 191) / 192));
  double best = pure * 0.98;
  int best_wide = 0;
  for (int a = 1; a * 256 < N; ++a) {
    const double cost = rounds(a) + 0.78 * rounds((N - a * 256 + 191) / 192) + 0.05;
    if (cost < best) {
      best = cost;
      best_wide = a * 256;
    }
  }
  return best_wide;
}

// Which kernel, and whether K is split.  A workgroup's K loop is a latency chain whatever the grid: about
// 1.1 us per k-tile for the 256-wide pipelined kernel, 0.8 us for the 128 x 128 one (a quarter of the math, but
// the same load / LDS / barrier round trip).  A grid that covers the chip keeps the 256-wide kernel (throughput
// is what counts, and that kernel has twice the math per byte).  A grid of fewer tiles than half the compute
// units (M = 1024 tokens x N = 2240: 48 workgroups on 256 CUs) leaves most of the chip idle for the whole
// chain; two remedies, by estimate:
//  * split-k: S ranges of >= 8 k-tiles (S <= 8, S x tiles <= CUs) shorten the chain to ceil(KT / S) k-tiles and
//    cost the fp32 partial planes (S x M x N x 4 bytes written and read once, about 6 bytes/ns at these sizes)
//    plus a second launch (about 5 us); taken when that beats the unsplit chain by 15 %.  Long-K narrow-N
//    shapes (the point conv of a few thousand tokens or less) split, wide-N or short-K ones do not.
//  * the 128 x 128 kernel, when its grid still fits one workgroup per CU and its chain beats the above.
struct GemmPlan {
  bool small;         // the 128 x 128 kernel
  int S, tiles, rem;  // k ranges; k-tiles per range; ranges that take one more
};
GemmPlan plan_gemm(int M, int N, int K, bool w8) {
  GemmPlan pl = {false, 1, 0, 0};
  const int KT = (K + BK - 1) / BK, cu = compute_units();
  const bool pipelined = K % 32 == 0 && K >= 64;
  const double us_tile = pipelined ? 1.1 : 1.4, us_tile_small = 0.8, us_launch = 5.0, bytes_per_us = 6.0e6;
  double best = KT * us_tile;
  if (pipelined) {
    const int ni = pick_ni(M, N);
    const int64_t tiles = (int64_t)((M + BT - 1) / BT) * ((N + 64 * ni - 1) / (64 * ni));
    if (tiles * 2 <= cu && KT >= 16 && (int64_t)M * N * 4 < ((int64_t)1 << 31)) {
      int smax = (int)(cu / tiles);
      if (smax > KT / 8) smax = KT / 8;
      if (smax > 8) smax = 8;
      double bound = best * 0.85;
      for (int s = 2; s <= smax; ++s) {
        const double t = (KT + s - 1) / s * us_tile + (double)s * M * N * 8.0 / bytes_per_us + us_launch;
        if (t < bound) {
          bound = best = t;
          pl.S = s;
        }
      }
    }
  }
  const int64_t tiles128 = (int64_t)((M + 127) / 128) * ((N + 127) / 128);
  if (tiles128 <= cu && K % (w8 ? 16 : 8) == 0 && KT * us_tile_small + 3.0 < best) {
    pl.small = true;
    pl.S = 1;
  }
  pl.tiles = KT / pl.S;
  pl.rem = KT % pl.S;
  return pl;
}
size_t split_bytes(const GemmPlan& pl, int M, int N) { return pl.S > 1 ? (size_t)pl.S * M * N * sizeof(float) : 0; }

template <bool W8, int NI, typename T = BF16>
int launch4(const uint16_t* a, const void* W, const float* scale, const EpiArgs& ep, uint16_t* c, int M, int N, int K,
            int64_t lda, int64_t ldw, int64_t ldc, int epilogue, hipStream_t s, const Taps* taps = nullptr,
            float* ws = nullptr, size_t ws_bytes = 0) {
  const int tiles_t = (M + BT - 1) / BT, tiles_c = (N + 64 * NI - 1) / (64 * NI);
  dim3 grid((unsigned)(tiles_t * tiles_c)), block(256);
  const Taps none = {0, 0, 0, 0, 0, nullptr};
  if constexpr (NI != 2) {  // the 128-wide tile exists unsplit and without taps only
    if (!taps && ws) {  // split-k when it pays and the caller's workspace holds the partial planes
      const GemmPlan pl = plan_gemm(M, N, K, W8);
      if (pl.S > 1 && ws_bytes >= split_bytes(pl, M, N)) {
        const Taps split = {0, 0, 0, pl.tiles, pl.rem, nullptr};
        hipLaunchKernelGGL((gemm4_kernel<W8, SANA_EPI_NONE, NI, 0, true, T>), dim3(grid.x, (unsigned)pl.S), block, 0, s,
                           a, W, scale, ep, reinterpret_cast<uint16_t*>(ws), M, N, K, lda, ldw, ldc, tiles_t, tiles_c,
                           split);
        if (hipGetLastError() != hipSuccess) return SANA_ERR_LAUNCH;
        const int64_t threads = (int64_t)M * (N / 8);
        dim3 egrid((unsigned)((threads + 255) / 256));
#define SANA_SPLIT_EPI(EPI) \
  hipLaunchKernelGGL((splitk_epilogue_kernel<EPI, T>), egrid, block, 0, s, ws, pl.S, ep, c, M, N, ldc)
        switch (epilogue) {
          case SANA_EPI_NONE: SANA_SPLIT_EPI(SANA_EPI_NONE); break;
          case SANA_EPI_BIAS: SANA_SPLIT_EPI(SANA_EPI_BIAS); break;
          case SANA_EPI_BIAS_SILU: SANA_SPLIT_EPI(SANA_EPI_BIAS_SILU); break;
          case SANA_EPI_GATE_RES: SANA_SPLIT_EPI(SANA_EPI_GATE_RES); break;
          default: return SANA_ERR_ARG;
        }
#undef SANA_SPLIT_EPI
        return hipGetLastError() == hipSuccess ? SANA_OK : SANA_ERR_LAUNCH;
      }
    }
    if (taps) {  // only the bf16 gated-residual instance exists with taps
      if (W8 || is_f16<T> || epilogue != SANA_EPI_GATE_RES) return SANA_ERR_ARG;
      if (taps->zero_last)
        hipLaunchKernelGGL((gemm4_kernel<false, SANA_EPI_GATE_RES, NI, 2>), grid, block, 0, s, a, W, scale, ep, c, M, N, K,
                           lda, ldw, ldc, tiles_t, tiles_c, *taps);
      else
        hipLaunchKernelGGL((gemm4_kernel<false, SANA_EPI_GATE_RES, NI, 1>), grid, block, 0, s, a, W, scale, ep, c, M, N, K,
                           lda, ldw, ldc, tiles_t, tiles_c, *taps);
      return hipGetLastError() == hipSuccess ? SANA_OK : SANA_ERR_LAUNCH;
    }
  } else {
    if (taps) return SANA_ERR_ARG;
  }
#define SANA_LAUNCH4(EPI)                                                                                         \
  hipLaunchKernelGGL((gemm4_kernel<W8, EPI, NI, 0, false, T>), grid, block, 0, s, a, W, scale, ep, c, M, N, K, lda, ldw, ldc, \
                     tiles_t, tiles_c, none)
  switch (epilogue) {
    case SANA_EPI_NONE: SANA_LAUNCH4(SANA_EPI_NONE); break;
    case SANA_EPI_BIAS: SANA_LAUNCH4(SANA_EPI_BIAS); break;
    case SANA_EPI_BIAS_SILU: SANA_LAUNCH4(SANA_EPI_BIAS_SILU); break;
    case SANA_EPI_GATE_RES: SANA_LAUNCH4(SANA_EPI_GATE_RES); break;
    default: return SANA_ERR_ARG;
  }
#undef SANA_LAUNCH4
  return hipGetLastError() == hipSuccess ? SANA_OK : SANA_ERR_LAUNCH;
}

template <bool W8, typename T = BF16>
int launch_small(const uint16_t* a, const void* W, const float* scale, const EpiArgs& ep, uint16_t* c, int M, int N,
                 int K, int64_t lda, int64_t ldw, int64_t ldc, int epilogue, hipStream_t s) {
  const int tiles_t = (M + 127) / 128, tiles_c = (N + 127) / 128;
  dim3 grid((unsigned)(tiles_t * tiles_c)), block(256);
#define SANA_LAUNCH_S(EPI)                                                                                          \
  hipLaunchKernelGGL((gemm_kernel<W8, EPI, 2, 2, T>), grid, block, 0, s, a, W, scale, ep, c, M, N, K, lda, ldw, ldc, \
                     tiles_t, tiles_c)
  switch (epilogue) {
    case SANA_EPI_NONE: SANA_LAUNCH_S(SANA_EPI_NONE); break;
    case SANA_EPI_BIAS: SANA_LAUNCH_S(SANA_EPI_BIAS); break;
    case SANA_EPI_BIAS_SILU: SANA_LAUNCH_S(SANA_EPI_BIAS_SILU); break;
    case SANA_EPI_GATE_RES: SANA_LAUNCH_S(SANA_EPI_GATE_RES); break;
    default: return SANA_ERR_ARG;
  }
#undef SANA_LAUNCH_S
  return hipGetLastError() == hipSuccess ? SANA_OK : SANA_ERR_LAUNCH;
}

template <bool W8, typename T = BF16>
int launch(const void* A, const void* W, const float* scale, const EpiArgs& ep, void* C, int M, int N, int K,
           int64_t lda, int64_t ldw, int64_t ldc, int epilogue, hipStream_t s, const Taps* taps = nullptr,
           void* workspace = nullptr, size_t workspace_bytes = 0) {
  const int64_t tiles_t = (M + BT - 1) / BT;
  if (tiles_t * ((N + 127) / 128) > (1 << 30)) return SANA_ERR_SHAPE;
  const uint16_t* a = static_cast<const uint16_t*>(A);
  uint16_t* c = static_cast<uint16_t*>(C);
  if (!taps && plan_gemm(M, N, K, W8).small)
    return launch_small<W8, T>(a, W, scale, ep, c, M, N, K, lda, ldw, ldc, epilogue, s);
  if (K % 32 == 0 && K >= 64) {  // the pipelined kernel; the generic one takes any K % 8 == 0 (int8: K % 16 == 0)
    float* ws = aligned16(workspace) ? static_cast<float*>(workspace) : nullptr;
    // Mixed channel tiling: the first n_wide channels in 256-wide tiles, the rest in 192-wide ones, as two launches
    // over disjoint column ranges of C, when that needs fewer rounds of the chip than either width alone (qkv at
    // 16384 tokens, N = 6720: 27 x 256 is 7 rounds of 256 tiles, 24 x 256 + 3 x 192 is 6 rounds + one of 192-wide
    // tiles, 6.8 round-equivalents).  Same k order per output: bit-identical to the single launch.
    if (!taps && plan_gemm(M, N, K, W8).S == 1) {
      const int n_wide = mixed_split(M, N);
      if (n_wide > 0) {
        const int rc = launch4<W8, 4, T>(a, W, scale, ep, c, M, n_wide, K, lda, ldw, ldc, epilogue, s, nullptr, nullptr, 0);
        if (rc != SANA_OK) return rc;
        EpiArgs ep2 = ep;
        if (ep2.bias) ep2.bias += n_wide;
        if (ep2.gate) ep2.gate += n_wide;
        if (ep2.res) ep2.res += n_wide;
        return launch4<W8, 3, T>(a, static_cast<const char*>(W) + (int64_t)n_wide * ldw * (W8 ? 1 : 2),
                              scale ? scale + n_wide : nullptr, ep2, c + n_wide, M, N - n_wide, K, lda, ldw, ldc, epilogue,
                              s, nullptr, nullptr, 0);
      }
    }
    // Few tokens, wide N (qkv of one 1024 px image: 4 x 35 tiles of 192 channels on 256 CUs): 128-wide tiles put
    // half as much math behind every k-tile of the chain and fill more of the chip (4 x 53 workgroups: 37 -> 31 us).
    // Taken when the 192-wide grid leaves a fifth of the CUs idle and the 128-wide one still fits.
    {
      const int64_t t128 = tiles_t * ((N + 127) / 128), t192 = tiles_t * ((N + 191) / 192);
      if (!taps && t128 <= compute_units() && t192 < compute_units() * 4 / 5 && plan_gemm(M, N, K, W8).S == 1)
        return launch4<W8, 2, T>(a, W, scale, ep, c, M, N, K, lda, ldw, ldc, epilogue, s, nullptr, nullptr, 0);
    }
    return pick_ni(M, N) == 3
               ? launch4<W8, 3, T>(a, W, scale, ep, c, M, N, K, lda, ldw, ldc, epilogue, s, taps, ws, workspace_bytes)
               : launch4<W8, 4, T>(a, W, scale, ep, c, M, N, K, lda, ldw, ldc, epilogue, s, taps, ws, workspace_bytes);
  }
  if (taps) return SANA_ERR_SHAPE;
  const int tiles_c = (N + BC - 1) / BC;
  dim3 grid((unsigned)(tiles_t * tiles_c)), block(256);
#define SANA_LAUNCH(EPI)                                                                                        \
  hipLaunchKernelGGL((gemm_kernel<W8, EPI, 4, 4, T>), grid, block, 0, s, a, W, scale, ep, c, M, N, K, lda, ldw, ldc, \
                     (int)tiles_t, tiles_c)
  switch (epilogue) {
    case SANA_EPI_NONE: SANA_LAUNCH(SANA_EPI_NONE); break;
    case SANA_EPI_BIAS: SANA_LAUNCH(SANA_EPI_BIAS); break;
    case SANA_EPI_BIAS_SILU: SANA_LAUNCH(SANA_EPI_BIAS_SILU); break;
    case SANA_EPI_GATE_RES: SANA_LAUNCH(SANA_EPI_GATE_RES); break;
    default: return SANA_ERR_ARG;
  }
#undef SANA_LAUNCH
  return hipGetLastError() == hipSuccess ? SANA_OK : SANA_ERR_LAUNCH;
}

int check_common(const void* A, const void* W, const void* bias, const void* C, int M, int N, int K, int64_t lda,
                 int64_t ldw, int64_t ldc, int epilogue, int kmult, int ldw_mult) {
  if (!A || !W || !C || M <= 0 || N <= 0 || K <= 0) return SANA_ERR_ARG;
  if ((epilogue == SANA_EPI_BIAS || epilogue == SANA_EPI_BIAS_SILU) && !bias) return SANA_ERR_ARG;
  if (epilogue < SANA_EPI_NONE || epilogue > SANA_EPI_GATE_RES) return SANA_ERR_ARG;
  if (K % kmult || N % 8) return SANA_ERR_SHAPE;
  if (lda < K || ldw < K || ldc < N) return SANA_ERR_ARG;
  if (lda >= (1 << 22) || ldw >= (1 << 22) || ldc >= (1 << 22)) return SANA_ERR_SHAPE;  // 32-bit offsets inside a tile's rows
  if (lda % 8 || ldw % ldw_mult || ldc % 8 || !aligned16(A) || !aligned16(W) || !aligned16(C)) return SANA_ERR_ALIGN;
  return SANA_OK;
}

int check_gate_res(const void* gate, const void* residual, int M, int N, int64_t ldr, int rows_per_gate,
                   int64_t gate_stride) {
  if (!gate || !residual || rows_per_gate <= 0) return SANA_ERR_ARG;
  if (ldr < N || gate_stride < 0) return SANA_ERR_ARG;
  if (ldr % 8 || gate_stride % 8 || !aligned16(gate) || !aligned16(residual)) return SANA_ERR_ALIGN;
  return SANA_OK;
}

// Sum of the per-token-tile partial states of the fused qkv projection: part[bh][nsplit][33 * 32] -> state[bh][33 * 32].
// One thread per element of one (batch, head) adds G-th tiles in tile order (batches of eight independent loads);
// with G = 4 (many tiles per batch entry) four threads share an element and their sums are added in a fixed order.
// Deterministic either way.
template <int G>
__global__ __launch_bounds__(256) void qkv_state_reduce_kernel(const float* __restrict__ part, float* __restrict__ state,
                                                                int nsplit, int total) {
  constexpr int ELEMS = 33 * 32, PER = 256 / G;
  __shared__ float red[G][PER];
  const int local = threadIdx.x % PER, grp = threadIdx.x / PER;
  const int gid = blockIdx.x * PER + local;  // element of the whole state array
  float s = 0.f;
  if (gid < total) {
    const int bh = gid / ELEMS, e = gid - bh * ELEMS;
    const float* p = part + ((int64_t)bh * nsplit) * ELEMS + e;
    for (int sp0 = grp; sp0 < nsplit; sp0 += 8 * G) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = (sp0 + G * u < nsplit) ? p[(int64_t)(sp0 + G * u) * ELEMS] : 0.f;
#pragma unroll
      for (int u = 0; u < 8; ++u) s += v[u];
    }
  }
  if (G == 1) {
    if (gid < total) state[gid] = s;
    return;
  }
  red[grp][local] = s;
  __syncthreads();
  if (grp == 0 && gid < total) {
    float t = red[0][local];
#pragma unroll
    for (int g = 1; g < G; ++g) t += red[g][local];
    state[gid] = t;
  }
}

// Rows of the fused qkv projection's weight layout for C = 32 * heads channels: the q rows padded to whole 256-wide
// tiles, then one tile per four heads, [K h | V h | K h+1 | V h+1] for the tile's first and second pair of heads.
int qkv_state_q_pad(int C) { return (C + 255) / 256 * 256; }
int qkv_state_rows_total(int C, int heads) { return qkv_state_q_pad(C) + (heads + 3) / 4 * 256; }

EpiArgs plain_epi(const void* bias) {
  EpiArgs e = {static_cast<const uint16_t*>(bias), nullptr, nullptr, 0, 0, 1, nullptr, 0, 0, 0, 0};
  return e;
}

}  // namespace
}  // namespace sana

using namespace sana;

#define SANA_API extern "C" __attribute__((visibility("default")))

SANA_API size_t sana_hip_gemm_workspace_bytes(int M, int N, int K) {
  if (M <= 0 || N <= 0 || K <= 0 || N % 8) return 0;
  return split_bytes(plan_gemm(M, N, K, false), M, N);
}

SANA_API int sana_hip_gemm_bf16(const void* A, const void* W, const void* bias, void* C, int M, int N, int K,
                                int64_t lda, int64_t ldw, int64_t ldc, int epilogue, void* workspace,
                                size_t workspace_bytes, void* stream) {
  if (epilogue == SANA_EPI_GATE_RES) return SANA_ERR_ARG;
  const int rc = check_common(A, W, bias, C, M, N, K, lda, ldw, ldc, epilogue, 8, 8);
  if (rc != SANA_OK) return rc;
  return launch<false>(A, W, nullptr, plain_epi(bias), C, M, N, K, lda, ldw, ldc, epilogue,
                       static_cast<hipStream_t>(stream), nullptr, workspace, workspace_bytes);
}

SANA_API int sana_hip_gemm_f16(const void* A, const void* W, const void* bias, void* C, int M, int N, int K,
                               int64_t lda, int64_t ldw, int64_t ldc, int epilogue, void* workspace,
                               size_t workspace_bytes, void* stream) {
  if (epilogue == SANA_EPI_GATE_RES) return SANA_ERR_ARG;
  const int rc = check_common(A, W, bias, C, M, N, K, lda, ldw, ldc, epilogue, 8, 8);
  if (rc != SANA_OK) return rc;
  return launch<false, F16>(A, W, nullptr, plain_epi(bias), C, M, N, K, lda, ldw, ldc, epilogue,
                            static_cast<hipStream_t>(stream), nullptr, workspace, workspace_bytes);
}

SANA_API int sana_hip_gemm_w8a16(const void* A, const int8_t* Wq, const float* scale, const void* bias, void* C,
                                 int M, int N, int K, int64_t lda, int64_t ldw, int64_t ldc, int epilogue,
                                 void* workspace, size_t workspace_bytes, void* stream) {
  if (!scale || epilogue == SANA_EPI_GATE_RES) return SANA_ERR_ARG;
  const int rc = check_common(A, Wq, bias, C, M, N, K, lda, ldw, ldc, epilogue, 16, 16);
  if (rc != SANA_OK) return rc;
  return launch<true>(A, Wq, scale, plain_epi(bias), C, M, N, K, lda, ldw, ldc, epilogue,
                      static_cast<hipStream_t>(stream), nullptr, workspace, workspace_bytes);
}

SANA_API int sana_hip_gemm_gate_residual(const void* A, const void* W, const float* w8_scale, const void* bias,
                                         const void* gate, const void* residual, void* C, int M, int N, int K,
                                         int64_t lda, int64_t ldw, int64_t ldr, int64_t ldc, int rows_per_gate,
                                         int64_t gate_stride, void* workspace, size_t workspace_bytes,
                                         void* stream) {
  const bool w8 = w8_scale != nullptr;
  int rc = check_common(A, W, bias, C, M, N, K, lda, ldw, ldc, SANA_EPI_GATE_RES, w8 ? 16 : 8, w8 ? 16 : 8);
  if (rc != SANA_OK) return rc;
  rc = check_gate_res(gate, residual, M, N, ldr, rows_per_gate, gate_stride);
  if (rc != SANA_OK) return rc;
  const EpiArgs e = {static_cast<const uint16_t*>(bias), static_cast<const uint16_t*>(gate),
                     static_cast<const uint16_t*>(residual), ldr, gate_stride, rows_per_gate, nullptr, 0, 0, 0, 0};
  hipStream_t s = static_cast<hipStream_t>(stream);
  return w8 ? launch<true>(A, W, w8_scale, e, C, M, N, K, lda, ldw, ldc, SANA_EPI_GATE_RES, s, nullptr, workspace,
                           workspace_bytes)
            : launch<false>(A, W, nullptr, e, C, M, N, K, lda, ldw, ldc, SANA_EPI_GATE_RES, s, nullptr, workspace,
                            workspace_bytes);
}

SANA_API int sana_hip_gemm_gate_residual_f16(const void* A, const void* W, const void* bias, const void* gate,
                                             const void* residual, void* C, int M, int N, int K, int64_t lda,
                                             int64_t ldw, int64_t ldr, int64_t ldc, int rows_per_gate,
                                             int64_t gate_stride, void* workspace, size_t workspace_bytes,
                                             void* stream) {
  int rc = check_common(A, W, bias, C, M, N, K, lda, ldw, ldc, SANA_EPI_GATE_RES, 8, 8);
  if (rc != SANA_OK) return rc;
  rc = check_gate_res(gate, residual, M, N, ldr, rows_per_gate, gate_stride);
  if (rc != SANA_OK) return rc;
  const EpiArgs e = {static_cast<const uint16_t*>(bias), static_cast<const uint16_t*>(gate),
                     static_cast<const uint16_t*>(residual), ldr, gate_stride, rows_per_gate, nullptr, 0, 0, 0, 0};
  return launch<false, F16>(A, W, nullptr, e, C, M, N, K, lda, ldw, ldc, SANA_EPI_GATE_RES,
                            static_cast<hipStream_t>(stream), nullptr, workspace, workspace_bytes);
}

SANA_API int sana_hip_tconv_residual(const void* X, const void* W, void* out, int M, int C, int taps,
                                     int64_t tap_rows, int64_t x_rows, const unsigned char* zero_last_tap,
                                     int64_t ldx, int64_t ldw, int64_t ldo, void* stream) {
  if (!X || !W || !out || M <= 0 || C <= 0 || taps <= 0 || !(taps & 1) || tap_rows <= 0) return SANA_ERR_ARG;
  if (zero_last_tap && taps < 3) return SANA_ERR_ARG;
  if (C % 64) return SANA_ERR_SHAPE;  // a tap is a whole number of k-tiles
  if (x_rows < (taps / 2) * tap_rows + M) return SANA_ERR_ARG;  // the centre tap (= the residual) must exist for every row
  if (ldx < C || ldw < (int64_t)taps * C || ldo < C) return SANA_ERR_ARG;
  if (ldx % 8 || ldw % 8 || ldo % 8 || !aligned16(X) || !aligned16(W) || !aligned16(out)) return SANA_ERR_ALIGN;
  if (x_rows * ldx * 2 >= ((int64_t)1 << 31)) return SANA_ERR_SHAPE;  // 32-bit byte offsets inside the buffer
  const uint16_t* x = static_cast<const uint16_t*>(X);
  const EpiArgs e = {nullptr, nullptr, x + (taps / 2) * tap_rows * ldx, ldx, 0, M, nullptr, 0, 0, 0, 0};
  const Taps tp = {C, tap_rows, x_rows, 0, 0, zero_last_tap};
  return launch<false>(X, W, nullptr, e, out, M, C, taps * C, ldx, ldw, ldo, SANA_EPI_GATE_RES,
                       static_cast<hipStream_t>(stream), &tp);
}

SANA_API int sana_hip_dequant_w8(const int8_t* Wq, const float* scale, void* W, int N, int K, int64_t ldw,
                                 int64_t ldo, void* stream) {
  if (!Wq || !scale || !W || N <= 0 || K <= 0) return SANA_ERR_ARG;
  if (K % 16) return SANA_ERR_SHAPE;
  if (ldw < K || ldo < K) return SANA_ERR_ARG;
  if (ldw % 16 || ldo % 8 || !aligned16(Wq) || !aligned16(W)) return SANA_ERR_ALIGN;
  const int64_t threads = (int64_t)N * (K / 16);
  if ((threads + 255) / 256 > 0x7fffffff) return SANA_ERR_SHAPE;
  hipLaunchKernelGGL(dequant_w8_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), Wq, scale, static_cast<uint16_t*>(W), N, K, ldw, ldo);
  return hipGetLastError() == hipSuccess ? SANA_OK : SANA_ERR_LAUNCH;
}

SANA_API int sana_hip_qkv_state_rows(int C, int heads, int32_t* rows, int capacity) {
  if (C <= 0 || heads <= 0 || C != 32 * heads) return SANA_ERR_SHAPE;
  const int q_pad = qkv_state_q_pad(C), total = qkv_state_rows_total(C, heads);
  if (!rows) return total;
  if (capacity < total) return SANA_ERR_ARG;
  for (int i = 0; i < q_pad; ++i) rows[i] = i < C ? i : -1;
  for (int i = q_pad; i < total; ++i) {
    const int l = (i - q_pad) & 255, tile = (i - q_pad) >> 8;
    const int head = 4 * tile + 2 * (l >> 7) + ((l >> 6) & 1), is_v = (l >> 5) & 1, e = l & 31;
    rows[i] = head < heads ? (1 + is_v) * C + 32 * head + e : -1;
  }
  return total;
}

SANA_API size_t sana_hip_gemm_qkv_state_workspace_bytes(int B, int N, int heads) {
  if (B <= 0 || N <= 0 || heads <= 0 || (N % 256 && B != 1)) return 0;
  return (size_t)B * heads * ((N + 255) / 256) * 33 * 32 * sizeof(float);
}

SANA_API int sana_hip_gemm_qkv_state(const void* A, const void* W_tiled, const void* bias_tiled, void* Q, float* state,
                                     void* workspace, size_t workspace_bytes, int B, int N, int C, int heads,
                                     int64_t lda, int64_t ldw, int64_t ldq, void* stream) {
  if (!A || !W_tiled || !Q || !state || B <= 0 || N <= 0 || C <= 0 || heads <= 0) return SANA_ERR_ARG;
  if (C != 32 * heads || C < 64) return SANA_ERR_SHAPE;
  // a token tile must not straddle two batch entries, and the rows of a ragged last tile must contribute nothing to
  // the state: they read as zero activations, which stay zero only without a bias
  if (N % 256 && (B != 1 || bias_tiled)) return SANA_ERR_SHAPE;
  if ((int64_t)B * N >= ((int64_t)1 << 30) || (int64_t)B * heads * 33 * 32 >= ((int64_t)1 << 31)) return SANA_ERR_SHAPE;
  const int M = B * N, rows_t = qkv_state_rows_total(C, heads);
  if (lda < C || ldw < C || ldq < C) return SANA_ERR_ARG;
  if (lda >= (1 << 22) || ldw >= (1 << 22) || ldq >= (1 << 22)) return SANA_ERR_SHAPE;
  if (lda % 8 || ldw % 8 || ldq % 8 || !aligned16(A) || !aligned16(W_tiled) || !aligned16(Q) ||
      (bias_tiled && !aligned16(bias_tiled)) || !aligned16(state))
    return SANA_ERR_ALIGN;
  const size_t need = sana_hip_gemm_qkv_state_workspace_bytes(B, N, heads);
  if (!workspace || workspace_bytes < need) return SANA_ERR_WORKSPACE;
  if (!aligned16(workspace)) return SANA_ERR_ALIGN;
  const int64_t tiles_t = (M + BT - 1) / BT, tiles_c = rows_t / 256;
  if (tiles_t * tiles_c > (1 << 30)) return SANA_ERR_SHAPE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const EpiArgs e = {static_cast<const uint16_t*>(bias_tiled), nullptr, nullptr, 0, 0, 1, static_cast<float*>(workspace),
                     C, qkv_state_q_pad(C), heads, (N + 255) / 256};
  const Taps none = {0, 0, 0, 0, 0, nullptr};
  hipLaunchKernelGGL((gemm4_kernel<false, SANA_EPI_QKV_STATE, 4>), dim3((unsigned)(tiles_t * tiles_c)), dim3(256), 0, s,
                     static_cast<const uint16_t*>(A), W_tiled, static_cast<const float*>(nullptr), e,
                     static_cast<uint16_t*>(Q), M, rows_t, C, lda, ldw, ldq, (int)tiles_t, (int)tiles_c, none);
  if (hipGetLastError() != hipSuccess) return SANA_ERR_LAUNCH;
  const int total = B * heads * 33 * 32, nsplit = (N + 255) / 256;
  if (nsplit > 16)
    hipLaunchKernelGGL(qkv_state_reduce_kernel<4>, dim3((unsigned)((total + 63) / 64)), dim3(256), 0, s,
                       static_cast<const float*>(workspace), state, nsplit, total);
  else
    hipLaunchKernelGGL(qkv_state_reduce_kernel<1>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s,
                       static_cast<const float*>(workspace), state, nsplit, total);
  return hipGetLastError() == hipSuccess ? SANA_OK : SANA_ERR_LAUNCH;
}
