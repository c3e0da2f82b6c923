// ReLU linear attention for head_dim 112 (the `linear_head_dim: 112` video configurations) on gfx950,
// bf16 / f16 io.  Same two phases and the same state layout as the head_dim-32 kernels --
// fp32 [B][h][n_chunks][113][112], row 112 = sum_n relu(k_n) -- but one head is now a 112 x 112
// problem of its own (3.5 x 3.5 MFMA tiles, padded to 4 x 4 with zero channels):
//
//   phase 1  workgroup = (batch, head, chunk, token split); each of its four waves takes interleaved
//            32-token tiles (16 with on-load transforms) and owns a whole 128 x 128 accumulator (256
//            registers).  Tiles go through wave-private LDS to become token-contiguous MFMA operands, as
//            in the head_dim-32 kernel; the waves are summed in LDS (two padded accumulator images) and
//            a second kernel sums the splits in a fixed order.
//   phase 2  workgroup = (batch, head, chunk, range of 192..512 tokens), steps of 32 tokens through
//            workgroup-shared LDS tiles; wave w produces output channels [32w, 32w+32) from its own slice
//            of the state (two bf16 terms of the fp32 values as MFMA 16x16x32 A operands for bf16 output,
//            three for fp32 output) plus a row block that carries ksum in every row, so each lane gets
//            its token's denominator.
#include "common.h"
#include "linattn_common.h"

namespace sana {
namespace {

constexpr int DH = 112;                 // head dim
constexpr int SE = (DH + 1) * DH;       // 12656 state elements per (batch, head, chunk)
constexpr int NCH = DH / 8;             // 14 16-byte chunks per token and head
constexpr int TILE = 32;

// Workgroup index -> (unit of four adjacent heads, head within it).  Four 224-byte head rows are seven whole
// 128-byte lines; a single head's row shares its first / last line with a neighbour.  Workgroup i runs on XCD
// i % 8, so the four heads of a unit take consecutive slots of ONE XCD: the shared lines are then fetched into
// one L2, once, instead of into two.  Returns false for the padding of the grid.
struct HeadUnit {
  int unit, head;
};
__device__ __forceinline__ bool head_unit(int idx, int units, int h, HeadUnit& u) {
  const int xcd = idx & 7, slot = idx >> 3;
  const int hgroups = (h + 3) >> 2;
  const int un = (slot >> 2) * 8 + xcd;
  u.unit = un / hgroups;
  u.head = (un - u.unit * hgroups) * 4 + (slot & 3);
  return un < units * hgroups && u.head < h;
}
inline int64_t head_unit_grid(int64_t units, int h) { return (units * ((h + 3) / 4) + 7) / 8 * 8 * 4; }

// ----------------------------------------------------------------------------
// phase 1.  1-D grid over units (batch, chunk, token split) x heads, see head_unit; block 256.
// partial[(bh * n_chunks + c) * nsplit + split][SE]
// ----------------------------------------------------------------------------
constexpr int LR = 160;  // LDS tile row stride in elements: 320 B puts the two token groups of a read 16 banks apart
constexpr int SMEM_BYTES = 2 * 128 * 128 * 4;  // two padded fp32 accumulator images for the wave reduction
                                             // (>= 4 waves x 2 tiles x 33 x LR x 2 B of staging)
static_assert(SMEM_BYTES >= 4 * 2 * (TILE + 1) * LR * 2, "staging must fit");

// PRE: on-load transforms, compile-time so that the tile code stays one branch-free block: bit 0 = q/k RMSNorm,
// bit 1 = rotary embedding
template <typename T, int PRE>
__global__ __launch_bounds__(256) void state112_kernel(const uint16_t* __restrict__ K, const uint16_t* __restrict__ V,
                                                       float* __restrict__ partial,
                                                       const int32_t* __restrict__ chunk_starts, int N, int h,
                                                       int n_chunks, int nsplit, int split_tokens, int units,
                                                       int64_t stride_b, int64_t stride_n, const QkPre pre) {
  __shared__ __attribute__((aligned(16))) unsigned char smem[SMEM_BYTES];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  HeadUnit hu;
  if (!head_unit(blockIdx.x, units, h, hu)) return;  // uniform over the workgroup
  const int head = hu.head;
  const int split = hu.unit % nsplit, c = (hu.unit / nsplit) % n_chunks, b = hu.unit / (nsplit * n_chunks);
  const ChunkRange cr = chunk_range(chunk_starts, c, N);
  const int t0 = cr.begin + split * split_tokens;
  const int t1 = min(cr.end, t0 + split_tokens);
  // tokens per tile: 32, or 16 with transforms (their operands -- rotary factors above all -- travel with the
  // tile, and a 32-token tile of them does not fit the registers next to the accumulator)
  constexpr int TT_ = PRE ? 16 : TILE;
  constexpr int TROWS = TT_ + 1;  // one spare row per tile: where the idle lanes of the transform mapping write
  uint16_t* lds_k = reinterpret_cast<uint16_t*>(smem) + wave * (2 * TROWS * LR);
  uint16_t* lds_v = lds_k + TROWS * LR;
  // channels 112..127 of every tile row are written once, as zeros, and never again
  for (int i = lane; i < 2 * TROWS * 2; i += 64) {  // (K rows, V rows) x 2 chunks of 8
    const int row = i >> 1, chunk = NCH + (i & 1);
    *reinterpret_cast<u32x4_t*>(lds_k + row * LR + chunk * 8) = u32x4_t{0u, 0u, 0u, 0u};
  }

  // load mapping, consecutive lanes on consecutive 16-byte pieces of a token's 224-byte head row:
  //   plain      piece id = lane + 64 i (i < 7): token id / 14, piece id % 14
  //   transforms lanes 0..55: token 4 i + lane / 14 (i < 4), piece lane % 14 -- a lane keeps ONE piece, so its norm
  //              weights are loop invariant and its ksum is 8 registers; the other 8 lanes load nothing (zeros)
  //              and write them to the spare row
  constexpr int NSLOT = PRE ? 4 : 7;
  const bool lane_ok = !PRE || lane < 4 * NCH;
  int ld_tok[NSLOT], ld_ch[NSLOT];
#pragma unroll
  for (int i = 0; i < NSLOT; ++i) {
    const int id = PRE ? 4 * NCH * i + lane : lane + 64 * i;
    ld_tok[i] = lane_ok ? id / NCH : TT_;
    ld_ch[i] = lane_ok ? id - (id / NCH) * NCH : lane - 4 * NCH;
  }
  const uint16_t* kbase = K + (int64_t)b * stride_b + head * DH;
  const uint16_t* vbase = V + (int64_t)b * stride_b + head * DH;
  constexpr bool has_norm = (PRE & 1) != 0, has_rope = (PRE & 2) != 0;

  f32x16_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  float acck[4] = {0.f, 0.f, 0.f, 0.f};  // ksum of channel 32 jb + lane % 32 over this lane's token half
  const u32x4_t zero4 = {0u, 0u, 0u, 0u};
  // The next tile's loads (and what its transforms need: 1/rms, rotary factors) are in flight during the MFMAs
  // of the current one.  (A second register set, two tiles ahead, measured no faster.)
  u32x4_t kreg[NSLOT], vreg[NSLOT];
  float rin[has_norm ? NSLOT : 1];
  f32x4_t cs[has_rope ? NSLOT : 1][2];
  u32x4_t kw = zero4;
  if (has_norm && lane_ok) kw = *reinterpret_cast<const u32x4_t*>(pre.weight + head * DH + ld_ch[0] * 8);
  // Buffer loads: a resource ends with the last token of the range, so pieces of tokens past it (and everything
  // of the idle lanes, whose offsets start at 2^31) read as zeros -- no branches or selects around the loads.
  // The range check covers the vector offset only, so the tile's part of the address goes there.
  const int row_b = (int)stride_n * 2;
  const __amdgpu_buffer_rsrc_t rsrc_k = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(kbase), 0, (int)(((int64_t)(t1 - 1) * stride_n + DH) * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_v = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(vbase), 0, (int)(((int64_t)(t1 - 1) * stride_n + DH) * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_r = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>(has_norm ? pre.rinv + (int64_t)b * N : nullptr), 0, has_norm ? t1 * 4 : 0, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_c = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>(pre.rope), 0, has_rope ? t1 * (DH * 4) : 0, 0x00020000);
  const int idle = (int)0x80000000u;
  int voff[NSLOT];
#pragma unroll
  for (int i = 0; i < NSLOT; ++i) voff[i] = lane_ok ? ld_tok[i] * row_b + ld_ch[i] * 16 : idle;
  auto issue_loads = [&](int tile) {
#pragma unroll
    for (int i = 0; i < NSLOT; ++i) {
      const int off = tile * row_b + voff[i];
      kreg[i] = __builtin_bit_cast(u32x4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc_k, off, 0, 0));
      vreg[i] = __builtin_bit_cast(u32x4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc_v, off, 0, 0));
      if (PRE) {
        const int tok = lane_ok ? tile + ld_tok[i] : idle / (DH * 4);
        if (has_norm) rin[i] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc_r, tok * 4, 0, 0));
        if (has_rope) {
          const int ro = tok * (DH * 4) + ld_ch[i] * 32;
          cs[i][0] = __builtin_bit_cast(f32x4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc_c, ro, 0, 0));
          cs[i][1] = __builtin_bit_cast(f32x4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc_c, ro + 16, 0, 0));
        }
      }
    }
  };
  // PRE: the MFMA operands in LDS are rotated, ksum needs the unrotated values: a second, unrotated
  // copy of the K tile would double the LDS traffic, so ksum is accumulated per lane and channel
  // here and folded over the lanes that share a piece once at the end
  float ks8[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

  const int tile0 = t0 + wave * TT_;
  if (tile0 < t1) issue_loads(tile0);
  // operand read mapping: lane -> channel j = lane%32 of a 32-channel block, k-group g = lane/32;
  // element r of k-step s is token 16*s + 2*r + g of the tile (both operands use the same bijection)
  const int j = lane & 31, g = lane >> 5;
  for (int tile = tile0; tile < t1; tile += 4 * TT_) {
#pragma unroll
    for (int i = 0; i < NSLOT; ++i) {
      u32x4_t kk = kreg[i];
      if (PRE) {
        if (has_norm) kk = rms_scale8(kk, rin[i], kw);
        kk = relu_pk16(kk);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          ks8[2 * e] += bf16_lo(kk[e]);
          ks8[2 * e + 1] += bf16_hi(kk[e]);
        }
        if (has_rope) kk = rope8(kk, cs[i][0], cs[i][1]);
      } else {
        kk = relu_pk16(kk);
      }
      *reinterpret_cast<u32x4_t*>(lds_k + ld_tok[i] * LR + ld_ch[i] * 8) = kk;
      *reinterpret_cast<u32x4_t*>(lds_v + ld_tok[i] * LR + ld_ch[i] * 8) = vreg[i];
    }
    if (tile + 4 * TT_ < t1) issue_loads(tile + 4 * TT_);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // wave-private LDS: in-order, no barrier needed
#pragma unroll
    for (int s = 0; s < TT_ / 16; ++s) {
      u32x4_t fk[4], fv[4];
#pragma unroll
      for (int blk = 0; blk < 4; ++blk) {
#pragma unroll
        for (int r2 = 0; r2 < 4; ++r2) {
          const int ta = 16 * s + 2 * (2 * r2) + g, tb = 16 * s + 2 * (2 * r2 + 1) + g;
          const uint32_t klo = lds_k[ta * LR + blk * 32 + j], khi = lds_k[tb * LR + blk * 32 + j];
          const uint32_t vlo = lds_v[ta * LR + blk * 32 + j], vhi = lds_v[tb * LR + blk * 32 + j];
          fk[blk][r2] = klo | (khi << 16);
          fv[blk][r2] = vlo | (vhi << 16);
        }
      }
#pragma unroll
      for (int ib = 0; ib < 4; ++ib)
#pragma unroll
        for (int jb = 0; jb < 4; ++jb) acc[ib][jb] = mfma_32x32x16<T>(fv[ib], fk[jb], acc[ib][jb]);
      if (!PRE) {
#pragma unroll
        for (int jb = 0; jb < 4; ++jb)
#pragma unroll
          for (int r2 = 0; r2 < 4; ++r2) acck[jb] = add_pk16<T>(fk[jb][r2], acck[jb]);
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // reads done before the next tile overwrites
  }

  if (PRE) {
    // lanes l, l + 14, l + 28, l + 42 hold the same piece of different tokens: through the wave's own LDS
    // region ([56 lanes][8] floats), then channel 32 jb + j adds its four entries, two per token half g
    float* fold = reinterpret_cast<float*>(lds_k);
    if (lane_ok) {
      *reinterpret_cast<f32x4_t*>(fold + lane * 8) = f32x4_t{ks8[0], ks8[1], ks8[2], ks8[3]};
      *reinterpret_cast<f32x4_t*>(fold + lane * 8 + 4) = f32x4_t{ks8[4], ks8[5], ks8[6], ks8[7]};
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int jb = 0; jb < 4; ++jb) {
      const int ch = jb * 32 + j;
      float sum = 0.f;
      if (ch < DH) {
        const float* f0 = fold + ((2 * g) * NCH + (ch >> 3)) * 8 + (ch & 7);
        sum = f0[0] + f0[NCH * 8];
      }
      acck[jb] = sum;
    }
  }
#pragma unroll
  for (int jb = 0; jb < 4; ++jb) acck[jb] += __shfl_xor(acck[jb], 32, 64);  // the two token halves

  // Cross-wave sum in LDS, two images of the padded 128 x 128 accumulator (no predicates): waves 2, 3 -> images
  // 0, 1; waves 0, 1 add them and write their sums back; then all four waves add the two images and store the
  // 113 x 112 state as whole 16-byte pieces.  ksum travels as row 112 of the image (that accumulator row belongs
  // to a zero channel).  D layout of 32x32 MFMA: lane -> column j = lane%32, register r -> row 8*(r/4) +
  // 4*(lane/32) + r%4.
  float* red = reinterpret_cast<float*>(smem);
  auto put = [&](float* img) {
#pragma unroll
    for (int ib = 0; ib < 4; ++ib)
#pragma unroll
      for (int jb = 0; jb < 4; ++jb)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          img[(ib * 32 + 8 * (r >> 2) + 4 * g + (r & 3)) * 128 + jb * 32 + j] = acc[ib][jb][r];
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the zero row 112 is written before ksum replaces it
    if (g == 0) {
#pragma unroll
      for (int jb = 0; jb < 4; ++jb) img[DH * 128 + jb * 32 + j] = acck[jb];
    }
  };
  auto take = [&](const float* img) {
#pragma unroll
    for (int ib = 0; ib < 4; ++ib)
#pragma unroll
      for (int jb = 0; jb < 4; ++jb)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          acc[ib][jb][r] += img[(ib * 32 + 8 * (r >> 2) + 4 * g + (r & 3)) * 128 + jb * 32 + j];
#pragma unroll
    for (int jb = 0; jb < 4; ++jb) acck[jb] += img[DH * 128 + jb * 32 + j];
  };
  __syncthreads();  // staging tiles are dead
  if (wave >= 2) put(red + (wave - 2) * 128 * 128);
  __syncthreads();
  if (wave < 2) {  // a wave rewrites the image it has just read itself: no barrier in between
    take(red + wave * 128 * 128);
    put(red + wave * 128 * 128);
  }
  __syncthreads();
  {
    const int64_t slot = ((int64_t)(b * h + head) * n_chunks + c) * nsplit + split;
    float* dst = partial + slot * SE;
    for (int p = threadIdx.x; p < (DH + 1) * (DH / 4); p += 256) {  // 16-byte pieces of the 113 x 112 state
      const int row = p / (DH / 4), c4 = p - row * (DH / 4);
      const f32x4_t x0 = *reinterpret_cast<const f32x4_t*>(red + row * 128 + c4 * 4);
      const f32x4_t x1 = *reinterpret_cast<const f32x4_t*>(red + 128 * 128 + row * 128 + c4 * 4);
      *reinterpret_cast<f32x4_t*>(dst + row * DH + c4 * 4) = x0 + x1;
    }
  }
}

// sum of the partials of one state in partial order (+ inclusive prefix over chunks when causal)
__global__ __launch_bounds__(256) void reduce112_kernel(const float* partial, float* state,
                                                        int BH, int n_chunks, int nparts, int causal) {
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (gid >= (int64_t)BH * SE) return;
  const int64_t bh = gid / SE;
  const int e = (int)(gid - bh * SE);
  float run = 0.f;
  for (int c = 0; c < n_chunks; ++c) {
    const float* p0 = partial + ((bh * n_chunks + c) * nparts) * SE + e;
    float s = 0.f;
    for (int sp0 = 0; sp0 < nparts; sp0 += 16) {
      float v[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) v[u] = (sp0 + u < nparts) ? p0[(int64_t)(sp0 + u) * SE] : 0.f;
#pragma unroll
      for (int u = 0; u < 16; ++u) s += v[u];
    }
    if (causal) {
      run += s;
      s = run;
    }
    state[(bh * n_chunks + c) * SE + e] = s;
  }
}

// ----------------------------------------------------------------------------
// phase 2.  1-D grid over units (batch, chunk, token range) x heads, see head_unit; block 256.
//
// The workgroup walks its token range in steps of 32 tokens.  Global memory is touched in whole rows
// only: consecutive threads load consecutive 16-byte pieces of the tokens' 224-byte head rows
// (transforms applied once, here) into an LDS tile, every wave takes its MFMA B operands from that
// tile, results go to an LDS output tile and leave as whole rows again.  Tiles are double buffered,
// the next tile's loads are in flight during the MFMAs: one barrier per step.
// ----------------------------------------------------------------------------
// fp32 -> bf16 terms hi + mid (+ lo), pairwise: one packed convert rounds two values
template <int NT>
__device__ __forceinline__ void split_terms(const float x[8], u32x4_t out[NT]) {
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    float r0 = x[2 * e], r1 = x[2 * e + 1];
#pragma unroll
    for (int term = 0; term < NT; ++term) {
      const uint32_t pk = pack_bf16(r0, r1);
      out[term][e] = pk;
      if (term + 1 < NT) {
        r0 -= bf16_lo(pk);
        r1 -= bf16_hi(pk);
      }
    }
  }
}

constexpr int TT = 32;             // tokens per step
constexpr int QROW = 136;          // LDS row stride of the 16-bit tiles, elements: 272 B = 68 banks, so the 16 tokens
                                   // of a b128 operand read land on 16 disjoint groups of 4 banks; pieces 14
                                   // and 15 of a row (the padded k range 112..127) stay zero
constexpr int OROW32 = 116;        // row stride of the fp32 output tile, floats (same argument: 116 % 64 = 52)

template <bool OUT_F32, int PRE>
__global__ __launch_bounds__(256) void apply112_kernel(const uint16_t* __restrict__ Q, const float* __restrict__ state,
                                                       void* __restrict__ out,
                                                       const int32_t* __restrict__ chunk_starts, int N, int h,
                                                       int n_chunks, int xranges, int wg_tokens, int units,
                                                       int64_t q_stride_b,
                                                       int64_t q_stride_n, int64_t o_stride_b, int64_t o_stride_n,
                                                       float eps, const QkPre pre) {
  constexpr int NQ = (PRE & 2) ? 2 : 1;  // with a rotary embedding: rotated (numerator) and unrotated (denominator) tiles
  constexpr int OT = OUT_F32 ? TT * OROW32 * 2 : TT * QROW;  // output tile, in 16-bit units
  __shared__ __attribute__((aligned(16))) uint16_t lds_q[2 * NQ * TT * QROW];
  __shared__ __attribute__((aligned(16))) uint16_t lds_o[2 * OT];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  HeadUnit hu;
  if (!head_unit(blockIdx.x, units, h, hu)) return;  // uniform over the workgroup
  const int head = hu.head;
  const int bx = hu.unit % xranges, c = (hu.unit / xranges) % n_chunks, b = hu.unit / (xranges * n_chunks);
  const ChunkRange cr = chunk_range(chunk_starts, c, N);
  const int t0 = cr.begin + bx * wg_tokens;
  const int t1 = min(cr.end, t0 + wg_tokens);
  if (t0 >= t1) return;  // uniform over the workgroup
  const int n = lane & 15, g = lane >> 4;
  constexpr bool has_norm = (PRE & 1) != 0, has_rope = (PRE & 2) != 0;

  // A operands.  MFMA 16x16x32: A lane -> row lane%16, k = 8*(lane/16)+e.  Row r of row block rb of this
  // wave is output channel 32*wave + 8*(r/4) + 4*rb + r%4, so that a lane (token n, group g') ends up
  // with the 8 contiguous channels 32*wave + 8*g' .. +7 (registers s of blocks 0 and 1).  Block 2
  // carries ksum in every row.  Channels and k indices past 112 are zero.
  const float* sp = state + ((int64_t)(b * h + head) * n_chunks + c) * SE;
  constexpr int NT = OUT_F32 ? 3 : 2;  // bf16 terms of an fp32 state value: 24 / 16 mantissa bits
  u32x4_t a[3][4][NT];                 // [row block][k block][term]
  {
    // buffer loads: rows / k groups outside the head's state get an out-of-range offset and read as zero
    const __amdgpu_buffer_rsrc_t rsrc_s = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(sp), 0, SE * 4, 0x00020000);
#pragma unroll
    for (int rb = 0; rb < 3; ++rb) {
      const int ch = 32 * wave + 8 * (n >> 2) + 4 * rb + (n & 3);
      const int row = rb < 2 ? ch : DH;
      const bool row_ok = rb == 2 || ch < DH;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) {
        const int k0 = kb * 32 + 8 * g;
        const int off = (row_ok && k0 < DH) ? (row * DH + k0) * 4 : (int)0x80000000u;
        const f32x4_t x0 = __builtin_bit_cast(f32x4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc_s, off, 0, 0));
        const f32x4_t x1 = __builtin_bit_cast(f32x4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc_s, off + 16, 0, 0));
        const float x[8] = {x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
        split_terms<NT>(x, a[rb][kb]);
      }
    }
  }

  // tile load mapping: piece id = tid + 256 i (i < 2, id < 448): token id / 14, 16-byte piece id % 14
  int ld_tok[2], ld_ch[2];
  bool ld_ok[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int id = tid + 256 * i;
    ld_ok[i] = id < TT * NCH;
    ld_tok[i] = id / NCH;
    ld_ch[i] = id - ld_tok[i] * NCH;
  }
  const uint16_t* qp = Q + (int64_t)b * q_stride_b + head * DH;
  const u32x4_t zero4 = {0u, 0u, 0u, 0u};
  const f32x4_t zerof = {0.f, 0.f, 0.f, 0.f};
  u32x4_t qreg[2], qw[2] = {zero4, zero4};
  float rin[2] = {0.f, 0.f};
  f32x4_t cs[2][2] = {{zerof, zerof}, {zerof, zerof}};
  if (has_norm) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
      if (ld_ok[i]) qw[i] = *reinterpret_cast<const u32x4_t*>(pre.weight + head * DH + ld_ch[i] * 8);
  }
  auto issue = [&](int t) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int tok = t + ld_tok[i];
      const bool ok = ld_ok[i] && tok < t1;
      qreg[i] = ok ? *reinterpret_cast<const u32x4_t*>(qp + (int64_t)tok * q_stride_n + ld_ch[i] * 8) : zero4;
      if (has_norm) rin[i] = ok ? pre.rinv[(int64_t)b * N + tok] : 0.f;
      if (has_rope) {
        const float* rp = pre.rope + ((int64_t)min(tok, t1 - 1) * (DH / 2) + ld_ch[i] * 4) * 2;
        cs[i][0] = ok ? *reinterpret_cast<const f32x4_t*>(rp) : zerof;
        cs[i][1] = ok ? *reinterpret_cast<const f32x4_t*>(rp + 4) : zerof;
      }
    }
  };
  auto stage = [&](int buf) {  // registers -> LDS tile(s); tokens past the range are zeros
    uint16_t* td = lds_q + buf * NQ * TT * QROW;  // unrotated: the denominator operand (and the numerator without rope)
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      if (!ld_ok[i]) continue;
      u32x4_t x = qreg[i];
      if (has_norm) x = rms_scale8(x, rin[i], qw[i]);
      x = relu_pk16(x);
      *reinterpret_cast<u32x4_t*>(td + ld_tok[i] * QROW + ld_ch[i] * 8) = x;
      if (has_rope)
        *reinterpret_cast<u32x4_t*>(td + TT * QROW + ld_tok[i] * QROW + ld_ch[i] * 8) = rope8(x, cs[i][0], cs[i][1]);
    }
  };

  const int och = 32 * wave + 8 * g;  // this lane's 8 output channels
  for (int i = tid; i < 2 * NQ * TT * 3; i += 256)  // pieces 14..16 of every q tile row: written once, as zeros
    *reinterpret_cast<u32x4_t*>(lds_q + (i / 3) * QROW + (NCH + i % 3) * 8) = zero4;
  issue(t0);
  stage(0);
  if (t0 + TT < t1) issue(t0 + TT);
  __syncthreads();
  int buf = 0;
  for (int t = t0; t < t1; t += TT, buf ^= 1) {
    const uint16_t* td = lds_q + buf * NQ * TT * QROW;
    const uint16_t* tb = has_rope ? td + TT * QROW : td;
    uint16_t* to = lds_o + buf * OT;
#pragma unroll
    for (int ss = 0; ss < TT / 16; ++ss) {
      u32x4_t qd[4], qb[4];
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) {
        const int off = (16 * ss + n) * QROW + (kb * 4 + g) * 8;  // pieces 14, 15 (kb = 3, g >= 2) hold zeros
        qb[kb] = *reinterpret_cast<const u32x4_t*>(tb + off);
        if (has_rope) qd[kb] = *reinterpret_cast<const u32x4_t*>(td + off);
      }
      f32x4_t acc[3];
#pragma unroll
      for (int rb = 0; rb < 3; ++rb) {
        f32x4_t s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int term = NT - 1; term >= 0; --term)  // smallest term first
#pragma unroll
          for (int kb = 0; kb < 4; ++kb) s = mfma_16x16x32_bf16(a[rb][kb][term], (has_rope && rb == 2) ? qd[kb] : qb[kb], s);
        acc[rb] = s;
      }
      if (och < DH) {
        const float den = acc[2][0] + eps;
        if (OUT_F32) {
          f32x4_t o0, o1;
#pragma unroll
          for (int s = 0; s < 4; ++s) {
            o0[s] = acc[0][s] / den;
            o1[s] = acc[1][s] / den;
          }
          float* op = reinterpret_cast<float*>(to) + (16 * ss + n) * OROW32 + och;
          *reinterpret_cast<f32x4_t*>(op) = o0;
          *reinterpret_cast<f32x4_t*>(op + 4) = o1;
        } else {
          const float inv = __builtin_amdgcn_rcpf(den);
          u32x4_t o;
          o.x = pack_bf16(acc[0][0] * inv, acc[0][1] * inv);
          o.y = pack_bf16(acc[0][2] * inv, acc[0][3] * inv);
          o.z = pack_bf16(acc[1][0] * inv, acc[1][1] * inv);
          o.w = pack_bf16(acc[1][2] * inv, acc[1][3] * inv);
          *reinterpret_cast<u32x4_t*>(to + (16 * ss + n) * QROW + och) = o;
        }
      }
    }
    // next tile: registers -> the other q tile (its last readers passed the previous barrier); loads of the one after
    if (t + TT < t1) {
      stage(buf ^ 1);
      if (t + 2 * TT < t1) issue(t + 2 * TT);
    }
    __syncthreads();
    // this step's output tile leaves as whole rows (it is next written two steps from now, behind the next barrier)
    if (OUT_F32) {
      float* ob = reinterpret_cast<float*>(out) + (int64_t)b * o_stride_b + head * DH;
      const float* tf = reinterpret_cast<const float*>(to);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int id = tid + 256 * i, tok = id / (2 * NCH), piece = id - tok * (2 * NCH);
        if (id < TT * 2 * NCH && t + tok < t1)
          *reinterpret_cast<f32x4_t*>(ob + (int64_t)(t + tok) * o_stride_n + piece * 4) =
              *reinterpret_cast<const f32x4_t*>(tf + tok * OROW32 + piece * 4);
      }
    } else {
      uint16_t* ob = reinterpret_cast<uint16_t*>(out) + (int64_t)b * o_stride_b + head * DH;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        if (ld_ok[i] && t + ld_tok[i] < t1)
          *reinterpret_cast<u32x4_t*>(ob + (int64_t)(t + ld_tok[i]) * o_stride_n + ld_ch[i] * 8) =
              *reinterpret_cast<const u32x4_t*>(to + ld_tok[i] * QROW + ld_ch[i] * 8);
      }
    }
  }
}

// MI355X: 256 compute units (a constant, so plans do not depend on the host the call is made on)
constexpr int compute_units112() { return 256; }

struct Plan112 {
  int nsplit, split_tokens;
};
Plan112 plan112(int B, int h, int n_chunks, int max_chunk_tokens) {
  // one workgroup per CU (256 accumulator registers per wave: one wave per SIMD), splits of at least 512 tokens
  const int items = B * h * n_chunks;
  int ns = 256 / items;  // rounding down: 260 workgroups on 256 CUs would take two rounds
  const int cap = (max_chunk_tokens + 511) / 512;
  if (ns > cap) ns = cap;
  if (ns < 1) ns = 1;
  if (ns > 64) ns = 64;
  Plan112 pl;
  pl.split_tokens = ((max_chunk_tokens + ns - 1) / ns + 127) / 128 * 128;
  pl.nsplit = (max_chunk_tokens + pl.split_tokens - 1) / pl.split_tokens;
  if (pl.nsplit < 1) pl.nsplit = 1;
  return pl;
}

}  // namespace

size_t workspace_bytes112(int B, int h, int n_chunks, int max_chunk_tokens) {
  const Plan112 pl = plan112(B, h, n_chunks, max_chunk_tokens);
  return (size_t)B * h * n_chunks * pl.nsplit * SE * sizeof(float);  // the partials are always written
}

int launch_state112(const void* k, const void* v, float* state, void* workspace, size_t workspace_bytes, int B, int N,
                    int h, int64_t stride_b, int64_t stride_n, const int32_t* chunk_starts, int n_chunks,
                    int max_chunk_tokens, int causal, int io_dtype, const QkPre& pre, hipStream_t s) {
  if (io_dtype != SANA_DT_BF16 && io_dtype != SANA_DT_F16) return SANA_ERR_DTYPE;
  const bool use_pre = pre.rinv || pre.rope;
  if (use_pre && io_dtype != SANA_DT_BF16) return SANA_ERR_DTYPE;
  // the kernel addresses one batch entry's tokens with 32-bit byte offsets (buffer loads)
  if ((int64_t)N * stride_n * 2 >= (int64_t)1 << 31 || (int64_t)N * DH * 4 >= (int64_t)1 << 31) return SANA_ERR_SHAPE;
  const Plan112 pl = plan112(B, h, n_chunks, max_chunk_tokens);
  const size_t need = workspace_bytes112(B, h, n_chunks, max_chunk_tokens);
  if (!workspace || workspace_bytes < need) return SANA_ERR_WORKSPACE;
  if (!aligned16(workspace)) return SANA_ERR_ALIGN;
  float* part = static_cast<float*>(workspace);
  const int64_t units = (int64_t)B * n_chunks * pl.nsplit, nwg = head_unit_grid(units, h);
  if (nwg > 0x7fffffff) return SANA_ERR_SHAPE;
  dim3 grid((unsigned)nwg);
  const uint16_t* kp = static_cast<const uint16_t*>(k);
  const uint16_t* vp = static_cast<const uint16_t*>(v);
#define SANA_ST112(T, PRE)                                                                                        \
  hipLaunchKernelGGL((state112_kernel<T, PRE>), grid, dim3(256), 0, s, kp, vp, part, chunk_starts, N, h, n_chunks, \
                     pl.nsplit, pl.split_tokens, (int)units, stride_b, stride_n, pre)
  const int mode = (pre.rinv ? 1 : 0) | (pre.rope ? 2 : 0);
  if (io_dtype == SANA_DT_F16) SANA_ST112(F16, 0);
  else if (mode == 3) SANA_ST112(BF16, 3);
  else if (mode == 2) SANA_ST112(BF16, 2);
  else if (mode == 1) SANA_ST112(BF16, 1);
  else SANA_ST112(BF16, 0);
#undef SANA_ST112
  if (hipGetLastError() != hipSuccess) return SANA_ERR_LAUNCH;
  const int64_t threads = (int64_t)B * h * SE;
  hipLaunchKernelGGL(reduce112_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, part, state, B * h,
                     n_chunks, pl.nsplit, (causal && n_chunks > 1) ? 1 : 0);
  return hipGetLastError() == hipSuccess ? SANA_OK : SANA_ERR_LAUNCH;
}

int launch_scan112(float* state, int B, int h, int n_chunks, hipStream_t s) {
  const int64_t threads = (int64_t)B * h * SE;
  hipLaunchKernelGGL(reduce112_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, state, state, B * h,
                     n_chunks, 1, 1);
  return hipGetLastError() == hipSuccess ? SANA_OK : SANA_ERR_LAUNCH;
}

int launch_apply112(const void* q, const float* state, void* out, int B, int N, int h, int64_t q_stride_b,
                    int64_t q_stride_n, int64_t o_stride_b, int64_t o_stride_n, const int32_t* chunk_starts,
                    int n_chunks, int max_chunk_tokens, float eps, int io_dtype, int out_dtype, const QkPre& pre,
                    hipStream_t s) {
  if (io_dtype != SANA_DT_BF16) return SANA_ERR_DTYPE;
  // Tokens per workgroup (a multiple of the 32-token step): long enough to pay for building the state
  // operands once (~256), and such that the grid fills whole rounds of the chip -- 3 workgroups per CU
  // fit (2 with transforms or fp32 output: registers), so 4 rounds of 256 tokens with the last one a third
  // full lose to 3 rounds of 288.
  const int mode = (pre.rinv ? 1 : 0) | (pre.rope ? 2 : 0);
  int wg_tokens = 256;
  {
    const int64_t slots = (int64_t)compute_units112() * ((mode || out_dtype == SANA_DT_F32) ? 2 : 3);
    double best = 1e30;
    for (int t = 192; t <= 512; t += 32) {
      const int64_t wgs = (int64_t)((max_chunk_tokens + t - 1) / t) * n_chunks * B * h;
      const double cost = (double)((wgs + slots - 1) / slots) * (t + 48);  // + the operand build, in token-equivalents
      if (cost < best) {
        best = cost;
        wg_tokens = t;
      }
    }
  }
  const int xranges = (max_chunk_tokens + wg_tokens - 1) / wg_tokens;
  const int64_t units = (int64_t)xranges * n_chunks * B, total = head_unit_grid(units, h);
  if (total > 0x7fffffff) return SANA_ERR_SHAPE;
  dim3 grid((unsigned)total);
  const uint16_t* qp = static_cast<const uint16_t*>(q);
#define SANA_AP112(F32, PRE)                                                                                         \
  hipLaunchKernelGGL((apply112_kernel<F32, PRE>), grid, dim3(256), 0, s, qp, state, out, chunk_starts, N, h, n_chunks, \
                     xranges, wg_tokens, (int)units, q_stride_b, q_stride_n, o_stride_b, o_stride_n, eps, pre)
  if (out_dtype == SANA_DT_F32) {
    if (mode == 3) SANA_AP112(true, 3);
    else if (mode == 2) SANA_AP112(true, 2);
    else if (mode == 1) SANA_AP112(true, 1);
    else SANA_AP112(true, 0);
  } else {
    if (mode == 3) SANA_AP112(false, 3);
    else if (mode == 2) SANA_AP112(false, 2);
    else if (mode == 1) SANA_AP112(false, 1);
    else SANA_AP112(false, 0);
  }
#undef SANA_AP112
  return hipGetLastError() == hipSuccess ? SANA_OK : SANA_ERR_LAUNCH;
}

}  // namespace sana
