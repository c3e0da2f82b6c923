// ReLU linear attention for gfx950: phase 1 (state = [V|1]^T relu(K) per head),
// split reduction + chunk prefix scan, phase 2 (apply to relu(Q), divide).
//
// Data layout: q, k, v and out are token-major [B][N][h*32] views (channel
// stride 1).  The state is fp32 [B][h][n_chunks][33][32]; row 32 holds
// sum_n relu(k_n).
//
// 16-bit io (bf16 / f16)
//   phase 1  one workgroup = (batch, pair of heads, chunk, token split); its four
//            waves take interleaved 32-token tiles.  A tile is loaded with
//            16-byte coalesced loads, written to wave-private LDS and read back
//            transposed (token-contiguous per channel) as MFMA 32x32x16
//            operands: S += V^T K; the ones-row (ksum) is a packed dot2 against (1, 1)
//            on the K operand registers.  Waves are summed in LDS.
//   phase 2  one wave = (pair of heads, token range); the fp32 state is split
//            into three bf16 terms (hi + mid + lo = all 24 mantissa bits) and
//            applied with MFMA 16x16x32; rows 32..47 of the A operand all carry
//            ksum so every lane gets its token's denominator in-lane.
// fp32 io (and f16 phase 2) uses MFMA 32x32x2 f32 directly from global memory.
#include <atomic>
#include <mutex>
#include <type_traits>

#include "common.h"
#include "linattn_common.h"

// tuning knobs of the bf16 apply kernel: tokens per workgroup, 16-token steps in flight per wave
#ifndef SANA_LA_APPLY_TOKENS
#define SANA_LA_APPLY_TOKENS 128
#endif
#ifndef SANA_LA_NT_LOAD
#define SANA_LA_NT_LOAD 0
#endif
#ifndef SANA_LA_NT_STORE
#define SANA_LA_NT_STORE 0
#endif
#ifndef SANA_LA_APPLY_U
#define SANA_LA_APPLY_U 4
#endif

namespace sana {
namespace {

constexpr int D = 32;
constexpr int STATE_ELEMS = (D + 1) * D;  // 1056
constexpr int TILE = 32;                  // tokens per phase-1 tile

// ----------------------------------------------------------------------------
// phase 1, 16-bit io
// grid: x = nsplit, y = n_chunks, z = B * pairs;  block 256
// dst: when nsplit == 1 the final state, else partial[(bh*n_chunks + c)*nsplit + split][1056]
// ----------------------------------------------------------------------------
// PRE: on-load transforms as compile-time bits (1 = q/k RMSNorm, 2 = rotary embedding, 4 = the rotation comes before
// the ReLU and ksum is taken from the rotated values: QkPre::rope_first)
template <typename T, int PRE>
__global__ __launch_bounds__(256) void linattn_state16_kernel(
    const uint16_t* __restrict__ K, const uint16_t* __restrict__ V, float* __restrict__ dst,
    const int32_t* __restrict__ chunk_starts, int N, int h, int n_chunks, int nsplit, int split_tokens,
    int64_t stride_b, int64_t stride_n, const QkPre pre) {
  // staging: per wave K tile [32 tok][64 ch] + V tile, 16-bit -> 8 KB per wave.
  // reduction: per wave 2 heads x 1056 fp32 -> 8448 B per wave.  The two uses
  // never overlap in time, so they share one buffer.
  __shared__ __attribute__((aligned(16))) unsigned char smem[4 * 2 * STATE_ELEMS * 4];
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int pairs = (h + 1) >> 1;
  const int b = blockIdx.z / pairs, p = blockIdx.z % pairs;
  const int c = blockIdx.y, split = blockIdx.x;
  const int C = h * D;
  const ChunkRange cr = chunk_range(chunk_starts, c, N);
  const int t0 = cr.begin + split * split_tokens;
  const int t1 = min(cr.end, t0 + split_tokens);

  uint16_t* stage = reinterpret_cast<uint16_t*>(smem) + wave * (2 * TILE * 64);
  uint16_t* lds_k = stage;
  uint16_t* lds_v = stage + TILE * 64;

  // load mapping: lane -> token (lane/8 + 8*i), 16-byte channel chunk lane%8
  const int ld_tok = lane >> 3;
  const int ld_ch = p * 64 + (lane & 7) * 8;
  const bool ch_ok = ld_ch < C;
  const uint16_t* kbase = K + (int64_t)b * stride_b + ld_ch;
  const uint16_t* vbase = V + (int64_t)b * stride_b + ld_ch;

  f32x16_t accS[2];
  float accK[2] = {0.f, 0.f};  // sum over this lane's tokens of relu(K)[tok][j]
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    accS[0][i] = 0.f;
    accS[1][i] = 0.f;
  }
  const u32x4_t zero4 = {0u, 0u, 0u, 0u};

  constexpr bool has_norm = (PRE & 1) != 0, has_rope = (PRE & 2) != 0, rope_first = (PRE & 4) != 0;
  u32x4_t kreg[4], vreg[4];
  // PRE: per-token 1/rms and this lane's four (cos, sin) pairs travel with the tile; the norm weight
  // of the lane's 8 channels is loop-invariant; ksum is accumulated here, per lane and channel,
  // from the unrotated values (the MFMA operands in LDS are rotated).
  float rin[has_norm ? 4 : 1];
  f32x4_t cs[has_rope ? 4 : 1][2];
  u32x4_t kw = zero4;
  float ks8[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (has_norm && ch_ok) kw = *reinterpret_cast<const u32x4_t*>(pre.weight + ld_ch);
  auto issue_loads = [&](int tile) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int tok = tile + ld_tok + 8 * i;
      if (ch_ok && tok < t1) {
        kreg[i] = load_stream<SANA_LA_NT_LOAD != 0>(reinterpret_cast<const u32x4_t*>(kbase + (int64_t)tok * stride_n));
        vreg[i] = load_stream<SANA_LA_NT_LOAD != 0>(reinterpret_cast<const u32x4_t*>(vbase + (int64_t)tok * stride_n));
        if (has_norm) rin[i] = pre.rinv[(int64_t)b * N + tok];
        if (has_rope) {
          const float* rp = pre.rope + ((int64_t)tok * 16 + (lane & 3) * 4) * 2;
          cs[i][0] = *reinterpret_cast<const f32x4_t*>(rp);
          cs[i][1] = *reinterpret_cast<const f32x4_t*>(rp + 4);
        }
      } else {
        kreg[i] = zero4;
        vreg[i] = zero4;
        if (has_norm) rin[i] = 0.f;
        if (has_rope) {
          cs[i][0] = f32x4_t{0.f, 0.f, 0.f, 0.f};
          cs[i][1] = cs[i][0];
        }
      }
    }
  };

  int tile = t0 + wave * TILE;
  if (tile < t1) issue_loads(tile);
  // operand read mapping: lane -> channel j = lane%32 (of head hh), k-group g = lane/32;
  // element r of k-step s is token 16*s + 2*r + g of the tile (any bijection works as
  // long as both operands use the same one: the MFMA contracts over tokens).
  const int j = lane & 31, g = lane >> 5;
  for (; tile < t1; tile += 4 * TILE) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      u32x4_t kk = kreg[i];
      if (PRE) {
        if (has_norm) kk = rms_scale8(kk, rin[i], kw);
        if (rope_first) kk = rope8(kk, cs[i][0], cs[i][1]);
        kk = relu_pk16(kk);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          ks8[2 * e] += bf16_lo(kk[e]);
          ks8[2 * e + 1] += bf16_hi(kk[e]);
        }
        if (has_rope && !rope_first) kk = rope8(kk, cs[i][0], cs[i][1]);
      } else {
        kk = relu_pk16(kk);
      }
      *reinterpret_cast<u32x4_t*>(lds_k + (ld_tok + 8 * i) * 64 + (lane & 7) * 8) = kk;
      *reinterpret_cast<u32x4_t*>(lds_v + (ld_tok + 8 * i) * 64 + (lane & 7) * 8) = vreg[i];
    }
    if (tile + 4 * TILE < t1) issue_loads(tile + 4 * TILE);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // wave-private LDS: in-order, no barrier needed
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        u32x4_t fk, fv;
#pragma unroll
        for (int r2 = 0; r2 < 4; ++r2) {
          const int ta = 16 * s + 2 * (2 * r2) + g, tb = 16 * s + 2 * (2 * r2 + 1) + g;
          const uint32_t klo = lds_k[ta * 64 + hh * 32 + j], khi = lds_k[tb * 64 + hh * 32 + j];
          const uint32_t vlo = lds_v[ta * 64 + hh * 32 + j], vhi = lds_v[tb * 64 + hh * 32 + j];
          fk[r2] = klo | (khi << 16);
          fv[r2] = vlo | (vhi << 16);
        }
        accS[hh] = mfma_32x32x16<T>(fv, fk, accS[hh]);  // S[i][j] += sum_tok V[tok][i] K[tok][j]
        if (!PRE) {
#pragma unroll
          for (int r2 = 0; r2 < 4; ++r2) accK[hh] = add_pk16<T>(fk[r2], accK[hh]);  // the "1" row of [V|1]
        }
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // reads done before the next tile overwrites
  }

  // cross-wave reduction in LDS.  D layout of 32x32 MFMA: lane -> column j = lane%32,
  // register r -> row 8*(r/4) + 4*(lane/32) + r%4.
  __syncthreads();
  float* red = reinterpret_cast<float*>(smem) + wave * (2 * STATE_ELEMS);
#pragma unroll
  for (int hh = 0; hh < 2; ++hh) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = 8 * (r >> 2) + 4 * g + (r & 3);
      red[hh * STATE_ELEMS + row * D + j] = accS[hh][r];
    }
    if (!PRE) {
      const float ks = accK[hh] + __shfl_xor(accK[hh], 32, 64);  // the two token halves of channel j
      if (g == 0) red[hh * STATE_ELEMS + D * D + j] = ks;
    }
  }
  if (PRE) {  // lanes with the same channel chunk (lane % 8) hold different tokens: fold them
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float x = ks8[e];
      x += __shfl_xor(x, 8, 64);
      x += __shfl_xor(x, 16, 64);
      x += __shfl_xor(x, 32, 64);
      if (lane < 8) red[(lane >> 2) * STATE_ELEMS + D * D + (lane & 3) * 8 + e] = x;
    }
  }
  __syncthreads();
  const float* all = reinterpret_cast<const float*>(smem);
  for (int e = tid; e < 2 * STATE_ELEMS; e += 256) {
    const int hh = e / STATE_ELEMS, idx = e - hh * STATE_ELEMS;
    const int head = 2 * p + hh;
    if (head >= h) continue;
    const float sum = ((all[e] + all[2 * STATE_ELEMS + e]) + all[4 * STATE_ELEMS + e]) + all[6 * STATE_ELEMS + e];
    const int64_t slot = ((int64_t)(b * h + head) * n_chunks + c) * nsplit + split;
    dst[slot * STATE_ELEMS + idx] = sum;
  }
}

// ----------------------------------------------------------------------------
// phase 1, fp32 io: MFMA 32x32x2 f32 straight from global memory.
// grid: x = nsplit, y = n_chunks, z = B * ceil(h/4); block 256, wave = one head.
// ----------------------------------------------------------------------------
__global__ __launch_bounds__(256) void linattn_state32_kernel(
    const float* __restrict__ K, const float* __restrict__ V, float* __restrict__ dst,
    const int32_t* __restrict__ chunk_starts, int N, int h, int n_chunks, int nsplit, int split_tokens,
    int64_t stride_b, int64_t stride_n) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int groups = (h + 3) >> 2;
  const int b = blockIdx.z / groups, head = (blockIdx.z % groups) * 4 + wave;
  if (head >= h) return;  // no barriers below
  const int c = blockIdx.y, split = blockIdx.x;
  const ChunkRange cr = chunk_range(chunk_starts, c, N);
  const int t0 = cr.begin + split * split_tokens;
  const int t1 = min(cr.end, t0 + split_tokens);
  const int j = lane & 31, g = lane >> 5;
  const float* kp = K + (int64_t)b * stride_b + head * D + j;
  const float* vp = V + (int64_t)b * stride_b + head * D + j;
  f32x16_t accS, accK;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    accS[i] = 0.f;
    accK[i] = 0.f;
  }
  constexpr int U = 8;  // 16 tokens in flight per wave
  for (int t = t0; t < t1; t += 2 * U) {
    float kk[U], vv[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int tok = t + 2 * u + g;
      const bool ok = tok < t1;
      kk[u] = ok ? fmaxf(kp[(int64_t)tok * stride_n], 0.f) : 0.f;
      vv[u] = ok ? vp[(int64_t)tok * stride_n] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      accS = __builtin_amdgcn_mfma_f32_32x32x2f32(vv[u], kk[u], accS, 0, 0, 0);
      accK = __builtin_amdgcn_mfma_f32_32x32x2f32(1.0f, kk[u], accK, 0, 0, 0);
    }
  }
  const int64_t slot = ((int64_t)(b * h + head) * n_chunks + c) * nsplit + split;
  float* o = dst + slot * STATE_ELEMS;
#pragma unroll
  for (int r = 0; r < 16; ++r) o[(8 * (r >> 2) + 4 * g + (r & 3)) * D + j] = accS[r];
  if (g == 0) o[D * D + j] = accK[0];
}

// ----------------------------------------------------------------------------
// split reduction (+ inclusive prefix over chunks when causal).
// One thread per (b*h, element); fixed summation order.
// ----------------------------------------------------------------------------
__global__ __launch_bounds__(256) void linattn_reduce_scan_kernel(const float* __restrict__ partial,
                                                                  float* __restrict__ state, int BH,
                                                                  int n_chunks, int nsplit, int causal) {
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (gid >= (int64_t)BH * STATE_ELEMS) return;
  const int64_t bh = gid / STATE_ELEMS;
  const int e = (int)(gid - bh * STATE_ELEMS);
  float run = 0.f;
  for (int c = 0; c < n_chunks; ++c) {
    const float* p0 = partial + ((bh * n_chunks + c) * nsplit) * STATE_ELEMS + e;
    // batches of sixteen independent loads (all in flight together), added in split order
    float s = 0.f;
    for (int sp0 = 0; sp0 < nsplit; sp0 += 16) {
      float v[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) v[u] = (sp0 + u < nsplit) ? p0[(int64_t)(sp0 + u) * STATE_ELEMS] : 0.f;
#pragma unroll
      for (int u = 0; u < 16; ++u) s += v[u];
    }
    if (causal) {
      run += s;
      s = run;
    }
    state[(bh * n_chunks + c) * STATE_ELEMS + e] = s;
  }
}

// ----------------------------------------------------------------------------
// phase 2, bf16 io.  grid: x = token ranges per chunk, y = n_chunks,
// z = B * ceil(pairs/4); block 256; wave = pair of heads.
// ----------------------------------------------------------------------------
struct SplitState {     // A operands of one head: 3 row blocks x 3 bf16 terms
  u32x4_t a[3][3];
};

__device__ __forceinline__ void split3(const float x[8], u32x4_t out[3]) {
  float r1[8], r2[8];
  uint32_t hi[8], mid[8], lo[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    hi[e] = f32_to_bf16_bits(x[e]);
    r1[e] = x[e] - bf16_bits_to_f32(hi[e]);
    mid[e] = f32_to_bf16_bits(r1[e]);
    r2[e] = r1[e] - bf16_bits_to_f32(mid[e]);
    lo[e] = f32_to_bf16_bits(r2[e]);
  }
#pragma unroll
  for (int e2 = 0; e2 < 4; ++e2) {
    out[0][e2] = hi[2 * e2] | (hi[2 * e2 + 1] << 16);
    out[1][e2] = mid[2 * e2] | (mid[2 * e2 + 1] << 16);
    out[2][e2] = lo[2 * e2] | (lo[2 * e2 + 1] << 16);
  }
}

template <bool OUT_F32, int PRE>
__global__ __launch_bounds__(256) void linattn_apply_bf16_kernel(
    const uint16_t* __restrict__ Q, const float* __restrict__ state, void* __restrict__ out,
    const int32_t* __restrict__ chunk_starts, int N, int h, int n_chunks, int wg_tokens,
    int64_t q_stride_b, int64_t q_stride_n, int64_t o_stride_b, int64_t o_stride_n, float eps,
    const QkPre pre, int xranges, int ngroups) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int pairs = (h + 1) >> 1;
  const int pgroups = (pairs + 3) >> 2;
  // 3-D grid (token range, chunk, batch x head group), or -- with many (chunk, batch, head group)
  // combinations -- a 1-D grid dealt so that all token ranges of one combination run on the same XCD
  // (workgroup ids go round-robin to the 8 XCDs): their common state is then fetched into one L2 only.
  int bx = blockIdx.x, by = blockIdx.y, bz = blockIdx.z;
  if (ngroups > 0) {
    const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
    const int grp = xcd + 8 * (idx / xranges);
    if (grp >= ngroups) return;  // no barriers below
    bx = idx % xranges, by = grp % n_chunks, bz = grp / n_chunks;
  }
  const int b = bz / pgroups, p = (bz % pgroups) * 4 + wave;
  if (p >= pairs) return;  // no barriers below
  const int c = by;
  const ChunkRange cr = chunk_range(chunk_starts, c, N);
  const int t0 = cr.begin + bx * wg_tokens;
  const int t1 = min(cr.end, t0 + wg_tokens);
  if (t0 >= t1) return;
  const int n = lane & 15, g = lane >> 4;
  const int nheads = (2 * p + 1 < h) ? 2 : 1;

  // A operands.  MFMA 16x16x32: A lane -> row lane%16, k = 8*(lane/16)+e.  Output
  // lane (token n, g') register s of row block rb is row 4*g'+s; we place channel
  // 8*(r/4) + 4*rb + r%4 in row r so that a lane ends up with 8 contiguous channels.
  SplitState st[2];
#pragma unroll
  for (int hh = 0; hh < 2; ++hh) {
    const int head = min(2 * p + hh, h - 1);
    const float* sp = state + ((int64_t)(b * h + head) * n_chunks + c) * STATE_ELEMS;
#pragma unroll
    for (int rb = 0; rb < 3; ++rb) {
      const int row = (rb < 2) ? (8 * (n >> 2) + 4 * rb + (n & 3)) : D;
      const f32x4_t x0 = *reinterpret_cast<const f32x4_t*>(sp + row * D + 8 * g);
      const f32x4_t x1 = *reinterpret_cast<const f32x4_t*>(sp + row * D + 8 * g + 4);
      const float x[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
      split3(x, st[hh].a[rb]);
    }
  }

  const u32x4_t zero4 = {0u, 0u, 0u, 0u};
  constexpr bool has_norm = (PRE & 1) != 0, has_rope = (PRE & 2) != 0, rope_first = (PRE & 4) != 0;
  u32x4_t qw[2] = {zero4, zero4};
  if (has_norm) {
#pragma unroll
    for (int hh = 0; hh < 2; ++hh)
      if (hh < nheads) qw[hh] = *reinterpret_cast<const u32x4_t*>(pre.weight + p * 64 + hh * D + 8 * g);
  }
  // Global accesses are whole 128-byte lines: lane l fetches 16-byte chunk l%8 of token l/8 (both heads
  // of the pair), two instructions per 16-token step, and the step goes through wave-private LDS to
  // reach the MFMA layout (lane = token n, channel group g); results return the same way, so a store
  // instruction writes eight full lines.  (Fetching straight in MFMA layout touches every line twice
  // with 64-byte pieces and is bound by the L1 tag rate: 4.2 TB/s read side against 5.8 here.)
  // LDS slot of (token n of the step, chunk c): 16 * (8n + (c ^ (n/2) % 8)): conflict-free both ways.
  constexpr int U = PRE ? SANA_LA_APPLY_U / 2 : SANA_LA_APPLY_U;  // 16-token steps in flight
  __shared__ __attribute__((aligned(16))) unsigned char stage_all[4 * (SANA_LA_APPLY_U + 1) * 2048];
  unsigned char* stage = stage_all + wave * ((SANA_LA_APPLY_U + 1) * 2048);
  const int ld_tok = lane >> 3, ld_chunk = lane & 7;
  const uint16_t* qrow = Q + (int64_t)b * q_stride_b + p * 64 + 8 * ld_chunk;
  const bool ld_ok = nheads == 2 || ld_chunk < 4;   // the second head of the last pair may not exist
  int slot_w[2], slot_r[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int tl = 8 * j + ld_tok;
    slot_w[j] = 16 * (8 * tl + (ld_chunk ^ ((tl >> 1) & 7)));
  }
#pragma unroll
  for (int hh = 0; hh < 2; ++hh) slot_r[hh] = 16 * (8 * n + ((4 * hh + g) ^ ((n >> 1) & 7)));
  for (int t = t0; t < t1; t += 16 * U) {
    u32x4_t raw[U][2];
    float rin[has_norm ? U : 1];
    f32x4_t cs[has_rope ? U : 1][2];
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int tok = t + 16 * u + 8 * j + ld_tok;
        raw[u][j] = (tok < t1 && ld_ok) ? load_stream<SANA_LA_NT_LOAD != 0>(reinterpret_cast<const u32x4_t*>(qrow + (int64_t)tok * q_stride_n)) : zero4;
      }
      const int tok = t + 16 * u + n;
      if (has_norm) rin[u] = tok < t1 ? pre.rinv[(int64_t)b * N + tok] : 0.f;
      if (has_rope) {
        const float* rp = pre.rope + ((int64_t)min(tok, t1 - 1) * 16 + g * 4) * 2;
        cs[u][0] = *reinterpret_cast<const f32x4_t*>(rp);
        cs[u][1] = *reinterpret_cast<const f32x4_t*>(rp + 4);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int j = 0; j < 2; ++j) *reinterpret_cast<u32x4_t*>(stage + u * 2048 + slot_w[j]) = raw[u][j];
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // wave-private LDS: in-order, no barrier needed
    unsigned char* ostage = stage + SANA_LA_APPLY_U * 2048;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int tok = t + 16 * u + n;
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        u32x4_t qd = *reinterpret_cast<const u32x4_t*>(stage + u * 2048 + slot_r[hh]);
        if (has_norm) qd = rms_scale8(qd, rin[u], qw[hh]);
        if (rope_first) qd = rope8(qd, cs[u][0], cs[u][1]);              // rotated first: both operands
        qd = relu_pk16(qd);                                              // denominator operand
        const u32x4_t qb = (has_rope && !rope_first) ? rope8(qd, cs[u][0], cs[u][1]) : qd;  // numerator operand
        f32x4_t acc[3];
#pragma unroll
        for (int rb = 0; rb < 3; ++rb) {
          const u32x4_t bop = rb < 2 ? qb : qd;
          f32x4_t a = {0.f, 0.f, 0.f, 0.f};
          a = mfma_16x16x32_bf16(st[hh].a[rb][2], bop, a);  // smallest term first
          a = mfma_16x16x32_bf16(st[hh].a[rb][1], bop, a);
          a = mfma_16x16x32_bf16(st[hh].a[rb][0], bop, a);
          acc[rb] = a;
        }
        const float den = acc[2][0] + eps;
        if (OUT_F32) {
          if (tok < t1 && hh < nheads) {
            const int64_t o_off = (int64_t)b * o_stride_b + (int64_t)tok * o_stride_n + p * 64 + hh * D + 8 * g;
            f32x4_t o0, o1;
#pragma unroll
            for (int s = 0; s < 4; ++s) {
              o0[s] = acc[0][s] / den;
              o1[s] = acc[1][s] / den;
            }
            float* op = reinterpret_cast<float*>(out) + o_off;
            store_stream<SANA_LA_NT_STORE != 0>(o0, reinterpret_cast<f32x4_t*>(op));
            store_stream<SANA_LA_NT_STORE != 0>(o1, reinterpret_cast<f32x4_t*>(op + 4));
          }
        } else {
          const float inv = __builtin_amdgcn_rcpf(den);
          u32x4_t o;
          o.x = pack_bf16(acc[0][0] * inv, acc[0][1] * inv);
          o.y = pack_bf16(acc[0][2] * inv, acc[0][3] * inv);
          o.z = pack_bf16(acc[1][0] * inv, acc[1][1] * inv);
          o.w = pack_bf16(acc[1][2] * inv, acc[1][3] * inv);
          *reinterpret_cast<u32x4_t*>(ostage + slot_r[hh]) = o;
        }
      }
      if (!OUT_F32) {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int tok_s = t + 16 * u + 8 * j + ld_tok;
          const u32x4_t o = *reinterpret_cast<const u32x4_t*>(ostage + slot_w[j]);
          if (tok_s < t1 && ld_ok)
            store_stream<SANA_LA_NT_STORE != 0>(o, reinterpret_cast<u32x4_t*>(reinterpret_cast<uint16_t*>(out) + (int64_t)b * o_stride_b +
                                                       (int64_t)tok_s * o_stride_n + p * 64 + 8 * ld_chunk));
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the reads are done before the next step overwrites
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }
}

// ----------------------------------------------------------------------------
// phase 2, fp32 / f16 io: MFMA 32x32x2 f32.  grid as above but wave = one head,
// z = B * ceil(h/4).  A lane -> state row lane%32, contraction index 16*(lane/32)+s;
// B lane -> token lane%32, same contraction index.  The denominator MFMA uses the
// ksum row in every A row, so the divide is lane-local.
// ----------------------------------------------------------------------------
template <typename TIn, typename TOut>
__device__ __forceinline__ TOut cvt_out(float x);
template <>
__device__ __forceinline__ float cvt_out<float, float>(float x) { return x; }
template <>
__device__ __forceinline__ float cvt_out<_Float16, float>(float x) { return x; }
template <>
__device__ __forceinline__ _Float16 cvt_out<_Float16, _Float16>(float x) { return (_Float16)x; }

template <typename TIn, typename TOut>
__global__ __launch_bounds__(256) void linattn_apply32_kernel(
    const TIn* __restrict__ Q, const float* __restrict__ state, TOut* __restrict__ out,
    const int32_t* __restrict__ chunk_starts, int N, int h, int n_chunks, int wg_tokens,
    int64_t q_stride_b, int64_t q_stride_n, int64_t o_stride_b, int64_t o_stride_n, float eps) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int groups = (h + 3) >> 2;
  const int b = blockIdx.z / groups, head = (blockIdx.z % groups) * 4 + wave;
  if (head >= h) return;
  const int c = blockIdx.y;
  const ChunkRange cr = chunk_range(chunk_starts, c, N);
  const int t0 = cr.begin + blockIdx.x * wg_tokens;
  const int t1 = min(cr.end, t0 + wg_tokens);
  if (t0 >= t1) return;
  const int n = lane & 31, g = lane >> 5;
  const float* sp = state + ((int64_t)(b * h + head) * n_chunks + c) * STATE_ELEMS;
  float a_num[16], a_den[16];
#pragma unroll
  for (int s = 0; s < 16; ++s) {
    a_num[s] = sp[n * D + 16 * g + s];
    a_den[s] = sp[D * D + 16 * g + s];
  }
  for (int t = t0; t < t1; t += 32) {
    const int tok = t + n;
    const bool ok = tok < t1;
    float qv[16];
    const TIn* qp = Q + (int64_t)b * q_stride_b + (int64_t)tok * q_stride_n + head * D + 16 * g;
#pragma unroll
    for (int s = 0; s < 16; ++s) qv[s] = ok ? fmaxf((float)qp[s], 0.f) : 0.f;
    f32x16_t num, den;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      num[i] = 0.f;
      den[i] = 0.f;
    }
#pragma unroll
    for (int s = 0; s < 16; ++s) {
      num = __builtin_amdgcn_mfma_f32_32x32x2f32(a_num[s], qv[s], num, 0, 0, 0);
      den = __builtin_amdgcn_mfma_f32_32x32x2f32(a_den[s], qv[s], den, 0, 0, 0);
    }
    if (ok) {
      // D layout: lane -> token (column) lane%32; register r -> channel 8*(r/4)+4*g+r%4
      const float dd = den[0] + eps;
      TOut* op = out + (int64_t)b * o_stride_b + (int64_t)tok * o_stride_n + head * D;
#pragma unroll
      for (int r = 0; r < 16; ++r) op[8 * (r >> 2) + 4 * g + (r & 3)] = cvt_out<TIn, TOut>(num[r] / dd);
    }
  }
}

// ----------------------------------------------------------------------------
// Per-token 1/rms of q and of k over all C channels (the statistic of the reference's
// RMSNorm before the head split): rinv = rsqrt(mean(x^2) + eps).  One wave per (token, tensor).
// grid: x = ceil(B*N/4), y = 2 (q, k); block 256.
// ----------------------------------------------------------------------------
__global__ __launch_bounds__(256) void qk_rms_kernel(const uint16_t* __restrict__ Q, const uint16_t* __restrict__ K,
                                                     float* __restrict__ rq, float* __restrict__ rk, int64_t BN,
                                                     int N, int C, int64_t stride_b, int64_t stride_n, float eps) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + wave;
  if (row >= BN) return;
  const uint16_t* x = (blockIdx.y == 0 ? Q : K) + (row / N) * stride_b + (row % N) * stride_n;
  float acc = 0.f;
  for (int c0 = lane * 8; c0 < C; c0 += 512) {
    const u32x4_t v = *reinterpret_cast<const u32x4_t*>(x + c0);  // cacheable: the attention kernels read q and k next
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float a = bf16_lo(v[e]), b2 = bf16_hi(v[e]);
      acc = fmaf(a, a, acc);
      acc = fmaf(b2, b2, acc);
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
  if (lane == 0) (blockIdx.y == 0 ? rq : rk)[row] = rsqrtf(acc / (float)C + eps);
}

// ---------------------------------------------------------------------------- host side

int pick_nsplit(int items, int max_chunk_tokens, int min_tokens) {
  // aim for >= 1024 workgroups (four per CU), but keep >= min_tokens tokens per split
  int ns = (1024 + items - 1) / items;
  const int cap = (max_chunk_tokens + min_tokens - 1) / min_tokens;
  if (ns > cap) ns = cap;
  if (ns < 1) ns = 1;
  if (ns > 64) ns = 64;
  return ns;
}
int split_len(int max_chunk_tokens, int nsplit, int granule) {
  int len = (max_chunk_tokens + nsplit - 1) / nsplit;
  return (len + granule - 1) / granule * granule;
}

struct StatePlan {
  int items;   // workgroups before splitting
  int nsplit;
  int split_tokens;
};
StatePlan plan_state(int B, int h, int n_chunks, int max_chunk_tokens, int io_dtype) {
  StatePlan pl;
  const int per_b = (io_dtype == SANA_DT_F32) ? (h + 3) / 4 : (h + 1) / 2;
  pl.items = B * per_b * n_chunks;
  // 16-bit: four waves x 32-token tiles per round; fp32: 16 tokens per wave iteration
  const bool f32 = io_dtype == SANA_DT_F32;
  pl.nsplit = pick_nsplit(pl.items, max_chunk_tokens, f32 ? 64 : 256);
  pl.split_tokens = split_len(max_chunk_tokens, pl.nsplit, f32 ? 16 : 128);
  // drop splits that would be empty after rounding the length up
  pl.nsplit = (max_chunk_tokens + pl.split_tokens - 1) / pl.split_tokens;
  if (pl.nsplit < 1) pl.nsplit = 1;
  return pl;
}

}  // namespace
}  // namespace sana

using namespace sana;

extern "C" __attribute__((visibility("default"))) size_t sana_hip_linattn_workspace_bytes(int B, int h, int d,
                                                                                          int n_chunks,
                                                                                          int max_chunk_tokens,
                                                                                          int io_dtype) {
  if (B <= 0 || h <= 0 || (d != D && d != 112) || n_chunks <= 0 || max_chunk_tokens <= 0) return 0;
  if (d == 112) return io_dtype == SANA_DT_F32 ? 0 : workspace_bytes112(B, h, n_chunks, max_chunk_tokens);
  const StatePlan pl = plan_state(B, h, n_chunks, max_chunk_tokens, io_dtype);
  return pl.nsplit > 1 ? (size_t)B * h * n_chunks * pl.nsplit * STATE_ELEMS * sizeof(float) : 0;
}

static int check_pre(const QkPre& pre, int io_dtype) {
  if (!pre.rinv && !pre.rope) return SANA_OK;
  if (io_dtype != SANA_DT_BF16) return SANA_ERR_DTYPE;
  if (pre.rinv && !pre.weight) return SANA_ERR_ARG;
  if (pre.rope_first && !pre.rope) return SANA_ERR_ARG;
  if ((pre.weight && !aligned16(pre.weight)) || (pre.rope && !aligned16(pre.rope))) return SANA_ERR_ALIGN;
  return SANA_OK;
}

static int state_impl(const void* k, const void* v, float* state, void* workspace, size_t workspace_bytes, int B,
                      int N, int h, int d, int64_t stride_b, int64_t stride_n, const int32_t* chunk_starts,
                      int n_chunks, int max_chunk_tokens, int causal, int io_dtype, const QkPre pre, void* stream) {
  if (!k || !v || !state || B <= 0 || N <= 0 || h <= 0 || n_chunks <= 0) return SANA_ERR_ARG;
  {
    const int rc = check_pre(pre, io_dtype);
    if (rc != SANA_OK) return rc;
  }
  if (d != D && d != 112) return SANA_ERR_SHAPE;
  if (n_chunks > 1 && !chunk_starts) return SANA_ERR_ARG;
  if (n_chunks == 1 && !chunk_starts) max_chunk_tokens = N;
  if (max_chunk_tokens <= 0 || max_chunk_tokens > N) return SANA_ERR_ARG;
  if (io_dtype != SANA_DT_F32 && io_dtype != SANA_DT_BF16 && io_dtype != SANA_DT_F16) return SANA_ERR_DTYPE;
  if (stride_n < (int64_t)h * d || stride_b < 0) return SANA_ERR_ARG;
  if ((int64_t)B * h > (1 << 22) || n_chunks > 65535) return SANA_ERR_SHAPE;
  const int esz = io_dtype == SANA_DT_F32 ? 4 : 2;
  if (!aligned16(k) || !aligned16(v) || !aligned16(state) || (stride_n * esz) % 16 || (stride_b * esz) % 16)
    return SANA_ERR_ALIGN;
  if (d == 112 && pre.rope_first) return SANA_ERR_SHAPE;  // the rotate-first order exists for head_dim 32 only
  if (d == 112)
    return launch_state112(k, v, state, workspace, workspace_bytes, B, N, h, stride_b, stride_n, chunk_starts, n_chunks,
                           max_chunk_tokens, causal, io_dtype, pre, static_cast<hipStream_t>(stream));
  const StatePlan pl = plan_state(B, h, n_chunks, max_chunk_tokens, io_dtype);
  float* dst = state;
  if (pl.nsplit > 1) {
    const size_t need = (size_t)B * h * n_chunks * pl.nsplit * STATE_ELEMS * sizeof(float);
    if (!workspace || workspace_bytes < need) return SANA_ERR_WORKSPACE;
    if (!aligned16(workspace)) return SANA_ERR_ALIGN;
    dst = static_cast<float*>(workspace);
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (io_dtype == SANA_DT_F32) {
    dim3 grid(pl.nsplit, n_chunks, B * ((h + 3) / 4));
    hipLaunchKernelGGL(linattn_state32_kernel, grid, dim3(256), 0, s, static_cast<const float*>(k),
                       static_cast<const float*>(v), dst, chunk_starts, N, h, n_chunks, pl.nsplit,
                       pl.split_tokens, stride_b, stride_n);
  } else {
    dim3 grid(pl.nsplit, n_chunks, B * ((h + 1) / 2));
    const int mode = (pre.rinv ? 1 : 0) | (pre.rope ? 2 : 0) | (pre.rope_first ? 4 : 0);
#define SANA_STATE16(T, PRE)                                                                                  \
  hipLaunchKernelGGL((linattn_state16_kernel<T, PRE>), grid, dim3(256), 0, s, static_cast<const uint16_t*>(k), \
                     static_cast<const uint16_t*>(v), dst, chunk_starts, N, h, n_chunks, pl.nsplit,           \
                     pl.split_tokens, stride_b, stride_n, pre)
    if (io_dtype == SANA_DT_F16) SANA_STATE16(F16, 0);
    else if (mode == 7) SANA_STATE16(BF16, 7);
    else if (mode == 6) SANA_STATE16(BF16, 6);
    else if (mode == 3) SANA_STATE16(BF16, 3);
    else if (mode == 2) SANA_STATE16(BF16, 2);
    else if (mode == 1) SANA_STATE16(BF16, 1);
    else SANA_STATE16(BF16, 0);
#undef SANA_STATE16
  }
  if (hipGetLastError() != hipSuccess) return SANA_ERR_LAUNCH;
  const bool scan = causal && n_chunks > 1;
  if (pl.nsplit > 1 || scan) {
    const int64_t threads = (int64_t)B * h * STATE_ELEMS;
    hipLaunchKernelGGL(linattn_reduce_scan_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, dst,
                       state, B * h, n_chunks, pl.nsplit, scan ? 1 : 0);
    if (hipGetLastError() != hipSuccess) return SANA_ERR_LAUNCH;
  }
  return SANA_OK;
}

extern "C" __attribute__((visibility("default"))) int sana_hip_linattn_state(
    const void* k, const void* v, float* state, void* workspace, size_t workspace_bytes, int B, int N, int h, int d,
    int64_t stride_b, int64_t stride_n, const int32_t* chunk_starts, int n_chunks, int max_chunk_tokens, int causal,
    int io_dtype, void* stream) {
  const QkPre none = {nullptr, nullptr, nullptr, 0};
  return state_impl(k, v, state, workspace, workspace_bytes, B, N, h, d, stride_b, stride_n, chunk_starts, n_chunks,
                    max_chunk_tokens, causal, io_dtype, none, stream);
}

extern "C" __attribute__((visibility("default"))) int sana_hip_linattn_state_pre(
    const void* k, const void* v, float* state, void* workspace, size_t workspace_bytes, int B, int N, int h, int d,
    int64_t stride_b, int64_t stride_n, const int32_t* chunk_starts, int n_chunks, int max_chunk_tokens, int causal,
    int io_dtype, const float* k_rinv, const void* k_weight, const float* rope, void* stream) {
  const QkPre pre = {k_rinv, static_cast<const uint16_t*>(k_weight), rope, 0};
  return state_impl(k, v, state, workspace, workspace_bytes, B, N, h, d, stride_b, stride_n, chunk_starts, n_chunks,
                    max_chunk_tokens, causal, io_dtype, pre, stream);
}

extern "C" __attribute__((visibility("default"))) int sana_hip_litela_state(
    const void* k, const void* v, float* state, void* workspace, size_t workspace_bytes, int B, int N, int h, int d,
    int64_t stride_b, int64_t stride_n, int io_dtype, const float* k_rinv, const void* k_weight, const float* rope,
    void* stream) {
  const QkPre pre = {k_rinv, static_cast<const uint16_t*>(k_weight), rope, rope ? 1 : 0};
  return state_impl(k, v, state, workspace, workspace_bytes, B, N, h, d, stride_b, stride_n, nullptr, 1, N, 0, io_dtype,
                    pre, stream);
}

// ---------------------------------------------------------------------------- phase 1 without a workspace argument
// For callers that cannot allocate (code under HIP graph capture, serving loops, harnesses that forbid it): the
// per-split partial states go to a fixed array in device memory instead of a caller-provided workspace.  Each GPU
// the library runs on holds its own copy of the array, at its own address, until the process ends.  `scratch` is a
// host-side stand-in for that symbol, not a device address: host code uses the address hipGetSymbolAddress returns
// for the current device and never the array's name.
static __device__ __align__(256) unsigned char scratch[SANA_HIP_NOALLOC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_addr[kMaxDevices];  // device address of `scratch` per GPU, looked up once per device
std::mutex g_scratch_mutex;

// The current device's copy of the array, or null when the runtime refuses the lookup.
void* scratch_of_current_device() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  void* p = g_scratch_addr[dev].load(std::memory_order_acquire);
  if (p) return p;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  p = g_scratch_addr[dev].load(std::memory_order_relaxed);
  if (!p) {
    void* addr = nullptr;
    if (hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch)) != hipSuccess || !addr) return nullptr;
    g_scratch_addr[dev].store(addr, std::memory_order_release);
    p = addr;
  }
  return p;
}
}  // namespace

extern "C" __attribute__((visibility("default"))) int sana_hip_linattn_state_noalloc(
    const void* k, const void* v, float* state, int B, int N, int h, int d, int64_t stride_b, int64_t stride_n,
    const int32_t* chunk_starts, int n_chunks, int max_chunk_tokens, int causal, int io_dtype, const float* k_rinv,
    const void* k_weight, const float* rope, void* stream) {
  if (B <= 0 || N <= 0 || h <= 0 || n_chunks <= 0) return SANA_ERR_ARG;
  const int longest = (n_chunks == 1 && !chunk_starts) ? N : max_chunk_tokens;
  const size_t need = sana_hip_linattn_workspace_bytes(B, h, d, n_chunks, longest, io_dtype);
  if (need > (size_t)SANA_HIP_NOALLOC_SCRATCH_BYTES) return SANA_ERR_SCRATCH_LIMIT;
  void* ws = scratch_of_current_device();
  if (!ws) return SANA_ERR_RUNTIME;
  // every partial state the reduction reads is written by the launch before it (empty splits write zeros), so the
  // array's old contents never reach a result and nothing has to be cleared
  const QkPre pre = {k_rinv, static_cast<const uint16_t*>(k_weight), rope, 0};
  return state_impl(k, v, state, ws, (size_t)SANA_HIP_NOALLOC_SCRATCH_BYTES, B, N, h, d, stride_b, stride_n,
                    chunk_starts, n_chunks, max_chunk_tokens, causal, io_dtype, pre, stream);
}

extern "C" __attribute__((visibility("default"))) int sana_hip_qk_rms(const void* q, const void* k, float* q_rinv,
                                                                      float* k_rinv, int B, int N, int C,
                                                                      int64_t stride_b, int64_t stride_n, float eps,
                                                                      int io_dtype, void* stream) {
  if (!q || !k || !q_rinv || !k_rinv || B <= 0 || N <= 0 || C <= 0) return SANA_ERR_ARG;
  if (io_dtype != SANA_DT_BF16) return SANA_ERR_DTYPE;
  if (C % 8) return SANA_ERR_SHAPE;
  if (stride_n < C || stride_b < 0) return SANA_ERR_ARG;
  if (!aligned16(q) || !aligned16(k) || (stride_n * 2) % 16 || (stride_b * 2) % 16) return SANA_ERR_ALIGN;
  const int64_t BN = (int64_t)B * N;
  if ((BN + 3) / 4 > 0x7fffffff) return SANA_ERR_SHAPE;
  hipLaunchKernelGGL(qk_rms_kernel, dim3((unsigned)((BN + 3) / 4), 2), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint16_t*>(q), static_cast<const uint16_t*>(k), q_rinv, k_rinv, BN, N, C,
                     stride_b, stride_n, eps);
  return hipGetLastError() == hipSuccess ? SANA_OK : SANA_ERR_LAUNCH;
}

extern "C" __attribute__((visibility("default"))) int sana_hip_linattn_chunk_scan(float* state, int B, int h, int d, int n_chunks, void* stream) {
  if (!state || B <= 0 || h <= 0 || n_chunks <= 0) return SANA_ERR_ARG;
  if (d != D && d != 112) return SANA_ERR_SHAPE;
  if (n_chunks == 1) return SANA_OK;
  if (d == 112) return launch_scan112(state, B, h, n_chunks, static_cast<hipStream_t>(stream));
  const int64_t threads = (int64_t)B * h * STATE_ELEMS;
  hipLaunchKernelGGL(linattn_reduce_scan_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), state, state, B * h, n_chunks, 1, 1);
  return hipGetLastError() == hipSuccess ? SANA_OK : SANA_ERR_LAUNCH;
}

static int apply_impl(const void* q, const float* state, void* out, int B, int N, int h, int d, int64_t q_stride_b,
                      int64_t q_stride_n, int64_t o_stride_b, int64_t o_stride_n, const int32_t* chunk_starts,
                      int n_chunks, int max_chunk_tokens, float eps, int io_dtype, int out_dtype, const QkPre pre,
                      void* stream) {
  if (!q || !state || !out || B <= 0 || N <= 0 || h <= 0 || n_chunks <= 0) return SANA_ERR_ARG;
  {
    const int rc = check_pre(pre, io_dtype);
    if (rc != SANA_OK) return rc;
  }
  if (d != D && d != 112) return SANA_ERR_SHAPE;
  if (n_chunks > 1 && !chunk_starts) return SANA_ERR_ARG;
  if (n_chunks == 1 && !chunk_starts) max_chunk_tokens = N;
  if (max_chunk_tokens <= 0 || max_chunk_tokens > N) return SANA_ERR_ARG;
  if (io_dtype != SANA_DT_F32 && io_dtype != SANA_DT_BF16 && io_dtype != SANA_DT_F16) return SANA_ERR_DTYPE;
  if (out_dtype != io_dtype && out_dtype != SANA_DT_F32) return SANA_ERR_DTYPE;
  if (q_stride_n < (int64_t)h * d || o_stride_n < (int64_t)h * d || q_stride_b < 0 || o_stride_b < 0)
    return SANA_ERR_ARG;
  if ((int64_t)B * h > (1 << 22) || n_chunks > 65535) return SANA_ERR_SHAPE;
  const int qsz = io_dtype == SANA_DT_F32 ? 4 : 2, osz = out_dtype == SANA_DT_F32 ? 4 : 2;
  if (!aligned16(q) || !aligned16(state) || !aligned16(out) || (q_stride_n * qsz) % 16 || (q_stride_b * qsz) % 16 ||
      (o_stride_n * osz) % 16 || (o_stride_b * osz) % 16)
    return SANA_ERR_ALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (d == 112 && pre.rope_first) return SANA_ERR_SHAPE;
  if (d == 112)
    return launch_apply112(q, state, out, B, N, h, q_stride_b, q_stride_n, o_stride_b, o_stride_n, chunk_starts,
                           n_chunks, max_chunk_tokens, eps, io_dtype, out_dtype, pre, s);
  const int wg_tokens = io_dtype == SANA_DT_BF16 ? SANA_LA_APPLY_TOKENS : 64;
  const unsigned gx = (unsigned)((max_chunk_tokens + wg_tokens - 1) / wg_tokens);
  if (io_dtype == SANA_DT_BF16) {
    const int pairs = (h + 1) / 2;
    dim3 grid(gx, n_chunks, B * ((pairs + 3) / 4));
    // many distinct states (chunk-causal video shapes): keep the readers of one state on one XCD
    int ngroups = n_chunks * B * ((pairs + 3) / 4);
    if (ngroups >= 64 && (int64_t)((ngroups + 7) / 8) * 8 * gx < 0x7fffffff)
      grid = dim3((unsigned)((ngroups + 7) / 8 * 8) * gx, 1, 1);
    else
      ngroups = 0;
#define SANA_APPLY(F32, PRE)                                                                                   \
  hipLaunchKernelGGL((linattn_apply_bf16_kernel<F32, PRE>), grid, dim3(256), 0, s, static_cast<const uint16_t*>(q), \
                     state, out, chunk_starts, N, h, n_chunks, wg_tokens, q_stride_b, q_stride_n, o_stride_b,     \
                     o_stride_n, eps, pre, (int)gx, ngroups)
    const int mode = (pre.rinv ? 1 : 0) | (pre.rope ? 2 : 0) | (pre.rope_first ? 4 : 0);
    if (out_dtype == SANA_DT_F32) {
      if (mode == 7) SANA_APPLY(true, 7);
      else if (mode == 6) SANA_APPLY(true, 6);
      else if (mode == 3) SANA_APPLY(true, 3);
      else if (mode == 2) SANA_APPLY(true, 2);
      else if (mode == 1) SANA_APPLY(true, 1);
      else SANA_APPLY(true, 0);
    } else {
      if (mode == 7) SANA_APPLY(false, 7);
      else if (mode == 6) SANA_APPLY(false, 6);
      else if (mode == 3) SANA_APPLY(false, 3);
      else if (mode == 2) SANA_APPLY(false, 2);
      else if (mode == 1) SANA_APPLY(false, 1);
      else SANA_APPLY(false, 0);
    }
#undef SANA_APPLY
  } else {
    dim3 grid(gx, n_chunks, B * ((h + 3) / 4));
    if (io_dtype == SANA_DT_F32)
      hipLaunchKernelGGL((linattn_apply32_kernel<float, float>), grid, dim3(256), 0, s, static_cast<const float*>(q),
                         state, static_cast<float*>(out), chunk_starts, N, h, n_chunks, wg_tokens, q_stride_b,
                         q_stride_n, o_stride_b, o_stride_n, eps);
    else if (out_dtype == SANA_DT_F32)
      hipLaunchKernelGGL((linattn_apply32_kernel<_Float16, float>), grid, dim3(256), 0, s,
                         static_cast<const _Float16*>(q), state, static_cast<float*>(out), chunk_starts, N, h,
                         n_chunks, wg_tokens, q_stride_b, q_stride_n, o_stride_b, o_stride_n, eps);
    else
      hipLaunchKernelGGL((linattn_apply32_kernel<_Float16, _Float16>), grid, dim3(256), 0, s,
                         static_cast<const _Float16*>(q), state, static_cast<_Float16*>(out), chunk_starts, N, h,
                         n_chunks, wg_tokens, q_stride_b, q_stride_n, o_stride_b, o_stride_n, eps);
  }
  return hipGetLastError() == hipSuccess ? SANA_OK : SANA_ERR_LAUNCH;
}

extern "C" __attribute__((visibility("default"))) int sana_hip_linattn_apply(
    const void* q, const float* state, void* out, int B, int N, int h, int d, int64_t q_stride_b, int64_t q_stride_n,
    int64_t o_stride_b, int64_t o_stride_n, const int32_t* chunk_starts, int n_chunks, int max_chunk_tokens,
    float eps, int io_dtype, int out_dtype, void* stream) {
  const QkPre none = {nullptr, nullptr, nullptr, 0};
  return apply_impl(q, state, out, B, N, h, d, q_stride_b, q_stride_n, o_stride_b, o_stride_n, chunk_starts,
                    n_chunks, max_chunk_tokens, eps, io_dtype, out_dtype, none, stream);
}

extern "C" __attribute__((visibility("default"))) int sana_hip_linattn_apply_pre(
    const void* q, const float* state, void* out, int B, int N, int h, int d, int64_t q_stride_b, int64_t q_stride_n,
    int64_t o_stride_b, int64_t o_stride_n, const int32_t* chunk_starts, int n_chunks, int max_chunk_tokens,
    float eps, int io_dtype, int out_dtype, const float* q_rinv, const void* q_weight, const float* rope,
    void* stream) {
  const QkPre pre = {q_rinv, static_cast<const uint16_t*>(q_weight), rope, 0};
  return apply_impl(q, state, out, B, N, h, d, q_stride_b, q_stride_n, o_stride_b, o_stride_n, chunk_starts,
                    n_chunks, max_chunk_tokens, eps, io_dtype, out_dtype, pre, stream);
}

extern "C" __attribute__((visibility("default"))) int sana_hip_litela_apply(
    const void* q, const float* state, void* out, int B, int N, int h, int d, int64_t q_stride_b, int64_t q_stride_n,
    int64_t o_stride_b, int64_t o_stride_n, float eps, int io_dtype, int out_dtype, const float* q_rinv,
    const void* q_weight, const float* rope, void* stream) {
  const QkPre pre = {q_rinv, static_cast<const uint16_t*>(q_weight), rope, rope ? 1 : 0};
  return apply_impl(q, state, out, B, N, h, d, q_stride_b, q_stride_n, o_stride_b, o_stride_n, nullptr, 1, N, eps,
                    io_dtype, out_dtype, pre, stream);
}
