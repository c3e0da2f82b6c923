// Softmax attention of many queries over a SHORT key set (the block's cross-attention to the text tokens:
// 16384 image tokens x 300 text tokens x 20 heads of 112 at the 4096 px latent), bf16 in and out.
//
//   out[b, n, h*d + :] = softmax_m(q[b, n, h, :] . k[b, m, h, :] * scale + bias[b, m]) . v[b, m, h, :]
//
// q and out are token-major [B, N, H*d] (what the linear layers on either side read and write: no head
// transposes), k and v are the two halves of the kv projection [B, Nk, 2, H*d].
//
// The key set of one (batch, head) fits LDS whole (Nk <= 320: K as [key][d padded to 32*DK] and V transposed as
// [d][key]: 150 KB at d = 112), so there is no online softmax: a wave takes 16*QT queries, multiplies them with
// all keys (v_mfma_f32_16x16x32_bf16, scores^T = K . Q^T: a lane owns one query and 4 keys of every 16-key tile),
// takes max / exp2 / sum in registers (two cross-lane steps over the four lane groups that share a query), and
// feeds the probabilities straight back as the column operand of out^T = V^T . P^T -- the k index of that
// product is permuted so that the 8 values a lane needs are the ones its own accumulators hold (keys
// 32s + 4g + {0..3} and 32s + 16 + 4g + {0..3} for lane group g), and V^T is stored in that key order.
// Workgroups are persistent over consecutive (batch, head, query block) items and restage K / V only when the
// (batch, head) changes.  Every K / V fragment read from LDS feeds QT MFMAs.
#include "common.h"

// Tuning knobs: query tiles of 16 per wave and pass (every K / V fragment read feeds that many MFMAs), waves per
// workgroup.  One tile and eight waves (two per SIMD, 196 registers) measured best: two tiles need either one wave
// per SIMD (nothing hides the LDS latency: 112 us against 75 us at 16384 x 300 x 20 heads of 112) or spill.
#ifndef SANA_XA_QT
#define SANA_XA_QT 1
#define SANA_XA_NW 8
#endif

namespace sana {
namespace {

constexpr int XA_NKP = 320;       // keys an LDS image holds (padded)
constexpr int XA_VPITCH = XA_NKP * 2;  // bytes per row of V^T

// 16-byte-slot swizzles that make 16 consecutive rows of one chunk hit 16 different bank groups
template <int DK>
__device__ __forceinline__ int xa_kkey(int row) {  // K rows of DK*64 bytes
  return DK == 4 ? (row & 15) : DK == 3 ? ((row >> 2) & 3) : DK == 2 ? ((row >> 1) & 7) : ((row >> 2) & 3);
}
// V^T rows of 640 bytes: rows alternate between the two halves of the bank space, (row / 2) % 8 spreads a 16-row
// fragment read over the 8 slots of a half; the (row / 16) % 4 term does the same for the transposing writes of
// the staging pass, whose lanes hold one key at rows 8 apart
__device__ __forceinline__ int xa_vkey(int row) { return ((row >> 1) ^ ((row >> 4) & 3)) & 7; }

// position of key m inside its group of 32 in V^T (and in the probability operand)
__device__ __forceinline__ int xa_vpos(int m) {
  const int s = m >> 5, w = m & 31, hi = w >> 4, g = (w >> 2) & 3, e = w & 3;
  return 32 * s + 8 * g + 4 * hi + e;
}

template <int DK, int DT, int QT, int NW, int NKT>
__global__ __launch_bounds__(64 * NW) void cross_attn_kernel(const uint16_t* __restrict__ q, const uint16_t* __restrict__ kv,
                                                         const float* __restrict__ bias, uint16_t* __restrict__ out, int B,
                                                         int N, int Nk, int H, int d, int64_t ldq, int64_t ldkv, int64_t ldo,
                                                         int64_t bias_stride, float scale_log2e, int qblocks, int items,
                                                         int items_per_wg) {
  constexpr int KPITCH = DK * 64, KCH = DK * 4;  // bytes / 16-byte chunks per K row
  constexpr int K_BYTES = XA_NKP * KPITCH, V_BYTES = DT * 16 * XA_VPITCH;
  __shared__ __attribute__((aligned(16))) unsigned char smem[K_BYTES + V_BYTES + XA_NKP * 4];
  unsigned char* sk = smem;
  unsigned char* sv = smem + K_BYTES;
  float* sb = reinterpret_cast<float*>(smem + K_BYTES + V_BYTES);  // per key: bias * log2(e), -inf past Nk
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int fr = lane & 15, fg = lane >> 4;

  int staged = -1;
  const int item0 = blockIdx.x * items_per_wg, item1 = min(items, item0 + items_per_wg);
  for (int item = item0; item < item1; ++item) {
    const int bh = item / qblocks, qb = item - bh * qblocks;
    const int b = bh / H, h = bh - b * H;
    if (bh != staged) {  // uniform
      __syncthreads();   // everyone is done with the previous head's K / V
      const uint16_t* kbase = kv + (int64_t)b * Nk * ldkv + (int64_t)h * d;
      const uint16_t* vbase = kbase + (int64_t)H * d;
      // a thread's loads go out in batches of SB before the LDS writes of the batch (the rows come out of the L2: one
      // load per round trip would make staging a chain of ~20 latencies)
      constexpr int NT = 64 * NW, SB = 5;
      for (int base = tid; base < XA_NKP * KCH; base += SB * NT) {
        u32x4_t val[SB];
#pragma unroll
        for (int i = 0; i < SB; ++i) {
          const int idx = base + i * NT, row = idx / KCH, c = idx - row * KCH;
          val[i] = u32x4_t{0u, 0u, 0u, 0u};
          if (row < Nk && 8 * c < d) val[i] = *reinterpret_cast<const u32x4_t*>(kbase + (int64_t)row * ldkv + 8 * c);
        }
#pragma unroll
        for (int i = 0; i < SB; ++i) {
          const int idx = base + i * NT, row = idx / KCH, c = idx - row * KCH;
          if (row < XA_NKP) *reinterpret_cast<u32x4_t*>(sk + row * KPITCH + ((c ^ xa_kkey<DK>(row)) << 4)) = val[i];
        }
      }
      // V^T: a thread takes 8 channels of one key and scatters them over 8 rows
      for (int base = tid; base < XA_NKP * DT * 2; base += SB * NT) {
        u32x4_t val[SB];
#pragma unroll
        for (int i = 0; i < SB; ++i) {
          const int idx = base + i * NT, row = idx / (DT * 2), c = idx - row * (DT * 2);
          val[i] = u32x4_t{0u, 0u, 0u, 0u};
          if (row < Nk && 8 * c < d) val[i] = *reinterpret_cast<const u32x4_t*>(vbase + (int64_t)row * ldkv + 8 * c);
        }
#pragma unroll
        for (int i = 0; i < SB; ++i) {
          const int idx = base + i * NT, row = idx / (DT * 2), c = idx - row * (DT * 2);
          if (row < XA_NKP) {
            const int p = xa_vpos(row);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const int dr = 8 * c + e;
              const uint16_t x = (uint16_t)(e & 1 ? val[i][e >> 1] >> 16 : val[i][e >> 1] & 0xffffu);
              *reinterpret_cast<uint16_t*>(sv + dr * XA_VPITCH + (((p >> 3) ^ xa_vkey(dr)) << 4) + (p & 7) * 2) = x;
            }
          }
        }
      }
      for (int m = tid; m < XA_NKP; m += 64 * NW)
        sb[m] = m < Nk ? (bias ? bias[(int64_t)b * bias_stride + m] * 1.44269504088896341f : 0.f) : -INFINITY;
      __syncthreads();
      staged = bh;
    }
    const int q0 = qb * (NW * 16 * QT) + wave * (16 * QT);
    if (q0 >= N) continue;  // (no barrier inside the per-item work below)
    const uint16_t* qbase = q + ((int64_t)b * N) * ldq + (int64_t)h * d;

    // ---- Q fragments: column operand, lane -> query fr, k = 32*ks + 8*fg .. +7
    u32x4_t qf[QT][DK];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
      const int qi = q0 + 16 * t + fr;
#pragma unroll
      for (int ks = 0; ks < DK; ++ks) {
        const int k0 = 32 * ks + 8 * fg;
        qf[t][ks] = (qi < N && k0 < d) ? *reinterpret_cast<const u32x4_t*>(qbase + (int64_t)qi * ldq + k0)
                                       : u32x4_t{0u, 0u, 0u, 0u};
      }
    }
    // ---- scores^T = K . Q^T: acc[t][kt][r] = query 16t + fr, key 16*kt + 4*fg + r
    f32x4_t sc[QT][NKT];
#pragma unroll
    for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
      for (int t = 0; t < QT; ++t) sc[t][kt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    // key tiles in pairs (two independent accumulator chains), the next pair's fragments requested before
    // this pair's MFMAs
    u32x4_t kf[2][2][DK];
    auto load_k = [&](int buf, int kp) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int row = 16 * (2 * kp + j) + fr;
        const unsigned char* rp = sk + row * KPITCH;
        const int key = xa_kkey<DK>(row);
#pragma unroll
        for (int ks = 0; ks < DK; ++ks) kf[buf][j][ks] = *reinterpret_cast<const u32x4_t*>(rp + (((4 * ks + fg) ^ key) << 4));
      }
    };
    load_k(0, 0);
#pragma unroll
    for (int kp = 0; kp < NKT / 2; ++kp) {
      if (kp + 1 < NKT / 2) load_k((kp + 1) & 1, kp + 1);
#pragma unroll
      for (int ks = 0; ks < DK; ++ks)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int t = 0; t < QT; ++t)
            sc[t][2 * kp + j] = mfma_16x16x32_bf16(kf[kp & 1][j][ks], qf[t][ks], sc[t][2 * kp + j]);
    }
    // ---- softmax over the keys of each query (log2 domain), probabilities back as packed bf16
    float rsum[QT];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
      float mx = -INFINITY;
#pragma unroll
      for (int kt = 0; kt < NKT; ++kt) {
        const f32x4_t kb = *reinterpret_cast<const f32x4_t*>(sb + 16 * kt + 4 * fg);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          sc[t][kt][r] = fmaf(sc[t][kt][r], scale_log2e, kb[r]);
          mx = fmaxf(mx, sc[t][kt][r]);
        }
      }
      mx = fmaxf(mx, __shfl_xor(mx, 16));
      mx = fmaxf(mx, __shfl_xor(mx, 32));
      float sum = 0.f;
#pragma unroll
      for (int kt = 0; kt < NKT; ++kt) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float p = __builtin_amdgcn_exp2f(sc[t][kt][r] - mx);  // rounded to bf16 where it is packed below
          sc[t][kt][r] = p;
          sum += p;
        }
      }
      sum += __shfl_xor(sum, 16);
      sum += __shfl_xor(sum, 32);
      rsum[t] = 1.0f / sum;
    }
    // ---- out^T = V^T . P^T: acc[t][dt][r] = query 16t + fr, channel 16*dt + 4*fg + r
    f32x4_t oc[QT][DT];
#pragma unroll
    for (int t = 0; t < QT; ++t)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) oc[t][dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    u32x4_t vf[2][DT];
    auto load_v = [&](int buf, int s) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const int row = 16 * dt + fr;
        vf[buf][dt] = *reinterpret_cast<const u32x4_t*>(sv + row * XA_VPITCH + (((4 * s + fg) ^ xa_vkey(row)) << 4));
      }
    };
    load_v(0, 0);
#pragma unroll
    for (int s = 0; s < NKT / 2; ++s) {
      if (s + 1 < NKT / 2) load_v((s + 1) & 1, s + 1);
      u32x4_t pf[QT];
#pragma unroll
      for (int t = 0; t < QT; ++t) {
        pf[t].x = pack_bf16(sc[t][2 * s][0], sc[t][2 * s][1]);
        pf[t].y = pack_bf16(sc[t][2 * s][2], sc[t][2 * s][3]);
        pf[t].z = pack_bf16(sc[t][2 * s + 1][0], sc[t][2 * s + 1][1]);
        pf[t].w = pack_bf16(sc[t][2 * s + 1][2], sc[t][2 * s + 1][3]);
      }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int t = 0; t < QT; ++t) oc[t][dt] = mfma_16x16x32_bf16(vf[s & 1][dt], pf[t], oc[t][dt]);
    }
    // ---- normalise and store: a lane holds 4 consecutive channels of its query per channel tile
    uint16_t* obase = out + ((int64_t)b * N) * ldo + (int64_t)h * d;
#pragma unroll
    for (int t = 0; t < QT; ++t) {
      const int qi = q0 + 16 * t + fr;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const int c0 = 16 * dt + 4 * fg;
        if (qi < N && c0 < d) {
          u32x2_t o;
          o.x = pack_bf16(oc[t][dt][0] * rsum[t], oc[t][dt][1] * rsum[t]);
          o.y = pack_bf16(oc[t][dt][2] * rsum[t], oc[t][dt][3] * rsum[t]);
          *reinterpret_cast<u32x2_t*>(obase + (int64_t)qi * ldo + c0) = o;
        }
      }
    }
  }
}

template <int DK, int DT, int QT, int NW, int NKT>
int launch_xa(const uint16_t* q, const uint16_t* kv, const float* bias, uint16_t* out, int B, int N, int Nk, int H, int d,
              int64_t ldq, int64_t ldkv, int64_t ldo, int64_t bias_stride, float scale, hipStream_t s) {
  const int qblocks = (N + NW * 16 * QT - 1) / (NW * 16 * QT);
  const int64_t items64 = (int64_t)B * H * qblocks;
  if (items64 > 0x7fffffff) return SANA_ERR_SHAPE;
  const int items = (int)items64, cus = 256;
  const int ipw = (items + cus - 1) / cus;
  const int grid = (items + ipw - 1) / ipw;
  hipLaunchKernelGGL((cross_attn_kernel<DK, DT, QT, NW, NKT>), dim3((unsigned)grid), dim3(64 * NW), 0, s, q, kv, bias, out, B, N, Nk, H, d,
                     ldq, ldkv, ldo, bias_stride, scale * 1.44269504088896341f, qblocks, items, ipw);
  return hipGetLastError() == hipSuccess ? SANA_OK : SANA_ERR_LAUNCH;
}

}  // namespace
}  // namespace sana

using namespace sana;

extern "C" __attribute__((visibility("default"))) int sana_hip_cross_attention(
    const void* q, const void* kv, const float* key_bias, void* out, int B, int N, int Nk, int H, int d, int64_t ldq,
    int64_t ldkv, int64_t ldo, int64_t bias_stride, float scale, void* stream) {
  if (!q || !kv || !out || B <= 0 || N <= 0 || Nk <= 0 || H <= 0 || d <= 0) return SANA_ERR_ARG;
  if (Nk > XA_NKP || d % 8 || d > 112 || d <= 64) return SANA_ERR_SHAPE;  // LDS: K + V^T of one head at d <= 112
  if (ldq < (int64_t)H * d || ldkv < 2 * (int64_t)H * d || ldo < (int64_t)H * d || (key_bias && bias_stride < Nk))
    return SANA_ERR_ARG;
  if (ldq % 8 || ldkv % 8 || ldo % 4 || !aligned16(q) || !aligned16(kv) || (reinterpret_cast<uintptr_t>(out) & 7u))
    return SANA_ERR_ALIGN;
  const uint16_t* qp = static_cast<const uint16_t*>(q);
  const uint16_t* kp = static_cast<const uint16_t*>(kv);
  uint16_t* op = static_cast<uint16_t*>(out);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define SANA_XA_GO(DK, DT, NKT) \
  launch_xa<DK, DT, SANA_XA_QT, SANA_XA_NW, NKT>(qp, kp, key_bias, op, B, N, Nk, H, d, ldq, ldkv, ldo, bias_stride, scale, s)
  // key tiles of 16 that are multiplied: all 20, or 10 for up to 160 keys (tiles past Nk hold zeros and -inf)
  if (d > 96) return Nk > 160 ? SANA_XA_GO(4, 7, 20) : SANA_XA_GO(4, 7, 10);
  return Nk > 160 ? SANA_XA_GO(3, 6, 20) : SANA_XA_GO(3, 6, 10);
#undef SANA_XA_GO
}
