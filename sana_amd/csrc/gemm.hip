// bf16 MFMA GEMM for gfx950:  C[M][N] = epilogue(A[M][K] . W[N][K]^T)
// with an int8-weight (W8A16) variant dequantised on the way into LDS.
//
// Both operands are K-contiguous, which is exactly the MFMA operand layout (a
// lane holds 8 consecutive k of one row), so nothing is transposed.  The MFMA
// "row" operand is the WEIGHT tile and the "column" operand the ACTIVATION
// tile: in the 32x32 accumulator layout a lane then owns one token (column)
// and 16 output channels.  Weight rows are stored to LDS in a permuted order
// (row 16*g + 4*q + s of a 32-row block goes to LDS row 8*q + 4*g + s) so that
// those 16 channels are contiguous and a lane stores 32 contiguous bytes of C.
//
// Workgroup tile 256 (tokens) x 256 (channels) x 64 (k), four waves in 2x2,
// each 128x128 = 4x4 MFMA 32x32x16 tiles (256 fp32 accumulators).  LDS is
// double buffered (2 x 64 KB); 16-byte chunks are XOR-swizzled by (row & 7) so
// that ds_read_b128 / ds_write_b128 are bank-conflict free.  Workgroup ids are
// remapped so that each XCD (own L2) works on a compact group of tiles.
#include "common.h"

namespace sana {
namespace {

constexpr int BT = 256;   // tokens (rows of A / C) per workgroup
constexpr int BC = 256;   // output channels (rows of W) per workgroup
constexpr int BK = 64;
constexpr int ROW_BYTES = BK * 2;            // 128
constexpr int TILE_BYTES = 256 * ROW_BYTES;  // 32 KB per operand per stage

__device__ __forceinline__ int swz(int row, int chunk) { return row * ROW_BYTES + ((chunk ^ (row & 7)) << 4); }

// LDS row of weight row n (within the 256-row tile): permute inside each 32-row block
__device__ __forceinline__ int wrow_to_lds(int n) {
  const int blk = n & ~31, r = n & 31;
  return blk + 8 * ((r >> 2) & 3) + 4 * (r >> 4) + (r & 3);
}

__device__ __forceinline__ uint32_t dequant2(uint32_t q4, int which, float s, float off) {
  // two int8 (bytes 2*which, 2*which+1 of q4, already biased by +128) -> packed bf16(q*s)
  // (the compiler turns these byte extracts into v_cvt_f32_ubyteN)
  const float f0 = (float)((q4 >> (16 * which)) & 0xffu);
  const float f1 = (float)((q4 >> (16 * which + 8)) & 0xffu);
  // (q+128)*s - 128*s == q*s exactly before the single fp32 rounding
  return pack_bf16(fmaf(f0, s, off), fmaf(f1, s, off));
}

template <bool W8, int EPI>
__global__ __launch_bounds__(256) void gemm_kernel(const uint16_t* __restrict__ A, const void* __restrict__ Wv,
                                                   const float* __restrict__ scale,
                                                   const uint16_t* __restrict__ bias, uint16_t* __restrict__ C,
                                                   int M, int N, int K, int64_t lda, int64_t ldw, int64_t ldc,
                                                   int tiles_t, int tiles_c) {
  __shared__ __attribute__((aligned(16))) unsigned char smem[4 * TILE_BYTES];  // [stage][A | W]
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
  // A tile: 256 rows x 8 chunks(16 B); thread -> chunk tid%8, rows tid/8 + 32*i
  const int a_chunk = tid & 7, a_row = tid >> 3;
  u32x4_t ra[8];
  // W tile bf16: same shape.  W8: 256 rows x 4 chunks of 16 int8; thread -> chunk tid%4, rows tid/4 + 64*i
  u32x4_t rw[W8 ? 4 : 8];
  const int w_chunk = W8 ? (tid & 3) : (tid & 7), w_row = W8 ? (tid >> 2) : (tid >> 3);
  const u32x4_t zero4 = {0u, 0u, 0u, 0u};

  auto load_tile = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int m = m0 + a_row + 32 * i, k = k0 + a_chunk * 8;
      ra[i] = (m < M && k < K) ? *reinterpret_cast<const u32x4_t*>(A + (int64_t)m * lda + k) : zero4;
    }
    if (W8) {
      const int8_t* Wq = static_cast<const int8_t*>(Wv);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = n0 + w_row + 64 * i, k = k0 + w_chunk * 16;
        // rows are 16-byte aligned and K % 16 == 0 on this path
        rw[i] = (n < N && k < K) ? *reinterpret_cast<const u32x4_t*>(Wq + (int64_t)n * ldw + k) : zero4;
      }
    } else {
      const uint16_t* Wb = static_cast<const uint16_t*>(Wv);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int n = n0 + w_row + 32 * i, k = k0 + w_chunk * 8;
        rw[i] = (n < N && k < K) ? *reinterpret_cast<const u32x4_t*>(Wb + (int64_t)n * ldw + k) : zero4;
      }
    }
  };
  float wscale[4], woff[4];
  if (W8) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = n0 + w_row + 64 * i;
      wscale[i] = n < N ? scale[n] : 0.f;
      woff[i] = -128.f * wscale[i];
    }
  }
  auto store_tile = [&](int stage) {
    unsigned char* sa = smem + stage * 2 * TILE_BYTES;
    unsigned char* sw = sa + TILE_BYTES;
#pragma unroll
    for (int i = 0; i < 8; ++i) *reinterpret_cast<u32x4_t*>(sa + swz(a_row + 32 * i, a_chunk)) = ra[i];
    if (W8) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int lrow = wrow_to_lds(w_row + 64 * i);
        u32x4_t q = rw[i];
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
      for (int i = 0; i < 8; ++i)
        *reinterpret_cast<u32x4_t*>(sw + swz(wrow_to_lds(w_row + 32 * i), w_chunk)) = rw[i];
    }
  };

  // ---- MFMA tiling: wave (wc, wt) owns channels [wc*128, +128) x tokens [wt*128, +128)
  const int wc = wave & 1, wt = wave >> 1;
  const int fr = lane & 31, fg = lane >> 5;
  f32x16_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int KT = (K + BK - 1) / BK;
  load_tile(0);
  store_tile(0);
  __syncthreads();
  for (int kt = 0; kt < KT; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < KT) load_tile((kt + 1) * BK);
    const unsigned char* sa = smem + cur * 2 * TILE_BYTES;
    const unsigned char* sw = sa + TILE_BYTES;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      u32x4_t fw[4], fa[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        fw[i] = *reinterpret_cast<const u32x4_t*>(sw + swz(wc * 128 + 32 * i + fr, 2 * ks + fg));
#pragma unroll
      for (int j = 0; j < 4; ++j)
        fa[j] = *reinterpret_cast<const u32x4_t*>(sa + swz(wt * 128 + 32 * j + fr, 2 * ks + fg));
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, fw[i]),
                                                             __builtin_bit_cast(bf16x8_t, fa[j]), acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < KT) store_tile(cur ^ 1);
    __syncthreads();
  }

  // ---- epilogue.  acc[i][j][r]: token m0 + wt*128 + 32*j + lane%32,
  // channel n0 + wc*128 + 32*i + 16*(lane/32) + r
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int n = n0 + wc * 128 + 32 * i + 16 * fg;
    float bv[16];
    if (EPI != SANA_EPI_NONE) {
#pragma unroll
      for (int r = 0; r < 16; ++r) bv[r] = (n + r < N) ? bf16_bits_to_f32(bias[n + r]) : 0.f;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int m = m0 + wt * 128 + 32 * j + fr;
      if (m >= M) continue;
      float v[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float x = acc[i][j][r];
        if (EPI != SANA_EPI_NONE) x += bv[r];
        if (EPI == SANA_EPI_BIAS_SILU) x = silu_f32(round_bf16(x));  // the reference rounds before the activation
        v[r] = x;
      }
      uint16_t* cp = C + (int64_t)m * ldc + n;
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        if (n + 8 * half < N) {  // N % 8 == 0: a chunk is either fully inside or outside
          u32x4_t o;
          o.x = pack_bf16(v[8 * half + 0], v[8 * half + 1]);
          o.y = pack_bf16(v[8 * half + 2], v[8 * half + 3]);
          o.z = pack_bf16(v[8 * half + 4], v[8 * half + 5]);
          o.w = pack_bf16(v[8 * half + 6], v[8 * half + 7]);
          *reinterpret_cast<u32x4_t*>(cp + 8 * half) = o;
        }
      }
    }
  }
}

template <bool W8>
int launch(const void* A, const void* W, const float* scale, const void* bias, void* C, int M, int N, int K,
           int64_t lda, int64_t ldw, int64_t ldc, int epilogue, hipStream_t s) {
  const int tiles_t = (M + BT - 1) / BT, tiles_c = (N + BC - 1) / BC;
  const int64_t total = (int64_t)tiles_t * tiles_c;
  if (total > (1 << 30)) return SANA_ERR_SHAPE;
  dim3 grid((unsigned)total), block(256);
  const uint16_t* a = static_cast<const uint16_t*>(A);
  const uint16_t* b = static_cast<const uint16_t*>(bias);
  uint16_t* c = static_cast<uint16_t*>(C);
  switch (epilogue) {
    case SANA_EPI_NONE:
      hipLaunchKernelGGL((gemm_kernel<W8, SANA_EPI_NONE>), grid, block, 0, s, a, W, scale, b, c, M, N, K, lda, ldw,
                         ldc, tiles_t, tiles_c);
      break;
    case SANA_EPI_BIAS:
      hipLaunchKernelGGL((gemm_kernel<W8, SANA_EPI_BIAS>), grid, block, 0, s, a, W, scale, b, c, M, N, K, lda, ldw,
                         ldc, tiles_t, tiles_c);
      break;
    case SANA_EPI_BIAS_SILU:
      hipLaunchKernelGGL((gemm_kernel<W8, SANA_EPI_BIAS_SILU>), grid, block, 0, s, a, W, scale, b, c, M, N, K, lda,
                         ldw, ldc, tiles_t, tiles_c);
      break;
    default:
      return SANA_ERR_ARG;
  }
  return hipGetLastError() == hipSuccess ? SANA_OK : SANA_ERR_LAUNCH;
}

int check_common(const void* A, const void* W, const void* bias, const void* C, int M, int N, int K, int64_t lda,
                 int64_t ldw, int64_t ldc, int epilogue, int kmult, int ldw_mult) {
  if (!A || !W || !C || M <= 0 || N <= 0 || K <= 0) return SANA_ERR_ARG;
  if (epilogue != SANA_EPI_NONE && !bias) return SANA_ERR_ARG;
  if (epilogue < SANA_EPI_NONE || epilogue > SANA_EPI_BIAS_SILU) return SANA_ERR_ARG;
  if (K % kmult || N % 8) return SANA_ERR_SHAPE;
  if (lda < K || ldw < K || ldc < N) return SANA_ERR_ARG;
  if (lda % 8 || ldw % ldw_mult || ldc % 8 || !aligned16(A) || !aligned16(W) || !aligned16(C)) return SANA_ERR_ALIGN;
  return SANA_OK;
}

}  // namespace
}  // namespace sana

using namespace sana;

extern "C" __attribute__((visibility("default"))) int sana_hip_gemm_bf16(const void* A, const void* W,
                                                                         const void* bias, void* C, int M, int N,
                                                                         int K, int64_t lda, int64_t ldw,
                                                                         int64_t ldc, int epilogue, void* stream) {
  const int rc = check_common(A, W, bias, C, M, N, K, lda, ldw, ldc, epilogue, 8, 8);
  if (rc != SANA_OK) return rc;
  return launch<false>(A, W, nullptr, bias, C, M, N, K, lda, ldw, ldc, epilogue, static_cast<hipStream_t>(stream));
}

extern "C" __attribute__((visibility("default"))) int sana_hip_gemm_w8a16(const void* A, const int8_t* Wq,
                                                                          const float* scale, const void* bias,
                                                                          void* C, int M, int N, int K, int64_t lda,
                                                                          int64_t ldw, int64_t ldc, int epilogue,
                                                                          void* stream) {
  if (!scale) return SANA_ERR_ARG;
  const int rc = check_common(A, Wq, bias, C, M, N, K, lda, ldw, ldc, epilogue, 16, 16);
  if (rc != SANA_OK) return rc;
  return launch<true>(A, Wq, scale, bias, C, M, N, K, lda, ldw, ldc, epilogue, static_cast<hipStream_t>(stream));
}
