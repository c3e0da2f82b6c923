// Pieces shared by the head_dim-32 and head_dim-112 linear-attention kernels.
#pragma once
#include "common.h"

namespace sana {

struct ChunkRange {
  int begin, end;
};
__device__ __forceinline__ ChunkRange chunk_range(const int32_t* chunk_starts, int c, int N) {
  ChunkRange r;
  if (chunk_starts) {
    r.begin = chunk_starts[c];
    r.end = chunk_starts[c + 1];
  } else {
    r.begin = 0;
    r.end = N;
  }
  return r;
}

// Optional transforms of q / k on load (bf16 io): RMSNorm over all channels of the token
// (per-token 1/rms from a statistics pass, per-channel weight), applied before the ReLU, and the
// rotary embedding applied after it.  The rotation acts on adjacent channel pairs (2i, 2i+1) of a
// head, i.e. on the two halves of one packed dword; only the numerator operands are rotated, the
// ksum row / denominator use the unrotated values.
struct QkPre {
  const float* rinv;       // [B][N], or null
  const uint16_t* weight;  // [h*d] bf16, with rinv
  const float* rope;       // [N][d/2][2] (cos, sin) per token and pair of a head, or null
  // 0: rotation after the ReLU, numerator operands only (LiteLAReLURope and the chunk-causal family);
  // 1: rotation BEFORE the ReLU, rounded to the io dtype, and everything -- numerator, ksum row, denominator --
  //    uses the rotated values (LiteLA.forward with image_rotary_emb, sana_blocks.py:282-286).  head_dim 32 only.
  int rope_first;
};

// bf16(w * (x * rinv)): the float chain of the reference RMSNorm, rounded once at the end
__device__ __forceinline__ u32x4_t rms_scale8(u32x4_t x, float rinv, u32x4_t w) {
  u32x4_t o;
#pragma unroll
  for (int e = 0; e < 4; ++e)
    o[e] = pack_bf16(bf16_lo(w[e]) * (bf16_lo(x[e]) * rinv), bf16_hi(w[e]) * (bf16_hi(x[e]) * rinv));
  return o;
}
// (x0 + i x1)(cos + i sin) on the four channel pairs of x; cs0 = (c, s) of pairs 0, 1; cs1 of pairs 2, 3
__device__ __forceinline__ u32x4_t rope8(u32x4_t x, f32x4_t cs0, f32x4_t cs1) {
  const float c[4] = {cs0[0], cs0[2], cs1[0], cs1[2]}, sn[4] = {cs0[1], cs0[3], cs1[1], cs1[3]};
  u32x4_t o;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float x0 = bf16_lo(x[e]), x1 = bf16_hi(x[e]);
    o[e] = pack_bf16(fmaf(x0, c[e], -(x1 * sn[e])), fmaf(x0, sn[e], x1 * c[e]));
  }
  return o;
}


// host-side launchers of the head_dim-112 kernels (linattn112.hip), bf16 io (state also f16); arguments as
// the C entry points, already validated by them
int launch_state112(const void* k, const void* v, float* state, void* workspace, size_t workspace_bytes, int B, int N,
                    int h, int64_t stride_b, int64_t stride_n, const int32_t* chunk_starts, int n_chunks,
                    int max_chunk_tokens, int causal, int io_dtype, const QkPre& pre, hipStream_t stream);
int launch_apply112(const void* q, const float* state, void* out, int B, int N, int h, int64_t q_stride_b,
                    int64_t q_stride_n, int64_t o_stride_b, int64_t o_stride_n, const int32_t* chunk_starts,
                    int n_chunks, int max_chunk_tokens, float eps, int io_dtype, int out_dtype, const QkPre& pre,
                    hipStream_t stream);
int launch_scan112(float* state, int B, int h, int n_chunks, hipStream_t stream);  // in-place prefix over chunks
size_t workspace_bytes112(int B, int h, int n_chunks, int max_chunk_tokens);

}  // namespace sana
