/* sana_hip.h — C ABI of libsana_hip.so: hand-written gfx950 (MI355X) kernels
 * for the SanaMSBlock hot path (LiteLA linear attention + GLUMBConv Mix-FFN).
 *
 * Conventions
 *   - Every pointer is a DEVICE pointer unless the comment says "host".
 *   - The caller owns every buffer.  The library allocates nothing and keeps
 *     no global state; scratch space is passed in as `workspace`.  (The one
 *     exception is sana_hip_linattn_state_noalloc, whose scratch is a fixed
 *     array inside the library image.)
 *   - All work is enqueued on `stream` (a hipStream_t passed as void*; NULL is
 *     the default stream).  No entry point synchronises with the host.
 *   - Return value: SANA_OK (0) or a negative SANA_ERR_* code.  Nothing is
 *     launched when an error is returned.  sana_hip_strerror() names a code.
 *   - Strides are in ELEMENTS of the io dtype.  The channel stride is always 1.
 *   - Channel c belongs to head c / d, lane c % d.  d = head_dim is 32 (every io dtype;
 *     the image models) or 112 (bf16 io, f16 for phase 1 only; the `linear_head_dim: 112`
 *     video models); any other d returns SANA_ERR_SHAPE.
 *
 * The reference (NVlabs/Sana) has no native seam for this path: its seam is the
 * Python module API (attn_type / ffn_type selection,
 * diffusion/model/nets/sana_multi_scale.py:77-140).  Each entry point below
 * names the reference code it replaces.
 */
#ifndef SANA_HIP_H_
#define SANA_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SANA_HIP_ABI_VERSION 8

/* io dtypes */
#define SANA_DT_F32 0
#define SANA_DT_BF16 1
#define SANA_DT_F16 2

/* error codes */
#define SANA_OK 0
#define SANA_ERR_ARG (-1)        /* null pointer, negative size, unknown enum      */
#define SANA_ERR_SHAPE (-2)      /* shape outside what the kernels support         */
#define SANA_ERR_ALIGN (-3)      /* pointer or stride not 16-byte aligned          */
#define SANA_ERR_WORKSPACE (-4)  /* workspace missing or too small                 */
#define SANA_ERR_LAUNCH (-5)     /* hipLaunchKernel reported an error              */
#define SANA_ERR_DTYPE (-6)      /* dtype not supported by this entry point        */
#define SANA_ERR_SCRATCH_LIMIT (-7) /* needs more than SANA_HIP_NOALLOC_SCRATCH_BYTES */
#define SANA_ERR_RUNTIME (-8)    /* a HIP runtime call (device / symbol lookup) failed */

/* GEMM epilogues */
#define SANA_EPI_NONE 0       /* C = A W^T                       */
#define SANA_EPI_BIAS 1       /* C = A W^T + bias                */
#define SANA_EPI_BIAS_SILU 2  /* C = silu(A W^T + bias)          */

int sana_hip_abi_version(void);
const char* sana_hip_strerror(int code);

/* ---------------------------------------------------------------------------
 * ReLU linear attention, phase 1: per-(batch, head[, chunk]) state
 *
 *   state[b][h][c][i][j] = sum over tokens n of chunk c of
 *                          vpad[n][i] * relu(k[n][j]),   i in 0..d, j in 0..d-1
 *   vpad[n][d] = 1, so row d is sum_n relu(k[n]).
 *
 * Replaces `relu(k)`, `F.pad(v, value=1)` and `vk = v @ k` of
 * LiteLA.attn_matmul (diffusion/model/nets/sana_blocks.py:248-256) and the
 * reference's Triton kernel pad_vk_mm_fwd
 * (diffusion/model/nets/fastlinear/modules/triton_lite_mla_kernels/pad_vk_mm_fwd.py:60-151).
 * With n_chunks > 1 and causal != 0 the states are additionally turned into an
 * inclusive prefix sum over chunks (cumsum_vk / cumsum_k_sum of
 * ChunkCausalAttention.forward, sana_blocks.py:481-485, rotary = identity).
 *
 *   k, v          [B][N][h*d] views: element (b, n, c) at b*stride_b + n*stride_n + c
 *   state         fp32 [B][h][n_chunks][d+1][d], contiguous
 *   chunk_starts  int32 [n_chunks+1] token offsets (0 = first, N = last), or NULL
 *                 when n_chunks == 1
 *   max_chunk_tokens  host value: the longest chunk, in tokens
 *   workspace     at least sana_hip_linattn_workspace_bytes(...) bytes, 16-byte aligned
 *                 (may be NULL when that function returns 0)
 * Accumulation is fp32 and deterministic (fixed summation order, no atomics).
 * d = 112 addresses the tokens of one batch entry with 32-bit byte offsets:
 * N * stride_n * 2 and N * 448 must stay below 2^31; its grids also want
 * B <= 65535 and B * h <= 2^22 (SANA_ERR_SHAPE otherwise).
 */
size_t sana_hip_linattn_workspace_bytes(int B, int h, int d, int n_chunks, int max_chunk_tokens,
                                        int io_dtype);

int sana_hip_linattn_state(const void* k, const void* v, float* state,
                           void* workspace, size_t workspace_bytes,
                           int B, int N, int h, int d,
                           int64_t stride_b, int64_t stride_n,
                           const int32_t* chunk_starts, int n_chunks, int max_chunk_tokens,
                           int causal, int io_dtype, void* stream);

/* Inclusive prefix sum over the chunk axis of fp32 [B][h][n_chunks][d+1][d],
 * in place.  The accumulation the streaming pipeline performs on the host side
 * (diffusion/longsana/pipeline/sana_inference_pipeline.py:242-263). */
int sana_hip_linattn_chunk_scan(float* state, int B, int h, int d, int n_chunks, void* stream);

/* ---------------------------------------------------------------------------
 * ReLU linear attention, phase 2: apply the state to relu(q) and divide
 *
 *   out[n][i] = sum_j state[i][j] relu(q[n][j])
 *               / (sum_j state[d][j] relu(q[n][j]) + eps)
 * with the state of the chunk token n belongs to.
 *
 * Replaces `relu(q)`, `out = vk @ q`, `.float()`, the slice/divide of
 * LiteLA.attn_matmul (sana_blocks.py:248,257-261) and the `.to(dtype)` of
 * LiteLA.forward (:286); Triton twin vk_q_mm_divide_fwd
 * (triton_lite_mla_kernels/vk_q_mm_divide_fwd.py:60-164).  eps is a runtime
 * value (1e-15 class default, 1e-8 inside SanaMSBlock).
 *
 *   q    [B][N][h*d] view (q_stride_b, q_stride_n), io dtype
 *   out  [B][N][h*d] view (o_stride_b, o_stride_n), out_dtype = io dtype or SANA_DT_F32
 */
int sana_hip_linattn_apply(const void* q, const float* state, void* out,
                           int B, int N, int h, int d,
                           int64_t q_stride_b, int64_t q_stride_n,
                           int64_t o_stride_b, int64_t o_stride_n,
                           const int32_t* chunk_starts, int n_chunks, int max_chunk_tokens,
                           float eps, int io_dtype, int out_dtype, void* stream);

/* ---------------------------------------------------------------------------
 * q/k RMSNorm and rotary embedding inside the attention kernels (bf16 io)
 *
 * LiteLAReLURope / ChunkCausalAttention / CachedCausalAttention
 * (sana_blocks.py:304-388, 391-495, 498-572) normalise q and k over ALL channels
 * of a token before the head split (`self.q_norm(q)`, RMSNorm of
 * diffusion/model/norms.py:182-231: weight * (x.float() * rsqrt(mean(x^2) + eps)),
 * rounded to the io dtype), apply ReLU, then rotate adjacent channel pairs
 * (2i, 2i+1) of every head by the complex factor freqs[n][i] (`apply_rotary_emb`,
 * sana_blocks.py:359-362).  Only the numerator uses the rotated values:
 *   vk = v @ k_rot^T,  out = vk @ q_rot,   z = 1 / (sum_n k[n] . q + eps).
 *
 * sana_hip_qk_rms writes the per-token statistic rsqrt(mean_c x[n][c]^2 + eps) of q
 * and of k ([B][N] fp32 each).  The *_pre variants of the two attention phases take
 *   rinv    [B][N] fp32 from sana_hip_qk_rms, or NULL (no norm)
 *   weight  [h*d] bf16 RMSNorm weight (required with rinv)
 *   rope    [N][d/2][2] fp32 (cos, sin) of freqs[n][i], shared by batch and heads, or NULL
 * and are otherwise identical to sana_hip_linattn_state / sana_hip_linattn_apply
 * (with all three NULL they are the same call).  SANA_ERR_DTYPE unless io is bf16.
 */
int sana_hip_qk_rms(const void* q, const void* k, float* q_rinv, float* k_rinv,
                    int B, int N, int C, int64_t stride_b, int64_t stride_n,
                    float eps, int io_dtype, void* stream);

int sana_hip_linattn_state_pre(const void* k, const void* v, float* state,
                               void* workspace, size_t workspace_bytes,
                               int B, int N, int h, int d,
                               int64_t stride_b, int64_t stride_n,
                               const int32_t* chunk_starts, int n_chunks, int max_chunk_tokens,
                               int causal, int io_dtype,
                               const float* k_rinv, const void* k_weight, const float* rope,
                               void* stream);

int sana_hip_linattn_apply_pre(const void* q, const float* state, void* out,
                               int B, int N, int h, int d,
                               int64_t q_stride_b, int64_t q_stride_n,
                               int64_t o_stride_b, int64_t o_stride_n,
                               const int32_t* chunk_starts, int n_chunks, int max_chunk_tokens,
                               float eps, int io_dtype, int out_dtype,
                               const float* q_rinv, const void* q_weight, const float* rope,
                               void* stream);

/* ---------------------------------------------------------------------------
 * The transform order of LiteLA.forward itself (diffusion/model/nets/sana_blocks.py:274-286): q and k are
 * RMS-normalised over all channels (`self.q_norm(q)`, :274-275), rotated BEFORE the ReLU by the real-valued rotary
 * embedding (`apply_rotary_emb(q, rotary_emb, use_real_unbind_dim=-2)`, :282-284 and :1549-1582: channel pairs
 * (2i, 2i+1) of a head, out = x * cos + rot(x) * sin in fp32, rounded to the io dtype), and only then enter
 * attn_matmul (:286), whose ReLU, vk, ksum row and denominator all see the rotated values.
 *   rope  [N][d/2][2] fp32 (cos, sin) of pair i -- the reference's cos / sin tables [N][d] with their two entries
 *         per pair equal (what its table builders produce) -- or NULL;  rinv / weight as for the *_pre entry points.
 * One chunk (LiteLA is not chunk-causal), head_dim 32, bf16 io (SANA_ERR_SHAPE / SANA_ERR_DTYPE otherwise); with
 * rope NULL these are sana_hip_linattn_state_pre / sana_hip_linattn_apply_pre. */
int sana_hip_litela_state(const void* k, const void* v, float* state,
                          void* workspace, size_t workspace_bytes,
                          int B, int N, int h, int d, int64_t stride_b, int64_t stride_n, int io_dtype,
                          const float* k_rinv, const void* k_weight, const float* rope, void* stream);

int sana_hip_litela_apply(const void* q, const float* state, void* out,
                          int B, int N, int h, int d,
                          int64_t q_stride_b, int64_t q_stride_n, int64_t o_stride_b, int64_t o_stride_n,
                          float eps, int io_dtype, int out_dtype,
                          const float* q_rinv, const void* q_weight, const float* rope, void* stream);

/* ---------------------------------------------------------------------------
 * Phase 1 for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.
 *
 * Same computation, arguments and result as sana_hip_linattn_state_pre (with k_rinv, k_weight and rope NULL: as
 * sana_hip_linattn_state), but there is no workspace argument: the per-split partial states go to a fixed
 * SANA_HIP_NOALLOC_SCRATCH_BYTES array of device memory that is part of the library image (every GPU the library
 * runs on holds its own copy until the process ends).  The call allocates and frees nothing.
 *   - A problem whose sana_hip_linattn_workspace_bytes(...) exceeds SANA_HIP_NOALLOC_SCRATCH_BYTES returns
 *     SANA_ERR_SCRATCH_LIMIT and launches nothing (the block shapes of the benchmark configurations need
 *     7.3 - 20.3 MiB, one video of 21 causal chunks with 20 heads of 112 30.9 MiB).
 *   - All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (two streams, two
 *     threads) race.  Calls on one stream are ordered and safe.  Old contents never reach a result.
 *   - The first call on each device resolves the array's address (hipGetSymbolAddress, once per device, the
 *     device being current); make that call outside graph capture.  SANA_ERR_RUNTIME if the lookup fails.
 */
#define SANA_HIP_NOALLOC_SCRATCH_BYTES (32u << 20)

int sana_hip_linattn_state_noalloc(const void* k, const void* v, float* state,
                                   int B, int N, int h, int d,
                                   int64_t stride_b, int64_t stride_n,
                                   const int32_t* chunk_starts, int n_chunks, int max_chunk_tokens,
                                   int causal, int io_dtype,
                                   const float* k_rinv, const void* k_weight, const float* rope,
                                   void* stream);

/* ---------------------------------------------------------------------------
 * Depthwise 3x3 conv (zero pad 1, stride 1) + bias + SiLU gate, channels-last
 *
 *   t[c]  = bias[c] + sum_{dy,dx} u[y+dy][x+dx][c] * w[c][dy+1][dx+1],  c in 0..2*Ch-1
 *   y[c]  = t[c] * silu(t[Ch + c]),                                     c in 0..Ch-1
 *
 * Replaces depth_conv, torch.chunk, glu_act and the multiply of
 * GLUMBConv._apply_spatial (diffusion/model/nets/basic_modules.py:164-167).
 *
 *   u     [BT][H][W][2*Ch] contiguous (the inverted conv's output, channels-last)
 *   w     [2*Ch][3][3] (= depth_conv.conv.weight [2Ch,1,3,3]), io dtype
 *   bias  [2*Ch] io dtype, or NULL
 *   y     [BT][H][W][Ch] contiguous
 *   round_like_reference != 0 rounds t, silu(t_g) and the product to the io
 *   dtype one after the other, as the reference's three separate torch ops do;
 *   0 keeps fp32 until the single final rounding.
 */
int sana_hip_dwconv3x3_silu_gate(const void* u, const void* w, const void* bias, void* y,
                                 int BT, int H, int W, int Ch,
                                 int round_like_reference, int io_dtype, void* stream);

/* ---------------------------------------------------------------------------
 * GEMM  C[M][N] = epilogue(A[M][K] . W[N][K]^T), bf16 in, fp32 accumulate, bf16 out
 *
 * Replaces nn.Linear qkv / proj (sana_blocks.py:270,289) and the 1x1 convs
 * inverted_conv (+ bias + SiLU) / point_conv (basic_modules.py:163,167).
 *
 *   A     [M][K] row-major with row stride lda
 *   W     [N][K] row-major with row stride ldw  (nn.Linear / 1x1-conv weight layout)
 *   bias  [N] bf16 or NULL (must be non-NULL for SANA_EPI_BIAS*)
 *   C     [M][N] row-major with row stride ldc
 * K and N must be multiples of 8 (16-byte rows); lda, ldw, ldc multiples of 8.
 *
 * workspace (optional): a shape with too few output tiles to occupy the chip (few tokens, narrow N, long
 * K: the proj and point-conv GEMMs of a single 1024 px image) runs faster as a split-k GEMM -- K cut into
 * up to 8 ranges whose fp32 partial results go through the workspace and are summed in a fixed order by a
 * second kernel that applies the epilogue.  sana_hip_gemm_workspace_bytes(M, N, K) is the size that
 * needs (0: this shape is never split).  With workspace NULL, misaligned or smaller than that, the GEMM
 * runs unsplit -- same result up to the fp32 summation order.  The plan depends on (M, N, K) only, so the
 * int8-weight GEMM and the gated-residual GEMM split the same way and stay bit-identical to this one.
 */
size_t sana_hip_gemm_workspace_bytes(int M, int N, int K);

int sana_hip_gemm_bf16(const void* A, const void* W, const void* bias, void* C,
                       int M, int N, int K, int64_t lda, int64_t ldw, int64_t ldc,
                       int epilogue, void* workspace, size_t workspace_bytes, void* stream);

/* The same GEMM for an fp16 model (the released Sana-600M configuration trains and samples in fp16,
 * configs/sana_config/1024ms/Sana_600M_img1024.yaml:22): A, W, bias and C are IEEE half, accumulation is fp32 on
 * v_mfma_f32_16x16x32_f16, the epilogues round to half where the bf16 form rounds to bf16.  Same arguments,
 * tile plans and split-k behaviour as sana_hip_gemm_bf16; replaces the same nn.Linear / 1x1-conv calls. */
int sana_hip_gemm_f16(const void* A, const void* W, const void* bias, void* C,
                      int M, int N, int K, int64_t lda, int64_t ldw, int64_t ldc,
                      int epilogue, void* workspace, size_t workspace_bytes, void* stream);

/* W8A16: W is int8 [N][K] with a per-output-channel fp32 scale [N].  Each
 * weight is dequantised in registers as bf16_rne(float(q) * scale[n]) — the same
 * value as torch's (q.float() * scale).bfloat16() — before the MFMA, so the
 * result equals sana_hip_gemm_bf16 on the dequantised weight.  No reference
 * counterpart (the reference has no W8A16 code); the quantiser is defined by the
 * benchmark configuration.  K and ldw must be multiples of 16. */
int sana_hip_gemm_w8a16(const void* A, const int8_t* Wq, const float* scale, const void* bias,
                        void* C, int M, int N, int K, int64_t lda, int64_t ldw, int64_t ldc,
                        int epilogue, void* workspace, size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------
 * Fused seams around the two modules (the reference runs them as separate
 * elementwise torch ops inside SanaMSBlock.forward,
 * diffusion/model/nets/sana_multi_scale.py:148-155, sana_blocks.py:44-45).
 *
 * GEMM + gated residual:  C = residual + gate[row / rows_per_gate] * (A W^T + bias)
 *   replaces `x + gate_msa * attn(...)` / `x + gate_mlp * mlp(...)` (:151-155)
 *   together with the module's last linear (proj / point_conv).  bf16 only.
 *   W is bf16 [N][K] when w8_scale is NULL, else int8 [N][K] with fp32 scales.
 *   gate: bf16 rows of N values, gate_stride elements apart, one row per
 *   rows_per_gate consecutive rows of C (= tokens per batch element);
 *   residual: bf16 [M][N] with row stride ldr (may alias C).  bias may be NULL.
 *   The linear output, the gate product and the sum are each rounded to bf16,
 *   as the reference's three ops do.  workspace: as for sana_hip_gemm_bf16
 *   (optional split-k).
 */
int sana_hip_gemm_gate_residual(const void* A, const void* W, const float* w8_scale, const void* bias,
                                const void* gate, const void* residual, void* C,
                                int M, int N, int K, int64_t lda, int64_t ldw, int64_t ldr, int64_t ldc,
                                int rows_per_gate, int64_t gate_stride,
                                void* workspace, size_t workspace_bytes, void* stream);

/* sana_hip_gemm_gate_residual for an fp16 model: every operand IEEE half (no int8 weights), the three roundings to
 * half.  Replaces the same lines of SanaMSBlock.forward (sana_multi_scale.py:151-155). */
int sana_hip_gemm_gate_residual_f16(const void* A, const void* W, const void* bias,
                                    const void* gate, const void* residual, void* C,
                                    int M, int N, int K, int64_t lda, int64_t ldw, int64_t ldr, int64_t ldc,
                                    int rows_per_gate, int64_t gate_stride,
                                    void* workspace, size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------
 * qkv projection + phase 1 of the linear attention in one GEMM (bf16, head_dim 32, no q/k transform):
 *   Q = A Wq^T (+ bias)            stored, bf16 [B*N][C] with row stride ldq
 *   state[b][h] = [V_h | 1]^T relu(K_h)  over the N tokens of batch entry b, fp32 [B*heads][33][32]
 * replaces `qkv = self.qkv(x)` together with the `vk = v @ k^T` half of LiteLA.forward
 * (diffusion/model/nets/sana_blocks.py:270-296, :245-263): k and v are never written -- the column tiles that
 * produce them are contracted over their tokens in the GEMM's epilogue (k and v rounded to bf16 first, products in
 * fp32, exactly the values sana_hip_linattn_state reads back from memory; the sums differ from its sums by fp32
 * summation order only).  sana_hip_linattn_apply then takes Q and the state.
 *   The weight comes in the layout sana_hip_qkv_state_rows describes: rows[i] is the row of the reference's
 *   [3C][C] qkv weight (and entry of its bias) that row i of W_tiled holds, or -1 for a zero row.  With rows ==
 *   NULL the function returns the number of rows; with a buffer of that capacity it fills it (host code, no GPU).
 *   A: bf16 [B*N][C] (row stride lda); W_tiled: bf16 [rows][C] (row stride ldw); bias_tiled: bf16 [rows] or NULL.
 *   C == 32 * heads; N % 256 == 0, or B == 1 and no bias (a ragged last tile's missing rows are then zeros that add
 *   nothing to the state).  workspace: sana_hip_gemm_qkv_state_workspace_bytes(B, N, heads) bytes (one
 *   partial state per 256 tokens, added in token order by a second launch: deterministic, no atomics). */
int sana_hip_qkv_state_rows(int C, int heads, int32_t* rows, int capacity);
size_t sana_hip_gemm_qkv_state_workspace_bytes(int B, int N, int heads);
int sana_hip_gemm_qkv_state(const void* A, const void* W_tiled, const void* bias_tiled, void* Q, float* state,
                            void* workspace, size_t workspace_bytes, int B, int N, int C, int heads,
                            int64_t lda, int64_t ldw, int64_t ldq, void* stream);

/* LayerNorm without affine (eps inside the rsqrt) + adaLN modulation:
 *   out[m][:] = LN(x[m][:]) * (1 + scale[m / rows_per_mod][:]) + shift[m / rows_per_mod][:]
 *   replaces `t2i_modulate(self.norm1(x), shift, scale)` (sana_multi_scale.py:152,155).
 *   x, out: [M][C] with row strides ldx / ldo; scale, shift: rows of C values, mod_stride elements
 *   apart; all of io_dtype, SANA_DT_BF16 or SANA_DT_F16 (the four roundings of the stock op chain are to
 *   that dtype).  C % 8 == 0, C <= 8192. */
int sana_hip_layernorm_modulate(const void* x, const void* scale, const void* shift, void* out,
                                int64_t M, int C, int64_t ldx, int64_t ldo,
                                int rows_per_mod, int64_t mod_stride, float eps, int io_dtype, void* stream);

/* The same with the residual update in front of the norm in the same pass:
 *   sum[m][:] = x[m][:] + y[m][:]   (rounded to bf16, as the stock add stores it)
 *   out[m][:] = LN(sum[m][:]) * (1 + scale[..]) + shift[..]
 * replaces `x = x + self.cross_attn(x, y, mask)` followed by `t2i_modulate(self.norm2(x), shift_mlp,
 * scale_mlp)` (sana_multi_scale.py:154-155).  y, sum: bf16 [M][C] with row strides ldy / lds; sum may alias x. */
int sana_hip_add_layernorm_modulate(const void* x, const void* y, const void* scale, const void* shift,
                                    void* sum, void* out, int64_t M, int C,
                                    int64_t ldx, int64_t ldy, int64_t lds, int64_t ldo,
                                    int rows_per_mod, int64_t mod_stride, float eps, int io_dtype, void* stream);

/* ---------------------------------------------------------------------------
 * int8 weight -> bf16: W[n][k] = bf16((float)Wq[n][k] * scale[n]), one rounding -- bit for bit the value
 * the int8 path of the GEMM feeds its MFMAs (and torch's `(Wq.float() * scale[:, None]).bfloat16()`).
 * No counterpart in the reference (W8A16 is defined by the benchmark configuration).  For GEMMs with many
 * rows (M of a few thousand and more) expanding the weight once per call and running the bf16 GEMM is
 * faster than converting inside the GEMM's main loop; the results are identical.
 *   Wq int8 [N][K] (row stride ldw, K % 16 == 0), scale fp32 [N], W bf16 [N][K] (row stride ldo)
 */
int sana_hip_dequant_w8(const int8_t* Wq, const float* scale, void* W, int N, int K,
                        int64_t ldw, int64_t ldo, void* stream);

/* Softmax attention of many queries over a short key set, bf16: the core of the block's cross-attention to the
 * text tokens (diffusion/model/nets/sana_blocks.py:69-98: F.scaled_dot_product_attention(q, k, v, attn_mask) at
 * :92, scale = head_dim ** -0.5, and the additive mask (1 - mask) * -10000 of :89-90).
 *   q:   bf16 [B][N][H*d] with row stride ldq (the q_linear output as it is: no head transpose);
 *   kv:  bf16 [B][Nk][2][H*d] with row stride ldkv >= 2*H*d (the kv_linear output: keys, then values);
 *   key_bias: fp32 [B] rows of Nk values bias_stride apart, added to the scaled scores of every head and query
 *        (0 / -10000 for the reference's padding mask), or NULL;
 *   out: bf16 [B][N][H*d] with row stride ldo (what proj reads).
 * Probabilities are rounded to bf16 before they multiply v, as fused attention kernels do; sums in fp32.
 * Nk <= 320, 64 < d <= 112, d % 8 == 0 (Sana: 2240 / 20 = 112, 1152 / 16 = 72); SANA_ERR_SHAPE otherwise. */
int sana_hip_cross_attention(const void* q, const void* kv, const float* key_bias, void* out, int B, int N,
                             int Nk, int H, int d, int64_t ldq, int64_t ldkv, int64_t ldo,
                             int64_t bias_stride, float scale, void* stream);

/* Gated residual update as one elementwise pass:
 *   out[m][:] = residual[m][:] + gate[m / rows_per_gate][:] * y[m][:]
 * with the product and the sum each rounded to bf16, as the reference's two ops do.  Replaces
 * `x + self.drop_path(gate_mlp * mlp_out)` (diffusion/model/nets/sana_multi_scale_video.py:321; per frame
 * :247-252) where the module's last op is not a GEMM of this library (the temporal Mix-FFN variants), and
 * `x + gate_msa * attn(...)` when a guidance processor or hook needs the attention output itself.
 *   y, residual, out: [M][C] with row strides ldy / ldr / ldo (out may alias residual or y);
 *   gate: rows of C values, gate_stride elements apart; all of io_dtype, SANA_DT_BF16 or SANA_DT_F16.
 *   C % 8 == 0. */
int sana_hip_gate_residual(const void* y, const void* gate, const void* residual, void* out,
                           int64_t M, int C, int64_t ldy, int64_t ldr, int64_t ldo,
                           int rows_per_gate, int64_t gate_stride, int io_dtype, void* stream);

/* ---------------------------------------------------------------------------
 * Temporal (t, 1) convolution over frames with full channel mixing, plus its residual, as ONE GEMM over a
 * virtual im2col of the token-major buffer (no copy of the activations):
 *
 *   out[m][:] = X[m + (taps/2)*tap_rows][:] + sum_{t < taps} W[:, t*C:(t+1)*C] . X[m + t*tap_rows][:]
 *
 * for m < M, where rows of X at or past x_rows read as zero.  With tap_rows = tokens per frame this is
 * `x + t_conv(x)` of GLUMBConvTemp.forward (diffusion/model/nets/basic_modules.py:250-264,
 * t_conv = Conv2d(C, C, (3, 1), padding (1, 0), bias=False)) on the frames of one batch entry: X points
 * at the frame in FRONT of the first output frame (zeros at the start of a sequence, the previous
 * chunk's last frame for ChunkGLUMBConvTemp / CachedGLUMBConvTemp, :302-349 / :374-392), and x_rows =
 * M + tap_rows ends the buffer behind the last output frame, which gives the zero padding on the right.
 * Roundings as the reference's: the convolution result to bf16, then the sum to bf16.
 *
 *   X     bf16 rows of C channels, row stride ldx; x_rows >= M + (taps/2)*tap_rows rows exist
 *   W     bf16 [C][taps*C], row stride ldw: W[o][t*C + i] = t_conv.weight[o][i][t][0]
 *   out   bf16 [M][C], row stride ldo (must not overlap X)
 *   taps  odd; C % 64 == 0; x_rows * ldx * 2 < 2^31
 *   zero_last_tap  NULL, or one byte per block of tap_rows output rows (per frame): non-zero = the last tap of
 *         these rows reads zeros instead of the rows behind them.  That is the zero padding ChunkGLUMBConvTemp
 *         puts behind every chunk (:302-349: a chunk sees the previous chunk's last frame in front and zeros
 *         behind), so all chunks of a sequence run as one launch.  taps >= 3 when given.
 */
int sana_hip_tconv_residual(const void* X, const void* W, void* out, int M, int C, int taps,
                            int64_t tap_rows, int64_t x_rows, const unsigned char* zero_last_tap,
                            int64_t ldx, int64_t ldw, int64_t ldo, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SANA_HIP_H_ */
