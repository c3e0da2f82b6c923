/* Plain-C, double-precision brute-force restatement of the two arithmetic
 * cores of the SanaMSBlock hot path.  TEST INFRASTRUCTURE ONLY: it exists to
 * pin oracle/sana_oracle.py (a different language, a different formula) and
 * is never linked into or called from the product.
 *
 * The linear attention is written in its QUADRATIC form, which the reference
 * itself states to be equivalent to the linear form
 * (diffusion/model/dc_ae/efficientvit/models/nn/ops.py:796-823 vs :738-793):
 *
 *   out[i, n] = sum_m v[i, m] * <relu k_m, relu q_n>
 *               / (sum_m <relu k_m, relu q_n> + eps)
 *
 * which is what LiteLA.attn_matmul computes through the d x (d+1) state
 * (diffusion/model/nets/sana_blocks.py:245-263).  The chunk-causal variant
 * restricts m to chunk(m) <= chunk(n) (sana_blocks.py:481-489, rotary = 1).
 *
 * The rotary family (LiteLAReLURope / ChunkCausalAttention / CachedCausalAttention,
 * sana_blocks.py:359-383, 481-489, 544-562) multiplies the channel pairs
 * (2p, 2p+1) of relu(q_n), relu(k_n), read as complex numbers, by a per-token
 * factor f[n][p] -- but only in the numerator; the denominator keeps the
 * unrotated vectors (`z` from `k`, `q` at :378; `vk`, `out` from `k_rotated`,
 * `q_rotated` at :380-381):
 *
 *   out[i, n] = sum_m v[i, m] * <rot_m(relu k_m), rot_n(relu q_n)>
 *               / (sum_m <relu k_m, relu q_n> + eps)
 *
 * The depthwise conv + gate follows GLUMBConv._apply_spatial
 * (diffusion/model/nets/basic_modules.py:161-167): 3x3, zero padding 1,
 * stride 1, one filter per channel, then a = first half, g = second half,
 * y = a * silu(g).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>

static double relu(double x) { return x > 0.0 ? x : 0.0; }

/* q, k, v: [BH][N][d] token-major doubles.  chunk_of: [N] int32 or NULL
 * (NULL = every token sees every token).  out: [BH][N][d]. */
void brute_relu_attention(const double* q, const double* k, const double* v,
                          const int32_t* chunk_of, double eps,
                          int BH, int N, int d, double* out) {
  for (int bh = 0; bh < BH; ++bh) {
    const double* Q = q + (size_t)bh * N * d;
    const double* K = k + (size_t)bh * N * d;
    const double* V = v + (size_t)bh * N * d;
    double* O = out + (size_t)bh * N * d;
    for (int n = 0; n < N; ++n) {
      double den = 0.0;
      for (int i = 0; i < d; ++i) O[(size_t)n * d + i] = 0.0;
      for (int m = 0; m < N; ++m) {
        if (chunk_of && chunk_of[m] > chunk_of[n]) continue;
        double s = 0.0;
        for (int j = 0; j < d; ++j) s += relu(K[(size_t)m * d + j]) * relu(Q[(size_t)n * d + j]);
        den += s;
        for (int i = 0; i < d; ++i) O[(size_t)n * d + i] += V[(size_t)m * d + i] * s;
      }
      for (int i = 0; i < d; ++i) O[(size_t)n * d + i] /= (den + eps);
    }
  }
}

/* The rotary family in quadratic form.  q, k, v, out, chunk_of as above;
 * f_re, f_im: [N][d/2] real and imaginary part of the per-token factors (any
 * complex number, not only unit ones), shared by all BH.  <.,.> is the plain
 * real dot product over the d channels of the rotated vectors. */
static void rotate_token(const double* x, const double* f_re, const double* f_im, int d, double* y) {
  for (int p = 0; p < d / 2; ++p) {
    const double a = relu(x[2 * p]), b = relu(x[2 * p + 1]);
    y[2 * p] = a * f_re[p] - b * f_im[p];
    y[2 * p + 1] = a * f_im[p] + b * f_re[p];
  }
}

void brute_relu_attention_rope(const double* q, const double* k, const double* v,
                               const double* f_re, const double* f_im,
                               const int32_t* chunk_of, double eps,
                               int BH, int N, int d, double* out) {
  double qr[512], kr[512];
  if (d > 512 || (d & 1)) return;
  for (int bh = 0; bh < BH; ++bh) {
    const double* Q = q + (size_t)bh * N * d;
    const double* K = k + (size_t)bh * N * d;
    const double* V = v + (size_t)bh * N * d;
    double* O = out + (size_t)bh * N * d;
    for (int n = 0; n < N; ++n) {
      double den = 0.0;
      rotate_token(Q + (size_t)n * d, f_re + (size_t)n * (d / 2), f_im + (size_t)n * (d / 2), d, qr);
      for (int i = 0; i < d; ++i) O[(size_t)n * d + i] = 0.0;
      for (int m = 0; m < N; ++m) {
        if (chunk_of && chunk_of[m] > chunk_of[n]) continue;
        rotate_token(K + (size_t)m * d, f_re + (size_t)m * (d / 2), f_im + (size_t)m * (d / 2), d, kr);
        double s_plain = 0.0, s_rot = 0.0;
        for (int j = 0; j < d; ++j) {
          s_plain += relu(K[(size_t)m * d + j]) * relu(Q[(size_t)n * d + j]);
          s_rot += kr[j] * qr[j];
        }
        den += s_plain;
        for (int i = 0; i < d; ++i) O[(size_t)n * d + i] += V[(size_t)m * d + i] * s_rot;
      }
      for (int i = 0; i < d; ++i) O[(size_t)n * d + i] /= (den + eps);
    }
  }
}

/* state[bh][i][j] = sum_n vpad[n][i] * relu(k[n][j]), i in 0..d (row d: ones). */
void brute_attention_state(const double* k, const double* v, int BH, int N, int d, double* state) {
  for (int bh = 0; bh < BH; ++bh) {
    const double* K = k + (size_t)bh * N * d;
    const double* V = v + (size_t)bh * N * d;
    double* S = state + (size_t)bh * (d + 1) * d;
    for (int i = 0; i <= d; ++i)
      for (int j = 0; j < d; ++j) {
        double s = 0.0;
        for (int n = 0; n < N; ++n) s += (i < d ? V[(size_t)n * d + i] : 1.0) * relu(K[(size_t)n * d + j]);
        S[(size_t)i * d + j] = s;
      }
  }
}

/* u: [BT][H][W][2C] channels-last doubles; w: [2C][3][3]; b: [2C];
 * y: [BT][H][W][C] = (dw(u)[c] + b[c]) * silu(dw(u)[C+c] + b[C+c]). */
void brute_dwconv_gate(const double* u, const double* w, const double* b,
                       int BT, int H, int W, int C, double* y) {
  const int C2 = 2 * C;
  for (int n = 0; n < BT; ++n)
    for (int yy = 0; yy < H; ++yy)
      for (int xx = 0; xx < W; ++xx)
        for (int c = 0; c < C; ++c) {
          double acc[2];
          for (int half = 0; half < 2; ++half) {
            const int ch = c + half * C;
            double s = b[ch];
            for (int dy = -1; dy <= 1; ++dy)
              for (int dx = -1; dx <= 1; ++dx) {
                const int iy = yy + dy, ix = xx + dx;
                if (iy < 0 || iy >= H || ix < 0 || ix >= W) continue;
                s += u[(((size_t)n * H + iy) * W + ix) * C2 + ch] * w[(size_t)ch * 9 + (dy + 1) * 3 + (dx + 1)];
              }
            acc[half] = s;
          }
          const double g = acc[1];
          y[(((size_t)n * H + yy) * W + xx) * C + c] = acc[0] * (g / (1.0 + exp(-g)));
        }
}
