"""Writes ``tests/golden/kat.npz``: known-answer vectors for the linear-attention (plain, chunk-causal, rotary) and
depthwise-gate kernels and for the qkv projection with the attention state in its epilogue, computed in fp64 by the plain-C
quadratic-form / 9-tap restatement (``oracle/bruteforce.c``).

The reference holds no numeric fixtures for this path, so these vectors are the build's own: they
freeze the brute-force answers on seeded inputs (all exactly representable in bf16), and both the
stock-PyTorch oracle (CPU test) and the HIP kernels (GPU test) are checked against the frozen file.

    python tests/golden/make_vectors.py
"""
import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", ".."))
from oracle import cbrute  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kat.npz")


def bf16_values(gen, *shape, scale=1.0):
    """N(0, scale) rounded to bf16, returned as float64 (exact)."""
    return (torch.randn(*shape, generator=gen) * scale).bfloat16().double().numpy()


def main():
    g = torch.Generator().manual_seed(20240229)
    vec = {}
    # ReLU linear attention, head_dim 32 and 112: q, k, v [BH, N, d] token-major
    for tag, BH, N, d in (("la32", 2, 40, 32), ("la112", 1, 24, 112)):
        q, k, v = (bf16_values(g, BH, N, d) for _ in range(3))
        vec[f"{tag}_q"], vec[f"{tag}_k"], vec[f"{tag}_v"] = q, k, v
        vec[f"{tag}_out"] = cbrute.relu_attention(q, k, v, 1e-8)
        vec[f"{tag}_state"] = cbrute.attention_state(k, v)
    # chunk-causal: token n sees the tokens of its own and of earlier chunks
    BH, N, d = 2, 36, 32
    q, k, v = (bf16_values(g, BH, N, d) for _ in range(3))
    chunk_of = np.repeat(np.arange(3, dtype=np.int32), 12)
    vec.update(cc_q=q, cc_k=k, cc_v=v, cc_chunk_of=chunk_of, cc_out=cbrute.relu_attention(q, k, v, 1e-8, chunk_of))
    # depthwise 3x3 (zero padding) + bias on 2C channels, then first half * silu(second half)
    BT, H, W, C = 2, 5, 6, 8
    u = bf16_values(g, BT, H, W, 2 * C)
    w = bf16_values(g, 2 * C, 3, 3, scale=0.3)
    b = bf16_values(g, 2 * C, scale=0.1)
    vec.update(dw_u=u, dw_w=w, dw_b=b, dw_out=cbrute.dwconv_gate(u, w, b))
    # rotary family: per-token complex factors on the channel pairs of relu(q), relu(k) in the NUMERATOR only
    # (unit modulus, generic angles, stored as fp32-exact cos / sin so every consumer rotates by the same numbers),
    # three chunks of 12 tokens for the chunk-causal form
    for tag, BH, N, d in (("rope32", 2, 36, 32), ("rope112", 1, 36, 112)):
        q, k, v = (bf16_values(g, BH, N, d) for _ in range(3))
        theta = (torch.rand(N, d // 2, generator=g, dtype=torch.float64) - 0.5) * 6.0
        cos, sin = torch.cos(theta).float().double().numpy(), torch.sin(theta).float().double().numpy()
        freqs = cos + 1j * sin
        chunk_of = np.repeat(np.arange(3, dtype=np.int32), 12)
        vec.update({f"{tag}_q": q, f"{tag}_k": k, f"{tag}_v": v, f"{tag}_cos": cos, f"{tag}_sin": sin,
                    f"{tag}_chunk_of": chunk_of,
                    f"{tag}_out": cbrute.relu_attention_rope(q, k, v, freqs, 1e-8),
                    f"{tag}_cc_out": cbrute.relu_attention_rope(q, k, v, freqs, 1e-8, chunk_of)})
    # qkv projection + attention state on small integers: every product, sum and rounding on the way is exact in
    # bf16 / fp32 (|q|, |k|, |v| <= 128, state entries < 2^23), so the answer is THE answer, bit for bit.
    # x [1, 512, 64], w [192, 64] (nn.Linear layout: q rows, k rows, v rows; two heads of 32)
    x = torch.randint(-2, 3, (1, 512, 64), generator=g).double().numpy()
    w = torch.randint(-1, 2, (192, 64), generator=g).double().numpy()
    qkv = x @ w.T                                                     # [1, 512, 192]
    heads = lambda t: np.ascontiguousarray(t.reshape(512, 2, 32).transpose(1, 0, 2))   # [BH = 2, N, d]
    vec.update(qkvs_x=x, qkvs_w=w, qkvs_q=qkv[..., :64],
               qkvs_state=cbrute.attention_state(heads(qkv[0, :, 64:128]), heads(qkv[0, :, 128:])))
    np.savez_compressed(OUT, **vec)
    print(f"wrote {OUT}: {os.path.getsize(OUT)} bytes, {len(vec)} arrays")


if __name__ == "__main__":
    main()
