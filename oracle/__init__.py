"""CPU oracle for the SanaMSBlock hot path (LiteLA + GLUMBConv).

TEST INFRASTRUCTURE ONLY.  Nothing in the product package imports this
directory.  Only the test-suite, the smoke check and the benchmark's
``cpu_baseline`` leg use it, and there only as the checker / the CPU figure,
never as the thing measured or shipped.

Contents
--------
``sana_oracle``   stock-PyTorch restatement of the reference modules
                  (LiteLA, GLUMBConv, SanaMSBlock, cross-attention, RMSNorm,
                  the chunk-causal family, the W8A16 quantiser).
``bruteforce.c``  an independent plain-C restatement (double precision,
                  quadratic / per-tap loops) used to pin ``sana_oracle``.
``cbrute``        ctypes loader for the C file.

Parity pins (every function here is pinned by at least one of them; see
``tests/test_oracle_*.py``):
  * quadratic-form brute force (plain C, fp64) for the linear attention and
    its chunk-causal variant,
  * 9-tap zero-padded loop (plain C, fp64) for the depthwise conv + gate,
  * library reductions (fp64 matmul; conv2d 1x1 == linear),
  * algebraic invariants (token permutation, linearity in v, constant v,
    all-negative q, state additivity, zero-gate block identity),
  * committed seeded fixtures under ``tests/golden``.
The timm base class of ``LiteLA`` (``timm==0.6.13``, not vendored in the
reference tree) is *parity unpinned*: its attribute set is inferred from the
reference call sites and the checkpoint converter's key list only.
"""
