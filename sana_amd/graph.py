"""Replaying blocks from a HIP graph.

At small shapes (one 1024 px image, the Sana-600M width) a block's ~25 launches take longer to issue from
Python than to run; the library allocates, clears and synchronises nothing, so a block -- or a whole chain of
blocks, one denoising step -- can be captured once and replayed with one launch.  The captured kernels hold raw
addresses: inputs are copied into static buffers before each replay, the scratch buffers the library used stay
alive for the life of the process, and the output tensor is overwritten by the next replay.
"""
from __future__ import annotations

from typing import Callable, Sequence

import torch


class GraphedCall:
    """``fn(*tensors)`` captured into a HIP graph on the tensors' device.

    ``fn`` must be a fixed sequence of device work on its tensor arguments (shapes, dtypes and every non-tensor
    argument baked in), e.g. ``lambda x, y, t: block(x, y, t, HW=(32, 32))``.  The example tensors become the
    captured input buffers: calling the object copies any argument that is another tensor into them (passing the
    example tensors themselves, updated in place, costs no copy), replays, and returns the captured output tensor
    (the same tensor every time: clone it to keep a result across calls)."""

    def __init__(self, fn: Callable[..., torch.Tensor], example: Sequence[torch.Tensor], warmup: int = 2):
        if not example or not all(torch.is_tensor(t) and t.is_cuda for t in example):
            raise ValueError("GraphedCall needs device tensors as example arguments")
        if warmup < 1:
            raise ValueError("GraphedCall needs at least one warm-up call: lazy allocations, host-to-device copies of "
                             "derived tables and the library's scratch buffer must exist before the capture starts")
        self._inputs = list(example)   # the example tensors ARE the captured input buffers
        with torch.no_grad():
            # One stream of this object's own for the warm-up AND the capture.  The library keeps its scratch buffer
            # per (device, stream): warming up on the stream that is captured afterwards creates that buffer eagerly,
            # in the ordinary memory pool, before the capture begins (allocated during the capture it would belong to
            # this graph's private pool while other graphs used it), and a stream per object gives every graph a
            # scratch buffer of its own, so two graphs replayed on different streams do not share one.
            self._stream = torch.cuda.Stream(device=example[0].device)
            self._stream.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(self._stream):
                for _ in range(warmup):
                    fn(*self._inputs)
            torch.cuda.current_stream().wait_stream(self._stream)
            self._graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self._graph, stream=self._stream):
                self._output = fn(*self._inputs)

    def __call__(self, *tensors: torch.Tensor) -> torch.Tensor:
        if len(tensors) != len(self._inputs):
            raise ValueError(f"expected {len(self._inputs)} tensors, got {len(tensors)}")
        for dst, src in zip(self._inputs, tensors):
            if dst.shape != src.shape or dst.dtype != src.dtype:
                raise ValueError(f"captured for {tuple(dst.shape)} {dst.dtype}, got {tuple(src.shape)} {src.dtype}")
            if dst.data_ptr() != src.data_ptr():
                dst.copy_(src)
        self._graph.replay()
        return self._output
