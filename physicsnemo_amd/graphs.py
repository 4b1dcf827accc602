"""HIP-graph replay of a forward pass.

One PhysicsAttention layer is five dependent kernel launches, a Transolver block about a dozen; on small meshes the
gaps between them are a visible share of the time.  `GraphedForward` records the launches of one call into a HIP
graph (through torch.cuda.CUDAGraph, which captures everything enqueued on the stream, the library's kernels
included) and replays it: same kernels, same arithmetic, one submission.

The library records nothing but kernel launches (no memset nodes), every buffer it uses is allocated by torch inside
the capture and therefore owned by the graph's memory pool, and shapes are fixed at capture time.
"""
from __future__ import annotations

import torch

__all__ = ["GraphedForward"]


class GraphedForward:
    """Capture `fn(*example_inputs)` once, then replay it on new inputs of the same shapes and dtypes.

    `fn` is called under `torch.no_grad()`; wrap it yourself if it needs an autocast context.  The returned tensors
    are the graph's static outputs: they are overwritten by the next call, so copy what must outlive it.
    """

    def __init__(self, fn, *example_inputs: torch.Tensor, warmup: int = 2):
        if not example_inputs or not all(t.is_cuda for t in example_inputs):
            raise RuntimeError("GraphedForward needs GPU tensors as example inputs")
        self._fn = fn
        self._static_in = [t.detach().clone() for t in example_inputs]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.no_grad(), torch.cuda.stream(side):
            for _ in range(max(1, warmup)):  # parameter caches, lazy initialisation: nothing of it may be captured
                fn(*self._static_in)
        torch.cuda.current_stream().wait_stream(side)
        self._graph = torch.cuda.CUDAGraph()
        with torch.no_grad(), torch.cuda.graph(self._graph):
            self._static_out = fn(*self._static_in)

    @property
    def inputs(self):
        """The graph's static input tensors: fill them in place and call `replay()` to avoid the copy of `__call__`."""
        return self._static_in

    def replay(self):
        self._graph.replay()
        return self._static_out

    def __call__(self, *inputs: torch.Tensor):
        if len(inputs) != len(self._static_in):
            raise ValueError(f"expected {len(self._static_in)} inputs, got {len(inputs)}")
        for dst, src in zip(self._static_in, inputs):
            if dst.shape != src.shape or dst.dtype != src.dtype:
                raise ValueError(f"captured for {tuple(dst.shape)} {dst.dtype}, got {tuple(src.shape)} {src.dtype}")
            if dst.data_ptr() != src.data_ptr():
                dst.copy_(src)
        self._graph.replay()
        return self._static_out
