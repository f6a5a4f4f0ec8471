"""HIP-graph replay of the forward pass (cf. thunder/transforms/cudagraph.py:47-387).

Decode with 225 quantised linears per token is launch-bound from Python; capturing one forward pass
into a HIP graph removes the host from the loop.  The weights, absmax and code tensors are static
inputs by construction (the reference tags them STATIC_MEMORY_LOCATION for the same reason,
thunder/transforms/quantization.py:178,186); the call arguments are copied into static buffers.
"""

from __future__ import annotations

import torch

from .transform_common import Transform


class HIPGraphRunner:
    """Capture ``fn(*tensors)`` once per input signature; afterwards copy inputs in and replay."""

    def __init__(self, fn, warmup: int = 2):
        self.fn = fn
        self.warmup = warmup
        self.cache: dict = {}

    @staticmethod
    def _key(args):
        return tuple((tuple(a.shape), a.dtype, a.device) if isinstance(a, torch.Tensor) else ("const", a) for a in args)

    def __call__(self, *args):
        key = self._key(args)
        entry = self.cache.get(key)
        if entry is None:
            static_in = [a.clone() if isinstance(a, torch.Tensor) else a for a in args]
            # warm-up and capture run on ONE side stream: per-stream state (the gemv workspace of
            # that stream, library handles) exists before the capture and is the one the graph uses
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(self.warmup):  # allocations, lazy library state, workspaces
                    self.fn(*static_in)
                torch.cuda.synchronize()
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=side):
                    static_out = self.fn(*static_in)
            torch.cuda.current_stream().wait_stream(side)
            entry = (graph, static_in, static_out)
            self.cache[key] = entry
        graph, static_in, static_out = entry
        for s, a in zip(static_in, args):
            if isinstance(a, torch.Tensor):
                s.copy_(a)
        graph.replay()
        return static_out


class HIPGraphTransform(Transform):
    """Marks a jitted module for graph replay: ``jit`` consults ``wrap_callable``."""

    def wrap_callable(self, fn):
        return HIPGraphRunner(fn)
