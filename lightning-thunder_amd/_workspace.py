"""Device scratch that the split-K kernels meet in: arrival counters (zero between calls) and partial
sums.  One buffer per (device, stream), because two calls that may overlap in time need different
buffers and calls on one stream never overlap.

Lifetime rules, chosen for callers that capture HIP graphs:

* A buffer that was handed out is never freed: a captured graph keeps the raw address, so an outgrown
  buffer is retired (kept alive), not released.
* Nothing is allocated while the stream is capturing.  ``torch.zeros`` there would record a memset node
  (unreliable in replayed graphs on this target) and tie the buffer to the capture's private pool; the
  call raises instead and tells the caller to warm up or to :meth:`reserve` first.
* Buffers start at ``floor_bytes``, large enough for every Llama-3-8B / 70B projection shape, so growth is
  the exception.

torch hands out streams from a fixed pool per device, which bounds the number of buffers.
"""

from __future__ import annotations

import torch

_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def current_stream_handle(device_index: int) -> int:
    if _raw_stream is not None:
        return _raw_stream(device_index)
    return torch.cuda.current_stream(device_index).cuda_stream


class WorkspacePool:
    def __init__(self, floor_bytes: int, what: str):
        self.floor_bytes = int(floor_bytes)
        self.what = what
        self._live: dict[tuple[int, int], torch.Tensor] = {}
        self._retired: list[torch.Tensor] = []

    def _key(self, device: torch.device, stream: int | None) -> tuple[int, int]:
        idx = device.index
        if idx is None:
            idx = torch.cuda.current_device() if device.type == "cuda" else -1
        return idx, current_stream_handle(idx) if stream is None else stream

    def get(self, device: torch.device, nbytes: int, stream: int | None = None) -> torch.Tensor:
        """The zero-initialised buffer of (device, stream), at least ``nbytes`` long."""
        key = self._key(device, stream)
        ws = self._live.get(key)
        if ws is not None and ws.numel() >= nbytes:
            return ws
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError(
                f"{self.what}: a {nbytes}-byte workspace would have to be allocated while the stream is capturing "
                f"(the stream has {'none' if ws is None else f'one of {ws.numel()} bytes'}). Run the call once on this "
                "stream before the capture, or call reserve_workspace() first."
            )
        new = torch.zeros(max(int(nbytes), self.floor_bytes), dtype=torch.uint8, device=device)
        if ws is not None:
            self._retired.append(ws)  # graphs captured earlier may still write here
        self._live[key] = new
        return new

    def reserve(self, device: torch.device, nbytes: int | None = None, stream: int | None = None) -> int:
        """Make sure (device, stream) owns a buffer of ``nbytes`` (default: the floor) before a capture."""
        return self.get(device, self.floor_bytes if nbytes is None else nbytes, stream).numel()

    def stats(self) -> dict:
        return {"live": len(self._live), "retired": len(self._retired),
                "bytes": sum(t.numel() for t in self._live.values()) + sum(t.numel() for t in self._retired)}
