"""HIP-graph replay of the image encoder for launch-bound shapes.

At small batch (ViT-B, one image) a forward is ~110 kernel launches of a few microseconds
each and the host cannot issue them fast enough.  `GraphedEncoder` records one forward of an
encoder at a fixed input shape into a HIP graph (torch.cuda.CUDAGraph) and replays it: every
launch of the hot path - the C-ABI calls enqueue on the current stream, which is the capturing
stream during the recording - becomes a graph node.  The library itself never allocates and
records no memset nodes; the tensors the Python layer creates come from the graph's private pool.

Nothing in the reference corresponds to this (it relies on torch.compile's CUDA graphs,
build_sam.py:95-141 `mode='max-autotune'`); it is the same idea without a tracing compiler.
"""

from typing import Optional

import torch
import torch.nn as nn


class GraphedEncoder(nn.Module):
    """Wraps `encoder` (ImageEncoderViT or any module with a static forward) for inputs of one
    fixed shape / dtype.  `forward(x)` copies x into the recorded input buffer, replays the
    graph and returns the recorded output buffer (valid until the next call)."""

    def __init__(self, encoder: nn.Module, example: torch.Tensor, warmup: int = 3) -> None:
        super().__init__()
        if not example.is_cuda:
            raise RuntimeError("samfast: GraphedEncoder needs a GPU example input")
        self.encoder = encoder
        self._in = example.clone()
        self._out: Optional[torch.Tensor] = None
        self._graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()  # default priority
        side.wait_stream(torch.cuda.current_stream())
        with torch.no_grad(), torch.cuda.stream(side):
            for _ in range(warmup):  # lazy initialisation (MIOpen search, weight re-layouts) happens here
                self.encoder(self._in)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        with torch.no_grad(), torch.cuda.graph(self._graph):
            self._out = self.encoder(self._in)

    @torch.no_grad()
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if x.shape != self._in.shape or x.dtype != self._in.dtype:
            raise RuntimeError(f"samfast: GraphedEncoder was recorded for {tuple(self._in.shape)} "
                               f"{self._in.dtype}, got {tuple(x.shape)} {x.dtype}")
        self._in.copy_(x)
        self._graph.replay()
        return self._out
