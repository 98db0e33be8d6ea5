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

from collections import OrderedDict
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


class ReplayedEncoder(nn.Module):
    """What the fast registry puts in place of `sam.image_encoder`: the stand-in, on this path, for
    `torch.compile(image_encoder, mode=compile_mode)` (segment_anything_fast/build_sam.py:67-71),
    whose `max-autotune` mode means CUDA-graph replay.

    Like the compiler's wrapper it keeps the encoder as the child module `_orig_mod` (state-dict keys
    gain that prefix, as they do in the reference after compilation) and forwards every other
    attribute to it, so `sam.image_encoder.blocks`, `.img_size`, `apply_dynamic_quant(sam.image_encoder)`
    and `SamPredictor.set_torch_image` work unchanged.

    forward(x): a GPU input of at most `max_rows` tokens (64 x 64 per image: four images) is
    launch-bound, so - in eval mode and with autograd off (torch.no_grad / inference_mode, as
    SamPredictor.set_torch_image runs) - the forward is recorded once per input shape into a HIP
    graph (GraphedEncoder) and replayed; larger batches, CPU tensors, calls that record gradients
    and `compile_mode=None` run the encoder eagerly.  The result is a fresh tensor (the graph's output buffer is overwritten by
    the next replay).

    A recorded graph holds the addresses of the weights it read.  Whatever replaces weights or
    modules drops the recordings: `.to()` / `.cuda()` / `.half()`, `load_state_dict`, and the
    swaps this package performs (`apply_dynamic_quant`, `apply_sparse`, `apply_fake_sparsity`,
    `tools.replace_with_custom_fn_if_matches_filter`).  Code that re-assigns submodules or
    parameters by hand calls `invalidate()`."""

    max_rows = 4 * 4096
    max_graphs = 4

    def __init__(self, encoder: nn.Module, compile_mode: Optional[str] = "max-autotune") -> None:
        super().__init__()
        self._orig_mod = encoder
        self.training = encoder.training
        self.compile_mode = compile_mode
        self._graphs = OrderedDict()
        self.register_load_state_dict_post_hook(lambda module, incompatible: module.invalidate())

    def __getattr__(self, name: str):
        try:
            return super().__getattr__(name)
        except AttributeError:
            return getattr(super().__getattr__("_orig_mod"), name)

    def invalidate(self) -> None:
        """Forget every recorded graph (the next forward records again)."""
        self._graphs.clear()

    def _apply(self, fn, *args, **kwargs):
        self.invalidate()  # device / dtype moves create new weight tensors
        return super()._apply(fn, *args, **kwargs)

    def train(self, mode: bool = True):
        self.invalidate()
        return super().train(mode)

    def replays(self, x: torch.Tensor) -> bool:
        """Whether forward(x) goes through a recorded graph."""
        if self.compile_mode is None or not x.is_cuda or x.dim() != 4 or self.training or torch.is_grad_enabled():
            return False
        enc = self._orig_mod
        patch = getattr(getattr(enc, "patch_embed", None), "proj", None)
        stride = patch.stride if patch is not None else (16, 16)
        rows = x.shape[0] * (x.shape[2] // stride[0]) * (x.shape[3] // stride[1])
        return 0 < rows <= self.max_rows and not torch.cuda.is_current_stream_capturing()

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if not self.replays(x):
            return self._orig_mod(x)
        key = (tuple(x.shape), x.dtype, x.device)
        graph = self._graphs.get(key)
        if graph is None:
            graph = GraphedEncoder(self._orig_mod, x)
            self._graphs[key] = graph
            while len(self._graphs) > self.max_graphs:
                self._graphs.popitem(last=False)
        else:
            self._graphs.move_to_end(key)
        return graph(x).clone()


def invalidate_recordings(model: nn.Module) -> None:
    """Drop the recorded graphs of every ReplayedEncoder at or below `model` (called by the
    functions of this package that swap modules or weights)."""
    for m in model.modules():
        if isinstance(m, ReplayedEncoder):
            m.invalidate()
