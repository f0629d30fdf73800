"""HIP-graph replay of small tensor programs around the compressed operators (decode and draft-verify steps).

A block of a decoder layer -- an MLP, a routed-expert block with its router, a group of projections -- is a fixed
sequence of launches on static weight addresses with no host synchronisation.  `GraphedBlock` keeps one captured graph
per input signature (shape, dtype) of such a block: the first call with a signature runs eagerly (that also builds
whatever the operators build lazily: row records, expert stacks, fused groups -- allocations that must not happen
inside a capture), the second captures, later ones copy the input into the graph's static input, replay, and hand out a
copy of the static output.  Anything that cannot be captured, inputs of more than `max_rows` rows (prefill) and calls
made while another capture is running stay eager.  Replay launches the same kernels with the same arguments: results
are bit-identical to eager execution.

Counterpart of the reference's formats/qvb8/moe_graph.py:58-178 (install_moe_graphs / install_mlp_graphs) and
decode/proj_graph.py:27-117; `QVB8_AMD_GRAPHS=0` turns it off.
"""
from __future__ import annotations

import os

import torch
import torch.nn as nn

MAX_ROWS = int(os.environ.get("QVB8_AMD_GRAPH_MAX_ROWS", "16"))
_POOL: dict = {}
_STREAM: dict = {}


def _per_device(table: dict, device, make):
    idx = device.index if device.index is not None else torch.cuda.current_device()
    if idx not in table:
        with torch.cuda.device(idx):
            table[idx] = make(idx)
    return table[idx]


class GraphedBlock(nn.Module):
    """Wraps `block` (one tensor in, one tensor out)."""

    def __init__(self, block: nn.Module, max_rows: int = MAX_ROWS):
        super().__init__()
        self.block = block
        self.max_rows = int(max_rows)
        self._graphs: dict = {}           # signature -> None (seen once) | False (not capturable) | (graph, static in, static out)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        rows = x.numel() // max(x.shape[-1], 1)
        if (os.environ.get("QVB8_AMD_GRAPHS", "1") == "0" or not x.is_cuda or rows > self.max_rows
                or torch.is_grad_enabled() and x.requires_grad or torch.cuda.is_current_stream_capturing()):
            return self.block(x)
        key = (tuple(x.shape), x.dtype, x.device)
        entry = self._graphs.get(key, "new")
        if entry == "new":
            self._graphs[key] = None
            return self.block(x)
        if entry is False:
            return self.block(x)
        if entry is None:
            entry = self._graphs[key] = self._capture(x)
            if entry is False:
                return self.block(x)
        graph, static_in, static_out = entry
        static_in.copy_(x)
        graph.replay()
        return static_out.clone()

    def _capture(self, x: torch.Tensor):
        dev = x.device
        pool = _per_device(_POOL, dev, lambda i: torch.cuda.graph_pool_handle())
        stream = _per_device(_STREAM, dev, lambda i: torch.cuda.Stream(device=i))
        static_in = x.detach().clone()
        try:
            stream.wait_stream(torch.cuda.current_stream(dev))
            with torch.cuda.stream(stream), torch.no_grad():
                self.block(static_in)                              # warm on the capture stream
            torch.cuda.current_stream(dev).wait_stream(stream)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.device(dev), torch.no_grad(), torch.cuda.graph(graph, pool=pool, stream=stream, capture_error_mode="thread_local"):
                static_out = self.block(static_in)
        except Exception as ex:                                   # noqa: BLE001  (whatever refuses capture: stay eager)
            torch.cuda.synchronize(dev)
            print(f"[qvb8_amd.graph] {type(self.block).__name__} {tuple(x.shape)}: capture failed ({type(ex).__name__}: {ex}); eager")
            return False
        if not isinstance(static_out, torch.Tensor):
            return False
        return graph, static_in, static_out

    def extra_repr(self):
        return f"max_rows={self.max_rows}, graphs={sum(1 for v in self._graphs.values() if isinstance(v, tuple))}"


def _uses_compressed_weights(module: nn.Module) -> bool:
    from qvb8_amd.formats.qvb8.backends_experts import QVBandExpertsV8
    from qvb8_amd.formats.qvb8.fuse import FusedMember
    from qvb8_amd.formats.qvb8.module import QVBandLinearV8
    return any(isinstance(m, (QVBandLinearV8, QVBandExpertsV8, FusedMember)) for m in module.modules())


def install_block_graphs(model: nn.Module, names=("mlp",), max_rows: int = MAX_ROWS) -> int:
    """Wraps every submodule called `mlp` (or any of `names`) that holds compressed weights in a GraphedBlock; returns
    how many.  Blocks must map one tensor to one tensor (an MLP, a MoE block that routes inside)."""
    n = 0
    for parent in list(model.modules()):
        for name in names:
            child = getattr(parent, name, None)
            if isinstance(child, nn.Module) and not isinstance(child, GraphedBlock) and _uses_compressed_weights(child):
                setattr(parent, name, GraphedBlock(child, max_rows))
                n += 1
    return n
