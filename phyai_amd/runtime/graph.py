"""hipGraph capture and replay of a fixed kernel sequence.

Semantics follow the reference's ``phyai/runtime/cuda_graph_manager.py:76-317``
(``CudaGraph`` / ``CudaGraphRegistry``): example inputs are cloned into static
buffers, the function is run a few times on a side stream so every lazy
allocation (here: the kernels' workspace, which the graph owns) exists, then it is recorded once into
a graph with the dispatcher in capture mode; ``replay`` copies new inputs into
the static buffers and launches the whole recording with a single call.  The
returned tensors alias static storage and are overwritten by the next replay.

On ROCm ``torch.cuda.CUDAGraph`` is a hipGraph.  Streams are created at the
default priority, and nothing in the recorded region may issue a memset: the
kernels clear what they need themselves.
"""

from __future__ import annotations

from typing import Any, Callable, Hashable

import torch

from phyai_amd.ops import WorkspaceOwner, workspace_owner
from phyai_amd.state import graph_capture


class HipGraphError(RuntimeError):
    """Capture / replay called out of order or with mismatching inputs."""


class HipGraph:
    def __init__(self, *, num_warmup_iters: int = 3, mempool: Any | None = None) -> None:
        if num_warmup_iters < 0:
            raise ValueError(f"num_warmup_iters must be non-negative, got {num_warmup_iters}.")
        self.num_warmup_iters = int(num_warmup_iters)
        self.mempool = mempool
        self._graph: torch.cuda.CUDAGraph | None = None
        self._inputs: dict[str, torch.Tensor] = {}
        self._output: Any = None
        # The kernels' scratch, owned by this graph: its addresses are part of the recording.
        self._workspace = WorkspaceOwner()
        self.capture_stream: torch.cuda.Stream | None = None

    @property
    def is_captured(self) -> bool:
        return self._graph is not None

    def _need_capture(self) -> None:
        if self._graph is None:
            raise HipGraphError("graph has not been captured yet.")

    def input_buffer(self, name: str) -> torch.Tensor:
        self._need_capture()
        if name not in self._inputs:
            raise HipGraphError(f"unknown input buffer {name!r}; known names are {sorted(self._inputs)!r}.")
        return self._inputs[name]

    def input_buffers(self) -> dict[str, torch.Tensor]:
        self._need_capture()
        return dict(self._inputs)

    def capture(self, fn: Callable[..., Any], example_inputs: dict[str, torch.Tensor]) -> None:
        """Warm ``fn(**inputs)`` up on a side stream, then record it."""
        if self._graph is not None:
            raise HipGraphError("graph already captured; construct a new instance for another fn / shape.")
        if not torch.cuda.is_available():
            raise HipGraphError("capture requires a GPU; none is available.")
        for name, t in example_inputs.items():
            if not isinstance(t, torch.Tensor):
                raise HipGraphError(f"example_inputs[{name!r}] must be a Tensor, got {type(t)!r}.")
            if not t.is_cuda:
                raise HipGraphError(f"example_inputs[{name!r}] must live on the GPU, got device={t.device}.")
        bufs = {name: t.clone() for name, t in example_inputs.items()}

        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side), workspace_owner(self._workspace):
            for _ in range(self.num_warmup_iters):
                fn(**bufs)
        torch.cuda.current_stream().wait_stream(side)

        graph = torch.cuda.CUDAGraph()
        kwargs = {"stream": side}
        if self.mempool is not None:
            kwargs["pool"] = self.mempool
        # The warm-up created this graph's workspace; recording finds it through the same owner.
        # Streams come from a pool and are handed out again: nothing may be keyed by them alone.
        with graph_capture(), workspace_owner(self._workspace), torch.cuda.graph(graph, **kwargs):
            out = fn(**bufs)
        self._graph, self._inputs, self._output, self.capture_stream = graph, bufs, out, side

    def replay(self, inputs: dict[str, torch.Tensor] | None = None) -> Any:
        self._need_capture()
        for name, t in (inputs or {}).items():
            buf = self._inputs.get(name)
            if buf is None:
                raise HipGraphError(f"unknown input {name!r}; known names are {sorted(self._inputs)!r}.")
            if t.shape != buf.shape:
                raise HipGraphError(f"input {name!r} shape {tuple(t.shape)} does not match captured "
                                    f"buffer shape {tuple(buf.shape)}.")
            buf.copy_(t, non_blocking=t.is_cuda)
        self._graph.replay()  # type: ignore[union-attr]
        return self._output


class HipGraphRegistry:
    """``key -> HipGraph`` for shape-bucketed replay (one graph per prefix length, per batch, ...)."""

    def __init__(self) -> None:
        self._graphs: dict[Hashable, HipGraph] = {}

    def register(self, key: Hashable, graph: HipGraph) -> None:
        if key in self._graphs:
            raise HipGraphError(f"key {key!r} already registered; deregister it first to overwrite.")
        if not graph.is_captured:
            raise HipGraphError(f"cannot register graph for key {key!r}: it has not been captured yet.")
        self._graphs[key] = graph

    def deregister(self, key: Hashable) -> HipGraph:
        if key not in self._graphs:
            raise HipGraphError(f"unknown key {key!r}.")
        return self._graphs.pop(key)

    def get(self, key: Hashable) -> HipGraph | None:
        return self._graphs.get(key)

    def has(self, key: Hashable) -> bool:
        return key in self._graphs

    __contains__ = has

    def __getitem__(self, key: Hashable) -> HipGraph:
        if key not in self._graphs:
            raise HipGraphError(f"unknown key {key!r}; registered keys: {sorted(map(repr, self._graphs))}.")
        return self._graphs[key]

    def __len__(self) -> int:
        return len(self._graphs)

    def keys(self):
        return self._graphs.keys()


__all__ = ["HipGraph", "HipGraphError", "HipGraphRegistry"]
