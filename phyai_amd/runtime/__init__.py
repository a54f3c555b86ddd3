"""Graph capture / replay for the per-step linear sequence."""

from phyai_amd.runtime.graph import HipGraph, HipGraphError, HipGraphRegistry

# Names the reference uses for the same objects (runtime/cuda_graph_manager.py).
CudaGraph = HipGraph
CudaGraphError = HipGraphError
CudaGraphRegistry = HipGraphRegistry

__all__ = ["HipGraph", "HipGraphError", "HipGraphRegistry", "CudaGraph", "CudaGraphError", "CudaGraphRegistry"]
# The denoise loop (phyai_amd.runtime.expert_loop) is imported from its module: it pulls in the
# layers, which import this package for the capture-mode flag.
