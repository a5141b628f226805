"""``from dion.cuda_graph import CudaGraphOptimizer`` -- the import path of microsoft/dion
(dion/cuda_graph.py:88), served by the hipGraph wrapper of ``dion_amd``."""
from dion_amd.hip_graph import CudaGraphOptimizer, HipGraphOptimizer

__all__ = ["CudaGraphOptimizer", "HipGraphOptimizer"]
