"""``dion.dion2_triton`` of microsoft/dion (dion/dion2_triton.py:30-242), served by ``dion_amd``.
``TRITON_AVAILABLE`` is kept for callers that gate on it: the fused kernel here does not need Triton."""
from dion_amd.functional import _build_index_map, dion2_post_orthogonalize_triton  # noqa: F401

TRITON_AVAILABLE = True

__all__ = ["TRITON_AVAILABLE", "dion2_post_orthogonalize_triton"]
