"""The tensor-free helpers of ``dion.opt_utils`` of microsoft/dion (dion/opt_utils.py:9-23).  The rest of
that module (DTensor conversion, batching across ranks, the generator runtime) belongs to the multi-GPU
control plane, which this package does not have."""
from dion_amd.functional import as_scalar_tensor, lm_head_lr_scale  # noqa: F401

__all__ = ["lm_head_lr_scale", "as_scalar_tensor"]
