"""``dion.scalar_opts`` of microsoft/dion (dion/scalar_opts.py:121-308), served by the multi-tensor HIP
kernels of ``dion_amd``."""
from dion_amd.functional import adamw_update_foreach, lion_update_foreach  # noqa: F401

__all__ = ["adamw_update_foreach", "lion_update_foreach"]
