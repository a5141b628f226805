"""``dion.nordion2`` of microsoft/dion (dion/nordion2.py), served by ``dion_amd``."""
from dion_amd.functional import nordion2_normalize_selected_stacked  # noqa: F401
from dion_amd.global_scope import nordion2_post_orthogonalize_masked  # noqa: F401
from dion_amd.optimizers import NorDion2  # noqa: F401

__all__ = ["NorDion2", "nordion2_post_orthogonalize_masked", "nordion2_normalize_selected_stacked"]
