"""``dion.dion2`` of microsoft/dion (dion/dion2.py), served by ``dion_amd``: the optimizer class and the
operator functions around the orthogonalization."""
from dion_amd.functional import (  # noqa: F401
    dion2_post_orthogonalize,
    dion2_post_orthogonalize_fused,
    dion2_pre_orthogonalize,
)
from dion_amd.global_scope import (  # noqa: F401
    dion2_post_orthogonalize_masked,
    dion2_pre_accumulate,
    make_select_and_orthogonalize as _make_select_and_orthogonalize,
)
from dion_amd.optimizers import Dion2  # noqa: F401

__all__ = ["Dion2", "dion2_pre_orthogonalize", "dion2_post_orthogonalize", "dion2_post_orthogonalize_fused",
           "dion2_pre_accumulate", "dion2_post_orthogonalize_masked"]
