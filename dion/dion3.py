"""``dion.dion3`` of microsoft/dion: ``Dion3`` is ``NorDion2`` (dion/__init__.py:9-10)."""
from dion_amd.optimizers import Dion3  # noqa: F401

__all__ = ["Dion3"]
