"""Mirror of ``aihwkit.simulator.rpu_base`` (src/aihwkit/simulator/rpu_base_src/rpu_base.cpp:12-86)."""
from . import devices, tiles, cuda  # noqa: F401

__all__ = ["devices", "tiles", "cuda"]
