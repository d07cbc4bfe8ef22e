"""MI355X-native implementation of the aihwkit analog-tile hot path.

``aihwkit_amd.rpu_base`` mirrors the module ``aihwkit.simulator.rpu_base`` (sub-modules ``devices``,
``tiles``, ``cuda``) for the analog tile: parameter structs with the same field names, ``create_array``
and GPU tile classes with ``forward`` / ``backward`` / ``update`` taking torch tensors.  All tile
arithmetic runs in ``lib/librpu_amd.so`` (HIP kernels for gfx950) through the C ABI of
``include/rpu_amd.h``.
"""
from . import rpu_base  # noqa: F401

__all__ = ["rpu_base"]
