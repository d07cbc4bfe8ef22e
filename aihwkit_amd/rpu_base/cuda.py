"""Mirror of ``rpu_base.cuda`` (src/aihwkit/simulator/rpu_base_src/rpu_base.cpp:60-85)."""
import os

from .._cabi import LIB_PATH


def is_compiled() -> bool:
    """Whether the GPU library has been built (the reference reports its CUDA build flag here)."""
    return os.path.exists(LIB_PATH)
