"""The reference-side binding (pybind11 + libtorch around the C entry points) compiles, links against librpu_amd.so
and imports; its CudaAnalogTile carries the reference's methods with the reference's argument names and defaults
(src/aihwkit/simulator/rpu_base_src/rpu_base_tiles_cuda.cpp:88-130,159-375).  No GPU call is made here."""
import inspect
import os
import sys

import pytest

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "binding"))
import build_binding  # noqa: E402


@pytest.fixture(scope="module")
def module():
    return build_binding.load()


def test_the_binding_builds_and_imports(module):
    assert os.path.exists(build_binding.MODULE)
    assert hasattr(module, "CudaAnalogTile")


def test_the_bound_class_has_the_reference_surface(module):
    cls = module.CudaAnalogTile
    for name in ("forward", "backward", "update", "get_weights", "set_weights", "set_learning_rate", "get_learning_rate",
                 "get_x_size", "get_d_size", "set_shared_weights", "set_delta_weights"):
        assert callable(getattr(cls, name)), name
    doc = cls.forward.__doc__
    for arg in ("x_input", "bias: bool = False", "x_trans: bool = False", "d_trans: bool = False", "is_test: bool = False",
                "non_blocking: bool = False"):
        assert arg in doc, arg
    doc = cls.backward.__doc__
    for arg in ("d_input", "bias: bool = False", "d_trans: bool = False", "x_trans: bool = False", "non_blocking: bool = False"):
        assert arg in doc, arg
    assert doc.index("d_trans") < doc.index("x_trans")             # backward takes d_trans before x_trans
    doc = cls.update.__doc__
    assert doc.index("x_input") < doc.index("d_input") < doc.index("bias")


def test_a_null_tile_is_refused(module):
    with pytest.raises(RuntimeError, match="null tile"):
        module.CudaAnalogTile(0)
