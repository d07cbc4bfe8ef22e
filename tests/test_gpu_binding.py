"""The compiled reference-side binding (tests/binding/rpu_base_tiles_amd.cpp: pybind11 + libtorch around the C entry
points) against the ctypes mirror: the same tile, seed and inputs give the same bits through either way in, with the
reference's layouts, error messages and the [x_size, d_size] shared-weight tensor of its CUDA tiles
(src/aihwkit/simulator/rpu_base_src/rpu_base_tiles_cuda.cpp:88-130,159-375)."""
import os
import sys

import numpy as np
import pytest
import torch

from aihwkit_amd.rpu_base import tiles
from helpers import config2

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "binding"))
import build_binding  # noqa: E402

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def module():
    return build_binding.load()


def pair(module, x_size=300, d_size=200, seed=11):
    meta, dev = config2()
    host = meta.create_array(x_size, d_size, dev)
    rng = np.random.default_rng(1)
    host.set_weights(torch.from_numpy(rng.uniform(-0.4, 0.4, (d_size, x_size)).astype(np.float32)))
    host.set_learning_rate(0.01)
    mirror = tiles.CudaAnalogTile(host)
    bound = module.CudaAnalogTile(host._h.value)
    mirror.set_seed(seed)
    bound.set_seed(seed)
    return host, mirror, bound


@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("trans", [False, True])
def test_forward_backward_update_equal_the_mirror(gpu_device, module, bias, trans):
    x_size, d_size, batch = 300, 200, 64
    _host, mirror, bound = pair(module, x_size, d_size)
    assert (bound.get_x_size(), bound.get_d_size()) == (x_size, d_size)
    assert bound.get_learning_rate() == pytest.approx(0.01)
    assert torch.equal(bound.get_weights(), mirror.get_weights())
    rng = np.random.default_rng(2)
    x = rng.uniform(-1, 1, (batch, x_size - int(bias))).astype(np.float32)
    d = (0.05 * rng.standard_normal((batch, d_size))).astype(np.float32)
    xg = torch.from_numpy(x.T.copy() if trans else x).cuda()
    dg = torch.from_numpy(d.T.copy() if trans else d).cuda()
    for _ in range(2):
        y_m = mirror.forward(xg, bias, trans, trans, False, False)
        y_b = bound.forward(xg, bias, trans, trans, False, False)
        assert y_b.shape == y_m.shape and torch.equal(y_b, y_m)
        g_m = mirror.backward(dg, bias, trans, trans, False)
        g_b = bound.backward(dg, bias, trans, trans, False)
        assert g_b.shape == g_m.shape and torch.equal(g_b, g_m)
        before = bound.get_weights().clone()
        mirror.update(xg, dg, bias, trans, trans, False)
        bound.update(xg, dg, bias, trans, trans, False)
        after = bound.get_weights()
        assert torch.equal(after, mirror.get_weights())
        assert float((after - before).abs().max()) > 1e-4
    # keyword form and leading batch dimensions, as the reference's layers call it
    x3 = torch.from_numpy(rng.uniform(-1, 1, (4, 8, x_size)).astype(np.float32)).cuda()
    y3 = bound.forward(x_input=x3, is_test=True, non_blocking=True)
    torch.cuda.synchronize()
    assert y3.shape == (4, 8, d_size)
    assert torch.equal(y3, mirror.forward(x3, False, False, False, True, False))


def test_the_shared_weight_tensor_of_the_reference(gpu_device, module):
    """set_shared_weights takes the [x_size, d_size] tensor of the reference's CUDA tiles: the tensor is the weight
    matrix from then on (an update changes it in place), results stay those of the mirror without a bound tensor."""
    x_size, d_size, batch = 256, 160, 48
    _host, mirror, bound = pair(module, x_size, d_size, seed=3)
    shared = torch.zeros(x_size, d_size, device="cuda")
    bound.set_shared_weights(shared)
    assert torch.equal(shared.t().cpu(), mirror.get_weights())
    rng = np.random.default_rng(4)
    xg = torch.from_numpy(rng.uniform(-1, 1, (batch, x_size)).astype(np.float32)).cuda()
    dg = torch.from_numpy((0.05 * rng.standard_normal((batch, d_size))).astype(np.float32)).cuda()
    assert torch.equal(bound.forward(xg), mirror.forward(xg, False, False, False, False, False))
    assert torch.equal(bound.backward(dg), mirror.backward(dg, False, False, False, False))
    bound.update(xg, dg, False)
    mirror.update(xg, dg, False, False, False, False)
    assert torch.equal(shared.t().cpu(), mirror.get_weights())
    assert torch.equal(bound.get_weights(), mirror.get_weights())
    with pytest.raises(RuntimeError, match=r"Invalid weights dimensions: expected \[256,160\] array"):
        bound.set_shared_weights(torch.zeros(d_size, x_size, device="cuda"))


def test_error_messages_of_the_reference(gpu_device, module):
    _host, _mirror, bound = pair(module, 40, 30)
    with pytest.raises(RuntimeError, match=r"Invalid x_input dimensions: expected \[40, \*\] array"):
        bound.forward(torch.zeros(8, 41, device="cuda"))
    with pytest.raises(RuntimeError, match=r"Invalid d_input dimensions: expected \[\*, 30\] array"):
        bound.backward(torch.zeros(31, 8, device="cuda"), False, True, True)
    with pytest.raises(RuntimeError, match="batch dimensions mismatch"):
        bound.update(torch.zeros(8, 40, device="cuda"), torch.zeros(9, 30, device="cuda"), False)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        bound.forward(torch.zeros(8, 40))
    bound.set_learning_rate(0.0)                       # a zero learning rate: update returns before any check
    bound.update(torch.zeros(8, 40), torch.zeros(9, 30), False)
