"""Pins of the indexed (convolution) oracle against torch's own convolution; CPU only.  The index matrix is built
the way the reference's conv layers build it (src/aihwkit/nn/modules/conv.py:534-575)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from aihwkit_amd.rpu_base import devices as dv
from helpers import make_meta, noise_free_io
from indexed_oracle import IndexedOracle
from oracle_lib import OracleTile


def conv_indices(image_shape, kernel, stride, padding, dilation, bias):
    """image_shape = (C, H, W); returns the int32 index vector and the number of patches."""
    size = int(np.prod(image_shape))
    idx = torch.arange(2, size + 2, dtype=torch.float64).reshape(1, *image_shape)
    idx = F.unfold(idx, kernel_size=kernel, stride=stride, padding=padding, dilation=dilation).flatten().round().to(torch.int32)
    patches = idx.numel() // (image_shape[0] * kernel[0] * kernel[1])
    if bias:
        idx = torch.cat((idx, torch.ones(patches, dtype=torch.int32)), 0)
    return idx, patches


def ideal_tile(x_size, d_size, lr=0.0):
    meta = make_meta(noise_free_io(is_perfect=True), noise_free_io(is_perfect=True))
    meta.update.pulse_type = dv.PulseType.NONE
    tile = OracleTile(x_size, d_size, meta._config(dv.IdealResistiveDeviceParameter()))
    tile.set_learning_rate(lr)
    return tile


@pytest.mark.parametrize("kernel,stride,padding,dilation,bias", [
    ((3, 3), (1, 1), (0, 0), (1, 1), False), ((5, 5), (1, 1), (2, 2), (1, 1), True), ((3, 2), (2, 1), (1, 0), (1, 2), True)])
def test_indexed_forward_backward_update_are_a_convolution(kernel, stride, padding, dilation, bias):
    rng = np.random.default_rng(0)
    c_in, c_out, height, width, n = 3, 4, 9, 8, 2
    indices, patches = conv_indices((c_in, height, width), kernel, stride, padding, dilation, bias)
    x_size = c_in * kernel[0] * kernel[1] + int(bias)
    tile = ideal_tile(x_size, c_out, lr=0.1)
    w = rng.normal(0, 0.3, (c_out, x_size)).astype(np.float32)
    tile.set_weights(w)
    orc = IndexedOracle(tile, indices.numpy(), patches)
    x = torch.from_numpy(rng.normal(0, 1, (n, c_in, height, width)).astype(np.float32)).requires_grad_(True)
    weight = torch.from_numpy(w[:, :x_size - int(bias)].reshape(c_out, c_in, *kernel).copy()).requires_grad_(True)
    b = torch.from_numpy(w[:, -1].copy()).requires_grad_(True) if bias else None
    y = F.conv2d(x, weight, b, stride=stride, padding=padding, dilation=dilation)
    got = orc.forward(x.detach().numpy())
    assert got.shape == (n, c_out, patches) and y.shape[2] * y.shape[3] == patches
    assert np.allclose(got, y.detach().numpy().reshape(n, c_out, patches), atol=1e-5)
    grad_out = torch.from_numpy(rng.normal(0, 1, tuple(y.shape)).astype(np.float32))
    y.backward(grad_out)
    got_dx = orc.backward(grad_out.numpy(), c_in * height * width)
    assert np.allclose(got_dx, x.grad.numpy().reshape(n, -1), atol=1e-5)        # overlapping patches add up
    orc.update(x.detach().numpy(), grad_out.numpy())                             # W -= lr * dW
    dw = weight.grad.numpy().reshape(c_out, -1)
    want = w.copy()
    want[:, :x_size - int(bias)] -= 0.1 * dw
    if bias:
        want[:, -1] -= 0.1 * b.grad.numpy()
    assert np.allclose(tile.get_weights(), want, atol=1e-5)
