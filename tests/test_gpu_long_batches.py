"""Updates over thousands of samples on small tiles (what the patches of a convolution are to its tile): the pulse loop
fetches the bit planes of eight 32-sample chunks at a time, with a variant for bit lines of a single pulse, and the
set-up kernel shares a workgroup between samples.  BL and pulse words must equal the oracle's choice, the weights the
oracle's update driven by the same words."""
import numpy as np
import pytest
import torch

from aihwkit_amd.rpu_base import tiles
from helpers import build_pair, constant_step, make_meta, noise_free_io, soft_bounds

pytestmark = pytest.mark.gpu
F = np.float32


@pytest.mark.parametrize("x_size,d_size,batch", [(26, 16, 5000), (70, 33, 2100), (300, 40, 1100)])
@pytest.mark.parametrize("d_cap,longest", [(0.09, 1), (0.29, 3), (5.0, 31)])     # bit lines of 1, up to 3, up to 31 pulses
def test_long_batches_follow_the_oracle(gpu_device, x_size, d_size, batch, d_cap, longest):
    rng = np.random.default_rng(x_size + longest)
    for dev in (constant_step(construction_seed=2, dw_min_std=0.0), soft_bounds(construction_seed=3, dw_min_std=0.0)):
        host, orc, _ = build_pair(make_meta(noise_free_io(), noise_free_io()), dev, x_size, d_size, gpu=False)
        w = rng.uniform(-0.3, 0.3, (d_size, x_size)).astype(F)
        host.set_weights(torch.from_numpy(w))
        orc.set_weights(w)
        gpu = tiles.CudaAnalogTile(host)
        gpu.set_learning_rate(0.01)
        orc.set_learning_rate(0.01)
        x = rng.uniform(-1, 1, (batch, x_size)).astype(F)
        d = np.clip(rng.normal(0, 1, (batch, d_size)) * d_cap / 2, -d_cap, d_cap).astype(F)   # BL = ceil(10 max |x| max |d|)
        x[7] = 0.0
        gpu.update(torch.from_numpy(x).cuda(), torch.from_numpy(d).cuda(), False)
        xw, dw, bl = gpu.get_update_words(batch)
        bl_orc, a_orc, b_orc = orc.update_bl_ab(x, d)
        assert np.array_equal(bl.numpy(), bl_orc)
        assert bl.max() == longest and bl[7] == 0
        orc.update_with_words(xw.numpy().astype(np.uint32), dw.numpy().astype(np.uint32), bl.numpy())
        assert np.abs(gpu.get_weights().numpy() - orc.get_weights()).max() <= 3e-6
        assert np.abs(gpu.get_weights().numpy() - w).max() > 1e-3


def test_long_batch_with_noise_has_the_oracle_s_moments(gpu_device):
    """Cycle-to-cycle noise on: mean and spread of the weight change over the cross-points of a small tile after 4000
    samples agree with the oracle's (different random streams: a statistical comparison)."""
    rng = np.random.default_rng(11)
    x_size, d_size, batch = 64, 48, 4000
    dev = soft_bounds(construction_seed=5, dw_min_std=0.3, dw_min_dtod=0.0, up_down_dtod=0.0, w_max_dtod=0.0, w_min_dtod=0.0)
    host, orc, _ = build_pair(make_meta(noise_free_io(), noise_free_io()), dev, x_size, d_size, gpu=False)
    w = np.zeros((d_size, x_size), F)
    host.set_weights(torch.from_numpy(w))
    orc.set_weights(w)
    gpu = tiles.CudaAnalogTile(host)
    gpu.set_learning_rate(0.01)
    orc.set_learning_rate(0.01)
    x = np.abs(rng.uniform(0.5, 1, (batch, x_size))).astype(F)
    d = -np.abs(rng.normal(0, 0.02, (batch, d_size))).astype(F)          # every step goes up
    gpu.update(torch.from_numpy(x).cuda(), torch.from_numpy(d).cuda(), False)
    orc.update(x, d)
    dw_gpu, dw_orc = gpu.get_weights().numpy() - w, orc.get_weights() - w
    assert dw_orc.mean() > 0.01
    assert dw_gpu.mean() == pytest.approx(dw_orc.mean(), rel=0.05)
    assert dw_gpu.std() == pytest.approx(dw_orc.std(), rel=0.15)
