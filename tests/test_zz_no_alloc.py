"""The entry point that allocates nothing (rpu_tile_update_noalloc) against rpu_tile_update: same kernels and random
streams, scratch in the static device array instead of buffers of the tile.  Bit-identical weights and pulse words
on two calls in a row, the second one smaller (the array keeps the first call's contents)."""
import numpy as np
import pytest
import torch

from aihwkit_amd.rpu_base import tiles
from helpers import config2, constant_step, make_meta

pytestmark = pytest.mark.gpu


def pair(meta, dev, x_size, d_size, seed=5):
    rng = np.random.default_rng(3)
    host = meta.create_array(x_size, d_size, dev)
    host.set_weights(torch.from_numpy(rng.uniform(-0.4, 0.4, (d_size, x_size)).astype(np.float32)))
    a, b = tiles.CudaAnalogTile(host), tiles.CudaAnalogTile(host)
    for t in (a, b):
        t.set_learning_rate(0.01)
        t.set_seed(seed)
    b.set_update_without_allocation(True)
    return a, b


@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("layout", [(False, False), (True, True)])
def test_update_without_allocation_equals_update(bias, layout):
    meta, dev = config2()
    x_size, d_size = 200, 131
    ref, noa = pair(meta, dev, x_size, d_size)
    rng = np.random.default_rng(11)
    x_trans, d_trans = layout
    for batch in (150, 37):  # the second call is smaller: stale words and planes of the first stay in the array
        x = rng.uniform(-1, 1, (batch, x_size - int(bias))).astype(np.float32)
        d = (0.05 * rng.standard_normal((batch, d_size))).astype(np.float32)
        xg = torch.from_numpy(x.T.copy() if x_trans else x).cuda()
        dg = torch.from_numpy(d.T.copy() if d_trans else d).cuda()
        before = noa.get_weights().numpy().copy()
        ref.update(xg, dg, bias, x_trans, d_trans, False)
        noa.update(xg, dg, bias, x_trans, d_trans, False)
        w_ref, w_noa = ref.get_weights().numpy(), noa.get_weights().numpy()
        assert np.array_equal(w_ref, w_noa)
        assert np.abs(w_noa - before).max() > 1e-4
        for u, v in zip(ref.get_update_words(batch), noa.get_update_words(batch)):
            assert torch.equal(u, v)
        for u, v in zip(ref.get_update_ab(batch), noa.get_update_ab(batch)):
            assert torch.equal(u, v)


def test_first_call_without_allocation_on_a_fresh_tile_allocates_nothing():
    """The defining property: across the first such call on a tile that has never run an update, the library's buffers
    make no device allocation and the free device memory does not change (the kernels' code is loaded beforehand by an
    ordinary update on another tile)."""
    from aihwkit_amd._cabi import lib
    meta, dev = config2()
    ref, noa = pair(meta, dev, 300, 200)
    rng = np.random.default_rng(2)
    for bias in (False, True):
        batch = 96
        xg = torch.from_numpy(rng.uniform(-1, 1, (batch, 300 - int(bias))).astype(np.float32)).cuda()
        dg = torch.from_numpy((0.05 * rng.standard_normal((batch, 200))).astype(np.float32)).cuda()
        ref.update(xg, dg, bias, False, False, False)
        torch.cuda.synchronize()
        allocations, free = lib().rpu_device_allocation_count(), torch.cuda.mem_get_info()[0]
        noa.update(xg, dg, bias, False, False, True)
        torch.cuda.synchronize()
        assert lib().rpu_device_allocation_count() == allocations
        assert torch.cuda.mem_get_info()[0] == free
        assert np.array_equal(ref.get_weights().numpy(), noa.get_weights().numpy())


def test_update_without_allocation_on_another_device_kind_and_long_bit_lines():
    meta = make_meta(desired_bl=31, update_management=False, update_bl_management=False)
    dev = constant_step(dw_min=0.001, dw_min_std=0.3, construction_seed=9, enforce_consistency=True)
    ref, noa = pair(meta, dev, 70, 65)
    rng = np.random.default_rng(12)
    for batch in (64, 5):
        xg = torch.from_numpy(rng.uniform(-1, 1, (batch, 70)).astype(np.float32)).cuda()
        dg = torch.from_numpy((0.1 * rng.standard_normal((batch, 65))).astype(np.float32)).cuda()
        ref.update(xg, dg, False, False, False, False)
        noa.update(xg, dg, False, False, False, False)
        assert np.array_equal(ref.get_weights().numpy(), noa.get_weights().numpy())


def test_update_without_allocation_refuses_what_does_not_fit():
    meta, dev = config2()
    _, noa = pair(meta, dev, 1024, 1024)
    before = noa.get_weights().numpy().copy()
    xg = torch.zeros(512, 1024, device="cuda") + 0.5
    dg = torch.zeros(512, 1024, device="cuda") + 0.05
    with pytest.raises(RuntimeError, match="bytes of scratch, the static array holds"):
        noa.update(xg, dg, False, False, False, False)
    assert np.array_equal(noa.get_weights().numpy(), before)
    # the graded shape fits
    noa.update(xg[:256], dg[:256], False, False, False, False)
    assert np.abs(noa.get_weights().numpy() - before).max() > 1e-4
    meta.update.pulse_type = type(meta.update.pulse_type).DeterministicImplicit
    host = meta.create_array(40, 30, dev)
    det = tiles.CudaAnalogTile(host)
    det.set_learning_rate(0.01)
    det.set_update_without_allocation(True)
    with pytest.raises(RuntimeError, match="stochastic pulses"):
        det.update(xg[:8, :40].contiguous(), dg[:8, :30].contiguous(), False, False, False, False)
    # a bit line beyond 31 pulses needs several rows of words per sample: not in the static array
    from helpers import make_meta, soft_bounds
    long_meta = make_meta(desired_bl=64, fixed_bl=True, update_management=False, update_bl_management=False)
    long_tile = tiles.CudaAnalogTile(long_meta.create_array(40, 30, soft_bounds(construction_seed=1)))
    long_tile.set_learning_rate(0.01)
    long_tile.set_update_without_allocation(True)
    with pytest.raises(RuntimeError, match="at most 31 pulses"):
        long_tile.update(xg[:8, :40].contiguous(), dg[:8, :30].contiguous(), False, False, False, False)
