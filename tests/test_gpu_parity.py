"""GPU parity tests: the HIP path (through the C ABI) against the CPU oracle on the same inputs.

Bar: pulse words / coincidence counts / bit-line lengths bit-exact; weights and outputs within 1e-5
absolute (fp32) when noise is off and pulses are deterministic or shared.
"""
import ctypes as C

import numpy as np
import pytest
import torch

from aihwkit_amd._cabi import lib
from aihwkit_amd.rpu_base import devices as dv
from aihwkit_amd.rpu_base import tiles
from helpers import (build_pair, config1, config1_data, config2, config2_data, constant_step, io_params,
                     make_meta, noise_free_io, soft_bounds)

pytestmark = pytest.mark.gpu

TOL = 1e-5


def cuda(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def test_philox_known_answers_on_device(gpu_device):
    # Random123 known-answer vectors for philox4x32-10
    kat = [
        ([0, 0, 0, 0], [0, 0], [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]),
        ([0xFFFFFFFF] * 4, [0xFFFFFFFF] * 2, [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]),
        ([0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344], [0xA4093822, 0x299F31D0],
         [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]),
    ]
    for ctr, key, want in kat:
        out = (C.c_uint32 * 4)()
        assert lib().rpu_philox4x32_10_device((C.c_uint32 * 4)(*ctr), (C.c_uint32 * 2)(*key), out, 0) == 0
        assert list(out) == want


@pytest.mark.parametrize("x_size,d_size,batch", [(64, 32, 32), (100, 70, 33), (512, 512, 100), (1024, 1024, 256),
                                                 # large workgroup tiles: 128 outputs x 64 samples ...
                                                 (1024, 1024, 4096), (777, 1000, 4700),
                                                 # ... and x 128 samples (512 of them: two on every CU), forward / backward
                                                 (96, 1024, 8192), (1024, 96, 8192),
                                                 # a long batch on a narrow tile: large tiles with idle outputs, the rows
                                                 # of a further round written only for the samples that go on
                                                 (300, 48, 16500)])
@pytest.mark.parametrize("bm", [dv.BoundManagementType.NONE, dv.BoundManagementType.Iterative])
def test_forward_exact_arithmetic_is_bit_exact(gpu_device, x_size, d_size, batch, bm):
    """With a power-of-two DAC step and weights on a 1/64 grid every product and partial sum is exact in
    fp32, so the summation order cannot matter: GPU and oracle must agree to the last bit."""
    rng = np.random.default_rng(5)
    f_io = noise_free_io(inp_res=1 / 128.0, out_res=1 / 512.0, bound_management=bm,
                         noise_management=dv.NoiseManagementType.AbsMax)
    meta = make_meta(f_io, noise_free_io(inp_res=1 / 128.0, out_res=1 / 512.0))
    dev = constant_step(w_max_dtod=0.0, w_min_dtod=0.0, w_max=1.0, w_min=-1.0, construction_seed=7)
    host, orc, _ = build_pair(meta, dev, x_size, d_size, gpu=False)
    w = (rng.integers(-38, 39, (d_size, x_size)) / 64.0).astype(np.float32)
    host.set_weights(torch.from_numpy(w))
    orc.set_weights(w)
    gpu = tiles.CudaAnalogTile(host)
    x = rng.uniform(-1, 1, (batch, x_size)).astype(np.float32)
    x[0] = 0.0  # the zero short-cut
    y_gpu = gpu.forward(cuda(x), False, False, False, False, False).cpu().numpy()
    y_orc = orc.forward(x)
    assert np.array_equal(y_gpu, y_orc)
    if bm != dv.BoundManagementType.NONE:
        assert np.array_equal(gpu.get_bm_rounds(batch).numpy(), orc.bm_rounds(batch))
        if x_size >= 512 or batch > 10000:
            assert orc.bm_rounds(batch).max() > 1  # the case does exercise re-runs
    # backward, same property
    d = rng.uniform(-1, 1, (batch, d_size)).astype(np.float32)
    assert np.array_equal(gpu.backward(cuda(d), False, False, False, False).cpu().numpy(), orc.backward(d))


def _compare_with_lsb_flips(y_gpu, y_orc, lsb_per_row, max_flip_fraction):
    diff = np.abs(y_gpu - y_orc)
    bad = diff > TOL
    # a differing entry must be exactly one ADC step (times the sample's output scale) away
    rows = np.nonzero(bad)[0]
    if rows.size:
        steps = diff[bad] / lsb_per_row[rows]
        assert np.allclose(steps, 1.0, atol=1e-3), steps
    return bad.mean() <= max_flip_fraction, bad.mean()


@pytest.mark.parametrize("cfg,data,shape", [(config1, config1_data, (512, 512, 100)),
                                            (config2, config2_data, (1024, 1024, 256))])
def test_forward_backward_benchmark_configs_noise_free(gpu_device, cfg, data, shape):
    """Real DAC / ADC steps (1/126, 1/510): pre-ADC sums differ in the last bits between summation
    orders, so an output may land on the other side of an ADC rounding edge.  Everything else must be
    within 1e-5 and the flips must be exactly one LSB and rare.  The rows left out here (another round
    count) and the values before the ADC are checked in test_gpu_benchmark_configs.py: those rows sit on
    the saturation edge, and the pre-ADC values agree on every row."""
    x_size, d_size, batch = shape
    meta, dev = cfg(noise=False)
    host, orc, _ = build_pair(meta, dev, x_size, d_size, gpu=False)
    w, x, d = data(x_size, d_size, batch)
    host.set_weights(torch.from_numpy(w))
    orc.set_weights(w)
    gpu = tiles.CudaAnalogTile(host)
    assert np.array_equal(gpu.get_weights().numpy(), orc.get_weights())

    y_gpu = gpu.forward(cuda(x), False, False, False, False, False).cpu().numpy()
    y_orc = orc.forward(x)
    r_gpu, r_orc = gpu.get_bm_rounds(batch).numpy(), orc.bm_rounds(batch)
    same_rounds = r_gpu == r_orc
    assert same_rounds.mean() > 0.97  # a flip at the ADC bound can change the round count of a sample
    out_step = (1.0 / 510.0) * 24.0 if cfg is config2 else (1.0 / 511.0) * 24.0
    nm = np.abs(x).max(axis=1)
    lsb = out_step * nm * (2.0 ** (r_orc - 1))
    ok, frac = _compare_with_lsb_flips(y_gpu[same_rounds], y_orc[same_rounds], lsb[same_rounds], 5e-3)
    assert ok, frac

    x_gpu = gpu.backward(cuda(d), False, False, False, False).cpu().numpy()
    x_orc = orc.backward(d)
    lsb_b = out_step * np.abs(d).max(axis=1)
    ok, frac = _compare_with_lsb_flips(x_gpu, x_orc, lsb_b, 5e-3)
    assert ok, frac


@pytest.mark.parametrize("x_trans,d_trans,bias", [(False, False, False), (True, False, False), (False, True, False),
                                                  (True, True, False), (False, False, True), (True, True, True)])
def test_forward_backward_layouts(gpu_device, x_trans, d_trans, bias):
    rng = np.random.default_rng(11)
    x_size, d_size, batch = 72, 40, 19
    f_io = noise_free_io(inp_res=1 / 128.0, out_res=1 / 512.0, bound_management=dv.BoundManagementType.Iterative)
    meta = make_meta(f_io, noise_free_io(inp_res=1 / 128.0, out_res=1 / 512.0))
    dev = constant_step(w_max_dtod=0.0, w_min_dtod=0.0, w_max=1.0, w_min=-1.0, construction_seed=7)
    host, orc, _ = build_pair(meta, dev, x_size, d_size, gpu=False)
    w = (rng.integers(-38, 39, (d_size, x_size)) / 64.0).astype(np.float32)
    host.set_weights(torch.from_numpy(w))
    orc.set_weights(w)
    gpu = tiles.CudaAnalogTile(host)
    xs = x_size - int(bias)
    x = rng.uniform(-1, 1, (xs, batch) if x_trans else (batch, xs)).astype(np.float32)
    y_gpu = gpu.forward(cuda(x), bias, x_trans, d_trans, False, False).cpu().numpy()
    assert y_gpu.shape == ((d_size, batch) if d_trans else (batch, d_size))
    assert np.array_equal(y_gpu, orc.forward(x, bias, x_trans, d_trans))
    d = rng.uniform(-1, 1, (d_size, batch) if d_trans else (batch, d_size)).astype(np.float32)
    x_gpu = gpu.backward(cuda(d), bias, d_trans, x_trans, False).cpu().numpy()
    assert x_gpu.shape == ((xs, batch) if x_trans else (batch, xs))
    assert np.array_equal(x_gpu, orc.backward(d, bias, d_trans, x_trans))


@pytest.mark.parametrize("x_size,d_size,batch", [(200, 150, 64),
                                                 (100, 48, 20000),     # large tiles with idle outputs, both directions
                                                 (60, 130, 4000)])
def test_floating_point_tile(gpu_device, x_size, d_size, batch):
    rng = np.random.default_rng(3)
    host = dv.FloatingPointTileParameter().create_array(x_size, d_size)
    w = rng.standard_normal((d_size, x_size)).astype(np.float32)
    host.set_weights(torch.from_numpy(w))
    gpu = tiles.CudaFloatingPointTile(host)
    x = rng.standard_normal((batch, x_size)).astype(np.float32)
    d = rng.standard_normal((batch, d_size)).astype(np.float32)
    y = gpu.forward(cuda(x)).cpu().numpy()
    assert np.allclose(y, x.astype(np.float64) @ w.T.astype(np.float64), atol=1e-4)
    xb = gpu.backward(cuda(d)).cpu().numpy()
    assert np.allclose(xb, d.astype(np.float64) @ w.astype(np.float64), atol=1e-4)
    gpu.set_learning_rate(0.1)
    gpu.update(cuda(x), cuda(d), False)
    want = w.astype(np.float64) - 0.1 * d.T.astype(np.float64) @ x.astype(np.float64)
    assert np.allclose(gpu.get_weights().numpy(), want, atol=1e-4 * max(1.0, batch / 64.0))


def _word_invariants(words, values, bl):
    words = words.astype(np.int64) & 0xFFFFFFFF
    pulses = words >> 1
    # no pulse beyond the sample's BL
    limit = (1 << bl.astype(np.int64)) - 1
    assert np.all((pulses & ~limit[:, None]) == 0)
    # sign bit only where the input is not positive, and zero input gives an empty word
    has = pulses != 0
    assert np.all(((words & 1) == 1)[has] == (values <= 0)[has])
    assert np.all(words[values == 0] == 0)


@pytest.mark.parametrize("device", ["constant", "soft"])
@pytest.mark.parametrize("um", [True, False])
def test_stochastic_update_words_drive_the_oracle_to_the_same_weights(gpu_device, device, um):
    """Cycle-to-cycle noise off: the GPU's packed pulse words, fed to the oracle's sparse update loop
    (the reference's updateVectorWithDeviceAndCounts protocol), must give the GPU's weights."""
    rng = np.random.default_rng(21)
    x_size, d_size, batch = 96, 80, 40
    meta = make_meta(desired_bl=31, update_management=um, update_bl_management=um)
    kw = dict(dw_min=0.001, dw_min_std=0.0, construction_seed=99, enforce_consistency=True)
    dev = constant_step(**kw) if device == "constant" else soft_bounds(**kw)
    host, orc, _ = build_pair(meta, dev, x_size, d_size, gpu=False)
    w = rng.uniform(-0.5, 0.5, (d_size, x_size)).astype(np.float32)
    host.set_weights(torch.from_numpy(w))
    orc.set_weights(w)
    gpu = tiles.CudaAnalogTile(host)
    gpu.set_seed(4)
    x = rng.uniform(-1, 1, (batch, x_size)).astype(np.float32)
    d = (0.3 * rng.standard_normal((batch, d_size))).astype(np.float32)
    x[3] = 0.0
    d[5, :7] = 0.0
    for lr in (0.01, 0.02):
        gpu.set_learning_rate(lr)
        orc.set_learning_rate(lr)
        gpu.update(cuda(x), cuda(d), False, False, False, False)
        xw, dw, bl = (t.numpy() for t in gpu.get_update_words(batch))
        bl_orc, a_orc, b_orc = orc.update_bl_ab(x, d)
        assert np.array_equal(bl, bl_orc)
        a_gpu, b_gpu = (t.numpy() for t in gpu.get_update_ab(batch))
        assert np.array_equal(a_gpu, a_orc) and np.array_equal(b_gpu, b_orc)  # probability scales, bit for bit
        _word_invariants(xw, x, bl)
        _word_invariants(dw, d, bl)
        assert (xw >> 1).any() and (dw >> 1).any()
        orc.update_with_words(xw, dw, bl)
        assert np.abs(gpu.get_weights().numpy() - orc.get_weights()).max() <= TOL
    assert np.abs(orc.get_weights() - np.clip(w, orc.get_hidden()[1], orc.get_hidden()[0])).max() > 1e-3


@pytest.mark.parametrize("desired_bl", [1, 2, 3, 4, 7, 8, 13])
@pytest.mark.parametrize("device", ["constant", "soft"])
def test_short_bit_lines_words_drive_the_oracle_to_the_same_weights(gpu_device, device, desired_bl):
    """Fixed bit-line lengths around the limits of the update kernel's pulse loops (counts kept in 2 or 3
    bit slices up to 3 / 7 slots, packed-word gathers beyond), with pulse probabilities high enough that a
    sample often has several coincidences; odd sizes leave idle lanes and a ragged last chunk."""
    rng = np.random.default_rng(100 + desired_bl)
    x_size, d_size, batch = 70, 37, 45
    meta = make_meta(desired_bl=desired_bl, update_management=False, update_bl_management=False)
    kw = dict(dw_min=0.002, dw_min_std=0.0, construction_seed=5, enforce_consistency=True)
    dev = constant_step(**kw) if device == "constant" else soft_bounds(**kw)
    host, orc, _ = build_pair(meta, dev, x_size, d_size, gpu=False)
    w = rng.uniform(-0.5, 0.5, (d_size, x_size)).astype(np.float32)
    host.set_weights(torch.from_numpy(w))
    orc.set_weights(w)
    gpu = tiles.CudaAnalogTile(host)
    gpu.set_seed(11)
    x = rng.uniform(-1, 1, (batch, x_size)).astype(np.float32)
    d = rng.uniform(-1, 1, (batch, d_size)).astype(np.float32)
    lr = 0.002 * desired_bl * 0.64  # A = B = sqrt(lr / (dw_min BL)) = 0.8
    counts_seen = set()
    for sign in (1.0, -1.0):
        gpu.set_learning_rate(sign * lr)
        orc.set_learning_rate(sign * lr)
        gpu.update(cuda(x), cuda(d), False, False, False, False)
        xw, dw, bl = (t.numpy() for t in gpu.get_update_words(batch))
        assert np.all(bl == desired_bl)
        n = np.bitwise_count((xw[:, None, :].view(np.uint32) & dw[:, :, None].view(np.uint32)) >> 1)
        counts_seen |= set(np.unique(n).tolist())
        orc.update_with_words(xw, dw, bl)
        assert np.abs(gpu.get_weights().numpy() - orc.get_weights()).max() <= TOL
    assert max(counts_seen) >= min(desired_bl, 3)  # samples with several coincidences did occur


@pytest.mark.parametrize("device", ["constant", "soft"])
def test_crossed_and_tight_bounds_clip_like_the_reference_order(gpu_device, device):
    """ConstantStep clips min(w_max) then max(w_min), LinearStep max(w_min) then min(w_max): with hidden
    parameters whose bounds are crossed (w_min > w_max) or equal, the order decides the result."""
    rng = np.random.default_rng(77)
    x_size, d_size, batch = 64, 32, 24
    meta = make_meta(desired_bl=5, update_management=False, update_bl_management=False)
    kw = dict(dw_min=0.01, dw_min_std=0.0, construction_seed=3, enforce_consistency=True)
    dev = constant_step(**kw) if device == "constant" else soft_bounds(**kw)
    host, orc, _ = build_pair(meta, dev, x_size, d_size, gpu=False)
    hidden = host.get_hidden_parameters()
    hi, lo = hidden[0].clone(), hidden[1].clone()
    hidden[0][:, ::3] = lo[:, ::3] * 0.5   # upper bound below zero ...
    hidden[1][:, ::3] = hi[:, ::3] * 0.5   # ... lower bound above zero: crossed
    hidden[1][:, 1::3] = hidden[0][:, 1::3]  # equal bounds
    host.set_hidden_parameters(hidden)
    orc.set_hidden(hidden.numpy())
    w = rng.uniform(-0.1, 0.1, (d_size, x_size)).astype(np.float32)
    host.set_weights(torch.from_numpy(w))
    gpu = tiles.CudaAnalogTile(host)
    gpu.set_seed(2)
    orc.set_weights(gpu.get_weights().numpy())  # both start from what the library's set_weights made of w
    lr = 0.01 * 5 * 0.81
    gpu.set_learning_rate(lr)
    orc.set_learning_rate(lr)
    x = rng.uniform(-1, 1, (batch, x_size)).astype(np.float32)
    d = rng.uniform(-1, 1, (batch, d_size)).astype(np.float32)
    gpu.update(cuda(x), cuda(d), False, False, False, False)
    xw, dw, bl = (t.numpy() for t in gpu.get_update_words(batch))
    orc.update_with_words(xw, dw, bl)
    got, want = gpu.get_weights().numpy(), orc.get_weights()
    assert np.abs(got - want).max() <= TOL
    assert np.abs(want - w).max() > 1e-3


def test_pulse_probabilities_saturate(gpu_device):
    """|v| * scale >= 1 gives all BL pulses, 0 gives none (the reference's bit-line maker test protocol)."""
    x_size, d_size, batch = 64, 64, 8
    meta = make_meta(desired_bl=31, update_management=False, update_bl_management=False)
    dev = constant_step(dw_min=0.001, dw_min_std=0.0, dw_min_dtod=0.0, construction_seed=1)
    host, orc, gpu = build_pair(meta, dev, x_size, d_size)
    lr = 0.031 * 4.0  # A = B = sqrt(lr / (dw_min * BL)) = 2
    gpu.set_learning_rate(lr)
    x = np.zeros((batch, x_size), np.float32)
    d = np.zeros((batch, d_size), np.float32)
    x[:, ::2] = 0.6
    x[:, 1::4] = -0.75
    d[:, ::2] = -1.0
    gpu.update(cuda(x), cuda(d), False)
    xw, dw, bl = (t.numpy().astype(np.int64) & 0xFFFFFFFF for t in gpu.get_update_words(batch))
    assert np.all(bl == 31)
    full = 0xFFFFFFFE
    assert np.all(xw[:, ::2] == full) and np.all(xw[:, 1::4] == (full | 1)) and np.all(xw[:, 3::4] == 0)
    assert np.all(dw[:, ::2] == (full | 1)) and np.all(dw[:, 1::2] == 0)


@pytest.mark.parametrize("device", ["constant", "soft"])
def test_deterministic_implicit_counts_are_bit_exact(gpu_device, device):
    rng = np.random.default_rng(8)
    x_size, d_size, batch = 70, 50, 24
    meta = make_meta(desired_bl=31, pulse_type=dv.PulseType.DeterministicImplicit, x_res_implicit=1 / 20.0,
                     d_res_implicit=1 / 30.0)
    kw = dict(dw_min=0.001, dw_min_std=0.0, construction_seed=5, enforce_consistency=True)
    dev = constant_step(**kw) if device == "constant" else soft_bounds(**kw)
    host, orc, _ = build_pair(meta, dev, x_size, d_size, gpu=False)
    w = rng.uniform(-0.4, 0.4, (d_size, x_size)).astype(np.float32)
    host.set_weights(torch.from_numpy(w))
    orc.set_weights(w)
    gpu = tiles.CudaAnalogTile(host)
    x = rng.uniform(-1, 1, (batch, x_size)).astype(np.float32)
    d = (0.2 * rng.standard_normal((batch, d_size))).astype(np.float32)
    gpu.set_learning_rate(0.02)
    orc.set_learning_rate(0.02)
    for _ in range(2):
        gpu.update(cuda(x), cuda(d), False)
        counts = gpu.get_implicit_counts(batch).numpy()
        assert np.array_equal(counts, orc.implicit_counts(x, d))
        assert np.abs(counts).max() >= 2
        orc.update(x, d)
        assert np.abs(gpu.get_weights().numpy() - orc.get_weights()).max() <= TOL


NM, BM = dv.NoiseManagementType, dv.BoundManagementType


@pytest.mark.parametrize("nm,nm_thres", [(NM.NONE, 0.0), (NM.AbsMax, 0.0), (NM.AbsMax, 0.5), (NM.Max, 0.0),
                                         (NM.Constant, 2.0), (NM.AbsMaxNPSum, 0.0)])
@pytest.mark.parametrize("bm", [BM.NONE, BM.Iterative, BM.IterativeWorstCase])
def test_forward_noise_and_bound_management_modes_bit_exact(gpu_device, nm, nm_thres, bm):
    """Every noise / bound management mode, with input / output asymmetry, an output scale and the
    negative-bound test switched off, in the exact-arithmetic setting (inputs and weights on binary grids)."""
    rng = np.random.default_rng(17)
    x_size, d_size, batch = 256, 96, 40
    f_io = noise_free_io(inp_res=1 / 128.0, out_res=1 / 512.0, bound_management=bm, noise_management=nm,
                         nm_thres=nm_thres, inp_asymmetry=0.25, out_asymmetry=0.5, out_scale=2.0, out_bound=4.0,
                         bm_test_negative_bound=False)
    b_io = noise_free_io(inp_res=1 / 128.0, out_res=1 / 512.0, noise_management=nm, nm_thres=nm_thres,
                         inp_asymmetry=0.25, out_scale=0.5)
    meta = make_meta(f_io, b_io)
    dev = constant_step(w_max_dtod=0.0, w_min_dtod=0.0, w_max=1.0, w_min=-1.0, construction_seed=7)
    host, orc, _ = build_pair(meta, dev, x_size, d_size, gpu=False)
    w = (rng.integers(-38, 39, (d_size, x_size)) / 64.0).astype(np.float32)
    host.set_weights(torch.from_numpy(w))
    orc.set_weights(w)
    gpu = tiles.CudaAnalogTile(host)
    x = (rng.integers(-64, 65, (batch, x_size)) / 64.0).astype(np.float32)
    x[1] = 0.0
    x[2] = -np.abs(x[2])  # Max noise management sees no positive entry
    y_gpu = gpu.forward(cuda(x), False, False, False, False, False).cpu().numpy()
    assert np.array_equal(y_gpu, orc.forward(x))
    if bm != BM.NONE:
        assert np.array_equal(gpu.get_bm_rounds(batch).numpy(), orc.bm_rounds(batch))
        if nm != NM.AbsMaxNPSum:  # the NP-sum scale is made so that the first round fits
            assert orc.bm_rounds(batch).max() >= 2
    d = (rng.integers(-64, 65, (batch, d_size)) / 64.0).astype(np.float32)
    assert np.array_equal(gpu.backward(cuda(d), False, False, False, False).cpu().numpy(), orc.backward(d))


def test_linear_step_additive_noise_device_and_negative_learning_rate(gpu_device):
    """LinearStep (not SoftBounds) with additive-noise form and mean-bound reference slopes, positive and
    negative learning rate: GPU words -> oracle device loop, 1e-5."""
    rng = np.random.default_rng(31)
    x_size, d_size, batch = 80, 48, 20
    dev = dv.LinearStepResistiveDeviceParameter()
    for k, v in dict(gamma_up=0.4, gamma_down=0.2, gamma_up_dtod=0.05, gamma_down_dtod=0.05, mult_noise=False,
                     dw_min=0.002, dw_min_std=0.0, construction_seed=9, enforce_consistency=True).items():
        setattr(dev, k, v)
    meta = make_meta(desired_bl=20)
    host, orc, _ = build_pair(meta, dev, x_size, d_size, gpu=False)
    w = rng.uniform(-0.4, 0.4, (d_size, x_size)).astype(np.float32)
    host.set_weights(torch.from_numpy(w))
    orc.set_weights(w)
    gpu = tiles.CudaAnalogTile(host)
    x = rng.uniform(-1, 1, (batch, x_size)).astype(np.float32)
    d = (0.2 * rng.standard_normal((batch, d_size))).astype(np.float32)
    before = orc.get_weights()
    for lr in (0.02, -0.02):
        gpu.set_learning_rate(lr)
        orc.set_learning_rate(lr)
        gpu.update(cuda(x), cuda(d), False, False, False, False)
        xw, dw, bl = (t.numpy() for t in gpu.get_update_words(batch))
        assert bl.max() <= 20
        orc.update_with_words(xw, dw, bl)
        assert np.abs(gpu.get_weights().numpy() - orc.get_weights()).max() <= TOL
    # the two calls push in opposite directions
    assert np.abs(orc.get_weights() - before).mean() < 0.5 * 0.002 * 20


@pytest.mark.parametrize("x_trans,d_trans,bias", [(True, True, False), (False, False, True), (True, False, True)])
def test_update_layouts_and_bias_column(gpu_device, x_trans, d_trans, bias):
    rng = np.random.default_rng(13)
    x_size, d_size, batch = 65, 33, 17
    meta = make_meta(desired_bl=31, pulse_type=dv.PulseType.DeterministicImplicit)
    dev = constant_step(dw_min=0.001, dw_min_std=0.0, construction_seed=5, enforce_consistency=True)
    host, orc, _ = build_pair(meta, dev, x_size, d_size, gpu=False)
    gpu = tiles.CudaAnalogTile(host)
    xs = x_size - int(bias)
    x = rng.uniform(-1, 1, (xs, batch) if x_trans else (batch, xs)).astype(np.float32)
    d = (0.3 * rng.standard_normal((d_size, batch) if d_trans else (batch, d_size))).astype(np.float32)
    gpu.set_learning_rate(0.05)
    orc.set_learning_rate(0.05)
    gpu.update(cuda(x), cuda(d), bias, x_trans, d_trans, False)
    orc.update(x, d, bias, x_trans, d_trans)
    assert np.abs(gpu.get_weights().numpy() - orc.get_weights()).max() <= TOL
    assert np.abs(orc.get_weights()).max() > 5e-3
    if bias:  # the bias column saw a constant input of one
        assert np.abs(orc.get_weights()[:, -1]).mean() > np.abs(orc.get_weights()[:, :-1]).mean()


@pytest.mark.parametrize("direction", ["forward", "backward"])
def test_output_noise_of_the_large_tile_kernel_is_standard_normal_and_unshared(gpu_device, direction):
    """Batch 4096 on a 1024 x 1024 tile runs on the 128 x 128 workgroup tiles.  With no ADC quantization and no bound
    management the difference to the same pass without output noise, divided by out_noise times the per-sample
    output factor (the abs-max of the input), must be standard normal and uncorrelated between samples, outputs
    and workgroup tiles."""
    rng = np.random.default_rng(21)
    size, batch, sigma = 1024, 4096, 0.06

    def tile(noise):
        io = noise_free_io(inp_res=1 / 126.0, out_res=-1.0, out_bound=1e6, out_noise=noise,
                           noise_management=dv.NoiseManagementType.AbsMax)
        meta = make_meta(io, io)
        dev = constant_step(w_max_dtod=0.0, w_min_dtod=0.0, w_max=1.0, w_min=-1.0, construction_seed=3)
        host = meta.create_array(size, size, dev)
        host.set_weights(torch.from_numpy(w))
        gpu = tiles.CudaAnalogTile(host)
        gpu.set_seed(77)
        return gpu

    w = rng.uniform(-0.3, 0.3, (size, size)).astype(np.float32)
    v = cuda(rng.uniform(-1, 1, (batch, size)).astype(np.float32))
    noisy, clean = tile(sigma), tile(0.0)
    if direction == "forward":
        y, y0 = noisy.forward(v, False, False, False, False, False), clean.forward(v, False, False, False, False, False)
    else:
        y, y0 = noisy.backward(v, False, False, False, False), clean.backward(v, False, False, False, False)
    z = ((y - y0) / (sigma * v.abs().amax(dim=1, keepdim=True))).double()
    n = z.numel()
    assert abs(z.mean().item()) < 4 / np.sqrt(n)
    assert abs(z.var().item() - 1) < 5 * np.sqrt(2 / n) + 2e-3          # fp32 rounding of y - y0 adds a little
    assert abs((z ** 4).mean().item() - 3) < 0.05
    zc = z - z.mean()
    for a, b in ((zc[:, :-1], zc[:, 1:]), (zc[:-1], zc[1:]), (zc[:, :128], zc[:, 128:256]), (zc[:128], zc[128:256]),
                 (zc[:, :512], zc[:, 512:])):
        assert abs((a * b).mean().item()) < 5 / np.sqrt(a.numel())


@pytest.mark.parametrize("x_size,d_size,bm", [(800, 64, BM.Iterative), (64, 800, BM.NONE)])
def test_operands_beyond_two_to_the_31_elements(gpu_device, x_size, d_size, bm):
    """Three million samples: the input (or output) matrix and the quantized-input scratch hold more than 2^31
    elements, so every row offset needs 64-bit arithmetic.  Exact-arithmetic setting; the oracle checks the first, middle
    and last rows and 200 random ones (rows are independent)."""
    batch = 3_000_000
    rng = np.random.default_rng(1)
    f_io = noise_free_io(inp_res=1 / 128.0, out_res=1 / 512.0, noise_management=NM.AbsMax, bound_management=bm, out_bound=4.0)
    b_io = noise_free_io(inp_res=1 / 128.0, out_res=1 / 512.0, noise_management=NM.AbsMax)
    dev = constant_step(w_max_dtod=0.0, w_min_dtod=0.0, w_max=1.0, w_min=-1.0, construction_seed=7)
    host, orc, _ = build_pair(make_meta(f_io, b_io), dev, x_size, d_size, gpu=False)
    w = (rng.integers(-38, 39, (d_size, x_size)) / 64.0).astype(np.float32)
    host.set_weights(torch.from_numpy(w))
    orc.set_weights(w)
    gpu = tiles.CudaAnalogTile(host)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(3)
    rows = np.concatenate([np.arange(0, 40), np.arange(batch // 2 - 20, batch // 2 + 20), np.arange(batch - 40, batch),
                           rng.integers(0, batch, 200)])
    pick = torch.from_numpy(rows).cuda()
    x = torch.randint(-64, 65, (batch, x_size), device="cuda", generator=gen).float() / 64.0
    assert max(x.numel(), batch * d_size) > 2 ** 31
    y = gpu.forward(x)
    assert np.array_equal(y[pick].cpu().numpy(), orc.forward(x[pick].cpu().numpy()))
    if bm != BM.NONE:
        rounds = gpu.get_bm_rounds(batch).numpy()
        assert np.array_equal(rounds[rows], orc.bm_rounds(len(rows))) and rounds.max() > 1
    del x, y
    d = torch.randint(-64, 65, (batch, d_size), device="cuda", generator=gen).float() / 64.0
    gx = gpu.backward(d)
    assert np.array_equal(gx[pick].cpu().numpy(), orc.backward(d[pick].cpu().numpy()))


@pytest.mark.parametrize("x_size,d_size,batch", [(33, 70000, 3), (70000, 33, 3), (5000, 5000, 2), (1, 1, 1), (1, 70000, 1),
                                                 (70000, 1, 5)])
def test_extreme_tile_shapes(gpu_device, x_size, d_size, batch):
    """One-line tiles, a single cross-point, more than 65535 rows or columns, 25 million cross-points: forward and
    backward bit-exact (exact-arithmetic setting), the stochastic update through the GPU's words to 1e-5, and the
    elementwise maintenance kernels run."""
    rng = np.random.default_rng(1)
    f_io = noise_free_io(inp_res=1 / 128.0, out_res=1 / 512.0, noise_management=NM.AbsMax, bound_management=BM.Iterative,
                         out_bound=4.0)
    b_io = noise_free_io(inp_res=1 / 128.0, out_res=1 / 512.0, noise_management=NM.AbsMax)
    dev = constant_step(w_max_dtod=0.0, w_min_dtod=0.0, w_max=1.0, w_min=-1.0, dw_min_std=0.0, construction_seed=7)
    host, orc, _ = build_pair(make_meta(f_io, b_io, desired_bl=31), dev, x_size, d_size, gpu=False)
    w = (rng.integers(-38, 39, (d_size, x_size)) / 64.0).astype(np.float32)
    host.set_weights(torch.from_numpy(w))
    orc.set_weights(w)
    gpu = tiles.CudaAnalogTile(host)
    x = (rng.integers(-64, 65, (batch, x_size)) / 64.0).astype(np.float32)
    d = (rng.integers(-64, 65, (batch, d_size)) / 64.0).astype(np.float32)
    assert np.array_equal(gpu.forward(cuda(x)).cpu().numpy(), orc.forward(x))
    assert np.array_equal(gpu.get_bm_rounds(batch).numpy(), orc.bm_rounds(batch))
    assert np.array_equal(gpu.backward(cuda(d)).cpu().numpy(), orc.backward(d))
    gpu.set_learning_rate(0.05)
    orc.set_learning_rate(0.05)
    gpu.update(cuda(x), cuda(0.2 * d), False)
    xw, dw, bl = (t.numpy() for t in gpu.get_update_words(batch))
    orc.update_with_words(xw, dw, bl)
    assert np.abs(gpu.get_weights().numpy() - orc.get_weights()).max() <= TOL
    if x_size * d_size > 1:
        assert np.abs(orc.get_weights() - w).max() > 0
    gpu.clip_weights(tiles.WeightClipParameter(type=tiles.WeightClipType.FIXED_VALUE, fixed_value=0.25))
    assert float(gpu.get_weights().abs().max()) <= 0.25


def test_empty_batches_do_nothing(gpu_device):
    """A batch of zero samples: empty outputs, untouched weights and random streams (the reference's loops over the
    samples run zero times)."""
    meta, dev = config1(noise=False)
    host, _orc, gpu = build_pair(meta, dev, 40, 24)
    gpu.set_learning_rate(0.05)
    w = gpu.get_weights()
    state = gpu.dump_extra()
    assert tuple(gpu.forward(torch.empty(0, 40, device="cuda")).shape) == (0, 24)
    assert tuple(gpu.backward(torch.empty(0, 24, device="cuda")).shape) == (0, 40)
    assert tuple(gpu.forward(torch.empty(40, 0, device="cuda"), False, True, True).shape) == (24, 0)
    gpu.update(torch.empty(0, 40, device="cuda"), torch.empty(0, 24, device="cuda"), False)
    assert torch.equal(gpu.get_weights(), w) and gpu.dump_extra() == state
    x = torch.rand(3, 40, device="cuda")
    assert tuple(gpu.forward(x).shape) == (3, 24)                 # and the tile works on as before


def test_none_with_device_update_is_the_outer_product_inside_the_bounds(gpu_device):
    """PulseType NoneWithDevice: per sample the floating-point outer product, then the device bounds (no pulses, no step
    sizes).  The clipping after every sample makes the result depend on the order of the batch."""
    rng = np.random.default_rng(21)
    for x_size, d_size, batch, bias, trans in ((70, 45, 9, False, False), (257, 33, 40, True, True), (1, 1, 3, False, False)):
        meta = make_meta(noise_free_io(), noise_free_io(), pulse_type=dv.PulseType.NoneWithDevice)
        dev = soft_bounds(construction_seed=3)
        host, orc, _ = build_pair(meta, dev, x_size, d_size, gpu=False)
        w = rng.uniform(-0.3, 0.3, (d_size, x_size)).astype(np.float32)
        host.set_weights(torch.from_numpy(w))
        orc.set_weights(host.get_weights().numpy())
        gpu = tiles.CudaAnalogTile(host)
        xs = x_size - int(bias)
        x = rng.uniform(-1, 1, (xs, batch) if trans else (batch, xs)).astype(np.float32)
        d = rng.normal(0, 0.5, (d_size, batch) if trans else (batch, d_size)).astype(np.float32)
        hidden = gpu.get_hidden_parameters().numpy()
        for lr in (1.0, -0.5):
            gpu.set_learning_rate(lr)
            orc.set_learning_rate(lr)
            before = gpu.get_weights().numpy()
            gpu.update(cuda(x), cuda(d), bias, trans, trans)
            orc.update(x, d, bias, trans, trans)
            got = gpu.get_weights().numpy()
            assert np.array_equal(got, orc.get_weights())            # the same float operations in the same order
            assert (got <= hidden[0]).all() and (got >= hidden[1]).all()
            if x_size > 1:
                at_bound = (got == hidden[0]) | (got == hidden[1])
                assert 0.01 < at_bound.mean() < 0.9
                xb = (x.T if trans else x)
                xb = np.concatenate([xb, np.ones((batch, 1), np.float32)], 1) if bias else xb
                once = np.clip(before - lr * (d if trans else d.T) @ xb, hidden[1], hidden[0])
                assert np.abs(got - once).max() > 1e-3                # clipping once at the end is not the same thing


def test_stochastic_pulse_type_is_the_compressed_one(gpu_device):
    """PulseType Stochastic (separate lists for positive and negative inputs in the reference's CPU code) gives every
    cross-point the pulses of StochasticCompressed: same seed, same weights."""
    rng = np.random.default_rng(4)
    x = rng.uniform(-1, 1, (20, 50)).astype(np.float32)
    d = rng.normal(0, 0.3, (20, 30)).astype(np.float32)
    results = []
    for pulse_type in (dv.PulseType.Stochastic, dv.PulseType.StochasticCompressed):
        meta = make_meta(noise_free_io(), noise_free_io(), pulse_type=pulse_type, desired_bl=31)
        host, _orc, gpu = build_pair(meta, soft_bounds(construction_seed=2), 50, 30)
        gpu.set_learning_rate(0.05)
        gpu.set_seed(77)
        gpu.update(cuda(x), cuda(d), False)
        results.append(gpu.get_weights())
    assert torch.equal(results[0], results[1]) and not torch.equal(results[0], torch.zeros_like(results[0]))
