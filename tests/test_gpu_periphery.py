"""GPU parity of the per-line periphery terms (voltage offsets, series resistance, output non-linearity with slope
calibration, per-line output noise) against the CPU restatement, through the Python mirror over the C ABI.  The
per-line values are read from the tile's extra state and given to the oracle, so both compute with the same lines."""
import copy

import numpy as np
import pytest
import torch

from aihwkit_amd.rpu_base import devices as dv
from aihwkit_amd.rpu_base import tiles
from helpers import build_pair, constant_step, io_params, make_meta

pytestmark = pytest.mark.gpu
F = np.float32
KINDS = ("v_offset", "out_nonlinearity", "out_noise_values")


def lines_of(tile, direction, kind):
    """The per-line values of one direction ('fwd' / 'bwd') from the extra state."""
    state = tile.dump_extra()
    prefix = f"rpu.{direction}.{kind}_"
    n = sum(1 for k in state if k.startswith(prefix))
    return np.array([state[f"{prefix}{i}.bits"] for i in range(n)], dtype=np.uint32).view(F)


def pair(x_size, d_size, seed=0, construction_seed=7, **io):
    base = dict(out_noise=0.0, inp_noise=0.0, out_res=-1.0)
    base.update(io)
    meta = make_meta(io_params(**base), io_params(**base))
    dev = constant_step(w_max=1.0, w_min=-1.0, w_max_dtod=0.0, w_min_dtod=0.0, construction_seed=construction_seed)
    host, orc, _gpu = build_pair(meta, dev, x_size, d_size, gpu=False)
    w = np.random.default_rng(seed).uniform(-0.6, 0.6, (d_size, x_size)).astype(F)
    host.set_weights(torch.from_numpy(w))
    orc.set_weights(w)
    gpu = tiles.CudaAnalogTile(host)
    for d, direction in enumerate(("fwd", "bwd")):
        for k, kind in enumerate(KINDS):
            v = lines_of(gpu, direction, kind)
            assert v.size == orc.get_lines(d, k).size
            if v.size:
                orc.set_lines(d, k, v)
    return orc, gpu, w


PNS = dv.AnalogMVType.PosNegSeparate
PNSD = dv.AnalogMVType.PosNegSeparateDigitalSum

CASES = {
    "digital_sum_ir_drop": dict(mv_type=PNSD, ir_drop=1.0),
    "digital_sum_series_resistance": dict(mv_type=PNSD, r_series=0.03, v_offset_std=0.1, v_offset_w_min=-1.0),
    "digital_sum_everything": dict(mv_type=PNSD, v_offset_std=0.1, r_series=0.01, out_nonlinearity=0.5,
                                   out_nonlinearity_std=0.2, ir_drop=1.0, out_asymmetry=0.05),
    "separate_passes_ir_drop": dict(mv_type=PNS, ir_drop=1.0),
    "separate_passes_series_resistance": dict(mv_type=PNS, r_series=0.03, v_offset_std=0.1, v_offset_w_min=-1.0),
    "separate_passes_everything": dict(mv_type=PNS, v_offset_std=0.1, r_series=0.01, out_nonlinearity=0.5,
                                       out_nonlinearity_std=0.2, ir_drop=1.0, out_asymmetry=0.05),
    "offsets": dict(v_offset_std=0.15),
    "offsets_reference_line": dict(v_offset_std=0.15, v_offset_w_min=-1.0),
    "series_resistance": dict(r_series=0.02, slope_calibration=0.4),
    "series_resistance_capped": dict(r_series=0.05, r_series_max_total=0.2, v_offset_std=0.1, v_offset_w_min=-0.6),
    "nonlinearity": dict(out_nonlinearity=0.8, out_nonlinearity_std=0.3),
    "nonlinearity_uncalibrated": dict(out_nonlinearity=0.8, out_nonlinearity_std=0.3, slope_calibration=0.0, out_asymmetry=0.1),
    "everything": dict(v_offset_std=0.1, v_offset_w_min=-1.0, r_series=0.01, out_nonlinearity=0.5, out_nonlinearity_std=0.2,
                       ir_drop=1.0, out_asymmetry=0.05),
}


@pytest.mark.parametrize("case", sorted(CASES))
@pytest.mark.parametrize("shape", [(37, 23, 50), (300, 200, 96), (129, 10, 33)])
def test_line_terms_with_quantized_inputs_and_bound_management(gpu_device, shape, case):
    x_size, d_size, batch = shape
    rng = np.random.default_rng(1)
    w = np.random.default_rng(0).uniform(-0.6, 0.6, (d_size, x_size)).astype(F)   # the weights `pair` sets
    x = rng.uniform(-1, 1, (batch, x_size)).astype(F)
    x[3] = 0.0                                                    # a zero sample short-cuts to zero
    x[5] *= 0.01
    x[7] = np.sign(w[0])                                          # one output far beyond the bound: many rounds
    d = rng.normal(0, 0.5, (batch, d_size)).astype(F)
    scaled = x / np.maximum(np.abs(x).max(axis=1, keepdims=True), 1e-9)
    out_bound = float(np.median(np.abs(scaled @ w.T).max(axis=1)))
    io = dict(CASES[case], out_bound=out_bound, noise_management=dv.NoiseManagementType.AbsMax,
              bound_management=dv.BoundManagementType.Iterative)
    if "ir_drop" in io:
        io["ir_drop_g_ratio"] = x_size * (0.3 * 0.5 * x_size) / 0.5
    orc, gpu, _w = pair(x_size, d_size, **io)
    plain_orc, _g, _w = pair(x_size, d_size, out_bound=out_bound, noise_management=dv.NoiseManagementType.AbsMax,
                             bound_management=dv.BoundManagementType.Iterative)
    want = orc.forward(x)
    got = gpu.forward(torch.from_numpy(x).cuda()).cpu().numpy()
    rounds = orc.bm_rounds(batch)
    # an uncalibrated non-linearity, or a series resistance on the large current of a pass, compresses the sums below
    # the bound; every other case needs a second round for some samples
    need = 1 if ("uncalibrated" in case or case.endswith("passes_series_resistance")) else 2
    assert rounds.max() >= need and len(set(rounds[rounds > 0])) >= need
    assert np.array_equal(gpu.get_bm_rounds(batch).numpy(), rounds)
    scale = np.abs(want).max()
    assert np.abs(got - want).max() <= 1e-5 * scale
    assert np.abs(want - plain_orc.forward(x)).max() > 1e-2 * scale      # the terms are far above the tolerance
    assert not got[3].any()
    want_b = orc.backward(d)
    got_b = gpu.backward(torch.from_numpy(d).cuda()).cpu().numpy()
    assert np.abs(got_b - want_b).max() <= 1e-5 * np.abs(want_b).max()
    assert np.abs(want_b - plain_orc.backward(d)).max() > 1e-3 * np.abs(want_b).max()
    got_t = gpu.forward(torch.from_numpy(np.ascontiguousarray(x.T)).cuda(), False, True, True).cpu().numpy()
    assert np.abs(got_t.T - want).max() <= 1e-5 * scale


def test_line_terms_with_a_bias_column_and_adc_quantization(gpu_device):
    rng = np.random.default_rng(2)
    x = rng.uniform(-1, 1, (40, 64)).astype(F)
    io = dict(v_offset_std=0.1, v_offset_w_min=-1.0, r_series=0.01, out_nonlinearity=0.5, out_nonlinearity_std=0.2,
              out_res=1.0 / 510, out_bound=12.0, noise_management=dv.NoiseManagementType.AbsMax,
              bound_management=dv.BoundManagementType.Iterative)
    orc, gpu, _w = pair(65, 31, **io)
    want = orc.forward(x, bias=True)
    got = gpu.forward(torch.from_numpy(x).cuda(), True).cpu().numpy()
    # an output may sit on the other side of an ADC rounding edge: every mismatch is one step and they are rare
    step = 24.0 / 510
    diff = np.abs(got - want)
    off = diff > 1e-5
    assert off.mean() < 5e-3 and np.allclose(diff[off], step, rtol=1e-3)
    d = rng.normal(0, 0.5, (40, 31)).astype(F)
    want_b = orc.backward(d, bias=True)
    got_b = gpu.backward(torch.from_numpy(d).cuda(), True).cpu().numpy()
    diff = np.abs(got_b - want_b) / np.abs(d).max(axis=1, keepdims=True)
    off = diff > 1e-5
    assert off.mean() < 5e-3 and np.allclose(diff[off], step, rtol=1e-3)


def moments_ok(z):
    n = z.size
    return abs(z.mean()) < 4 / np.sqrt(n) and abs(z.std() - 1) < 4 / np.sqrt(2 * n)


def test_per_line_output_noise_and_the_order_of_the_steps(gpu_device):
    rng = np.random.default_rng(3)
    x_size, d_size, batch = 96, 160, 256
    x = rng.uniform(-1, 1, (batch, x_size)).astype(F)
    base = dict(inp_res=-1.0, out_bound=1e6, noise_management=dv.NoiseManagementType.NONE,
                bound_management=dv.BoundManagementType.NONE)
    x64 = x.astype(np.float64)
    # per-line levels |out_noise (1 + out_noise_std xi)|: every output line has its own sigma, forward and backward
    _orc, gpu, w = pair(x_size, d_size, out_noise=0.1, out_noise_std=0.5, **base)
    levels = lines_of(gpu, "fwd", "out_noise_values").astype(np.float64)
    assert levels.size == d_size and levels.std() > 0.03 and abs(levels.mean() / 0.1 - 1) < 4 * 0.5 / np.sqrt(d_size) + 0.01
    y = gpu.forward(torch.from_numpy(x).cuda()).cpu().numpy().astype(np.float64)
    z = (y - x64 @ w.astype(np.float64).T) / levels[None, :]
    assert moments_ok(z) and np.abs(z.std(axis=0) - 1).max() < 5 / np.sqrt(2 * batch)
    d = rng.uniform(-1, 1, (batch, d_size)).astype(F)
    levels_b = lines_of(gpu, "bwd", "out_noise_values").astype(np.float64)
    assert levels_b.size == x_size and not np.array_equal(levels_b[:50], levels[:50])
    gx = gpu.backward(torch.from_numpy(d).cuda()).cpu().numpy().astype(np.float64)
    assert moments_ok((gx - d.astype(np.float64) @ w.astype(np.float64)) / levels_b[None, :])
    # output noise is added after the non-linearity (its sigma is not compressed), weight noise before it
    orc, gpu, w = pair(x_size, d_size, out_noise=0.3, out_nonlinearity=2.0, slope_calibration=0.0, **dict(base, out_bound=4.0))
    nl = lines_of(gpu, "fwd", "out_nonlinearity").astype(np.float64)
    np.testing.assert_allclose(nl, np.full(d_size, 0.5), rtol=1e-6)
    y = gpu.forward(torch.from_numpy(x).cuda()).cpu().numpy().astype(np.float64)
    clean = x64 @ w.astype(np.float64).T
    assert moments_ok((y - clean / (1 + 0.5 * np.abs(clean))) / 0.3)
    orc, gpu, w = pair(x_size, d_size, w_noise=0.05, w_noise_type=dv.WeightNoiseType.AdditiveConstant, v_offset_std=0.3,
                       **base)
    vo = lines_of(gpu, "fwd", "v_offset").astype(np.float64)
    assert (vo == 0).sum() > d_size // 4 and (vo > 0).sum() > d_size // 4
    y = gpu.forward(torch.from_numpy(x).cuda()).cpu().numpy().astype(np.float64)
    z = (y - clean * (1 - vo)[None, :]) / (0.05 * np.linalg.norm(x64, axis=1))[:, None]
    assert moments_ok(z)                                         # offsets scale the sums, not the noise after them


def test_separate_passes_without_nonlinear_terms_and_their_noise(gpu_device):
    rng = np.random.default_rng(5)
    x_size, d_size, batch = 96, 160, 64
    x = rng.uniform(-1, 1, (batch, x_size)).astype(F)
    d = rng.uniform(-1, 1, (batch, d_size)).astype(F)
    # with nothing non-linear in the inputs the two passes add up to the one pass, quantized inputs and ADC included
    io = dict(out_bound=12.0, noise_management=dv.NoiseManagementType.AbsMax, bound_management=dv.BoundManagementType.Iterative)
    orc, gpu, w = pair(x_size, d_size, mv_type=PNS, **io)
    _o, one, _w = pair(x_size, d_size, **io)
    got = gpu.forward(torch.from_numpy(x).cuda()).cpu().numpy()
    assert np.abs(got - orc.forward(x)).max() <= 1e-5 * np.abs(got).max()
    assert np.abs(got - one.forward(torch.from_numpy(x).cuda()).cpu().numpy()).max() <= 1e-5 * np.abs(got).max()
    got_b = gpu.backward(torch.from_numpy(d).cuda()).cpu().numpy()
    assert np.abs(got_b - orc.backward(d)).max() <= 1e-5 * np.abs(got_b).max()
    # weight noise is drawn per pass (variances add up to the one-pass law); output noise once, for the sum
    base = dict(inp_res=-1.0, out_bound=1e6, noise_management=dv.NoiseManagementType.NONE,
                bound_management=dv.BoundManagementType.NONE)
    x64, w64 = x.astype(np.float64), w.astype(np.float64)
    _o, gpu, _w = pair(x_size, d_size, mv_type=PNS, w_noise=0.05, w_noise_type=dv.WeightNoiseType.AdditiveConstant, **base)
    y = gpu.forward(torch.from_numpy(x).cuda()).cpu().numpy().astype(np.float64)
    assert moments_ok((y - x64 @ w64.T) / (0.05 * np.linalg.norm(x64, axis=1))[:, None])
    _o, gpu, _w = pair(x_size, d_size, mv_type=PNS, w_noise=0.1, w_noise_type=dv.WeightNoiseType.PCMRead, **base)
    y = gpu.forward(torch.from_numpy(x).cuda()).cpu().numpy().astype(np.float64)
    assert moments_ok((y - x64 @ w64.T) / (0.1 * np.sqrt((x64 ** 2) @ np.abs(w64).T)))
    _o, gpu, _w = pair(x_size, d_size, mv_type=PNS, out_noise=0.2, **base)
    y = gpu.forward(torch.from_numpy(x).cuda()).cpu().numpy().astype(np.float64)
    assert moments_ok((y - x64 @ w64.T) / 0.2)


def test_digital_sum_of_separately_converted_passes(gpu_device):
    """PosNegSeparateDigitalSum: each pass goes through the ADC stage on its own (noise, quantization, clipping, bound
    test) and the converted values are added.  (1) With a wide ADC and no quantization it is the analog sum, i.e. the
    one-pass tile.  (2) With the real ADC step every output is the sum of two codes: a multiple of the step, within the
    flips of a rounding edge of the oracle's; the bound test is per pass (the round counts equal the oracle's; with
    random signs a pass carries half the inputs, so samples whose analog sum saturates get by with fewer rounds).
    (3) Output noise is drawn per pass: its variance is twice the one-pass variance."""
    rng = np.random.default_rng(8)
    x_size, d_size, batch = 96, 160, 64
    x = rng.uniform(-1, 1, (batch, x_size)).astype(F)
    d = rng.uniform(-1, 1, (batch, d_size)).astype(F)
    io = dict(out_bound=1e6, noise_management=dv.NoiseManagementType.AbsMax, bound_management=dv.BoundManagementType.Iterative)
    orc, gpu, w = pair(x_size, d_size, mv_type=PNSD, **io)
    _o, one, _w = pair(x_size, d_size, **io)
    got = gpu.forward(torch.from_numpy(x).cuda()).cpu().numpy()
    assert np.abs(got - orc.forward(x)).max() <= 1e-5 * np.abs(got).max()
    assert np.abs(got - one.forward(torch.from_numpy(x).cuda()).cpu().numpy()).max() <= 1e-5 * np.abs(got).max()
    # (2)
    step = 2 * 2.0 / 510
    io = dict(out_bound=2.0, out_res=1.0 / 510, noise_management=dv.NoiseManagementType.AbsMax,
              bound_management=dv.BoundManagementType.Iterative)
    orc, gpu, w = pair(x_size, d_size, mv_type=PNSD, **io)
    _o, analog, _w = pair(x_size, d_size, mv_type=PNS, **io)
    want = orc.forward(x)
    got = gpu.forward(torch.from_numpy(x).cuda()).cpu().numpy()
    rounds = gpu.get_bm_rounds(batch).numpy()
    assert np.array_equal(rounds, orc.bm_rounds(batch))
    analog.forward(torch.from_numpy(x).cuda())
    assert (rounds <= analog.get_bm_rounds(batch).numpy()).all() and rounds.sum() < analog.get_bm_rounds(batch).numpy().sum()
    scale = np.abs(x).max(axis=1, keepdims=True) * 2.0 ** (rounds[:, None] - 1)   # output factor of the last round
    codes = got / (step * scale)
    assert np.abs(codes - np.rint(codes)).max() < 2e-3
    diff = np.abs(got - want) / (step * scale)
    off = diff > 1e-3
    assert off.mean() < 5e-3 and np.allclose(diff[off], 1.0, atol=1e-2)
    want_b = orc.backward(d)
    got_b = gpu.backward(torch.from_numpy(d).cuda()).cpu().numpy()
    diff = np.abs(got_b - want_b) / (step * np.abs(d).max(axis=1, keepdims=True))
    off = diff > 1e-3
    assert off.mean() < 5e-3 and np.allclose(diff[off], 1.0, atol=1e-2)
    # (3)
    base = dict(inp_res=-1.0, out_bound=1e6, noise_management=dv.NoiseManagementType.NONE,
                bound_management=dv.BoundManagementType.NONE)
    _o, gpu, w = pair(x_size, d_size, mv_type=PNSD, out_noise=0.2, **base)
    y = gpu.forward(torch.from_numpy(x).cuda()).cpu().numpy().astype(np.float64)
    assert moments_ok((y - x.astype(np.float64) @ w.astype(np.float64).T) / (0.2 * np.sqrt(2.0)))


def test_read_asymmetry_of_the_negative_pass(gpu_device):
    rng = np.random.default_rng(6)
    for x_size, d_size, batch in ((37, 23, 50), (300, 200, 96)):
        x = rng.uniform(-1, 1, (batch, x_size)).astype(F)
        d = rng.normal(0, 0.5, (batch, d_size)).astype(F)
        io = dict(mv_type=PNS, w_read_asymmetry_dtod=0.3, ir_drop=1.0, ir_drop_g_ratio=x_size * (0.3 * 0.5 * x_size) / 0.5,
                  out_bound=float(0.2 * np.sqrt(x_size)), noise_management=dv.NoiseManagementType.AbsMax,
                  bound_management=dv.BoundManagementType.Iterative)
        orc, gpu, w = pair(x_size, d_size, **io)
        plain, _g, _w = pair(x_size, d_size, **dict(io, w_read_asymmetry_dtod=0.0))
        for direction in (0, 1):
            factors = gpu.get_read_asymmetry(bool(direction)).numpy()
            assert factors.shape == (d_size, x_size) and abs(factors.std() / 0.3 - 1) < 0.1
            orc.set_lines(direction, 3, factors.ravel())
        assert not np.array_equal(gpu.get_read_asymmetry(False).numpy(), gpu.get_read_asymmetry(True).numpy())
        want = orc.forward(x)
        got = gpu.forward(torch.from_numpy(x).cuda()).cpu().numpy()
        assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()
        assert np.array_equal(gpu.get_bm_rounds(batch).numpy(), orc.bm_rounds(batch))
        assert np.abs(want - plain.forward(x)).max() > 1e-2 * np.abs(want).max()
        want_b = orc.backward(d)
        got_b = gpu.backward(torch.from_numpy(d).cuda()).cpu().numpy()
        assert np.abs(got_b - want_b).max() <= 1e-5 * np.abs(want_b).max()
        # factors set from outside: all ones is the tile without asymmetry
        ones = torch.ones(d_size, x_size)
        gpu.set_read_asymmetry(ones, False)
        got1 = gpu.forward(torch.from_numpy(x).cuda()).cpu().numpy()
        assert np.abs(got1 - plain.forward(x)).max() <= 1e-5 * np.abs(got1).max()
        twin = copy.deepcopy(gpu)
        assert np.array_equal(twin.get_read_asymmetry(True).numpy(), gpu.get_read_asymmetry(True).numpy())
    _o, off, _w = pair(8, 8, mv_type=PNS)
    with pytest.raises(RuntimeError, match="No read asymmetry factors"):
        off.get_read_asymmetry(False)


def test_line_values_are_state(gpu_device):
    """They are fixed by the construction seed, travel with copies and the extra state, and can be set."""
    io = dict(v_offset_std=0.2, out_nonlinearity=0.6, out_nonlinearity_std=0.25, out_noise_std=0.5, out_noise=0.0,
              noise_management=dv.NoiseManagementType.NONE, bound_management=dv.BoundManagementType.NONE, inp_res=-1.0,
              out_bound=12.0)
    rng = np.random.default_rng(4)
    x = torch.from_numpy(rng.uniform(-1, 1, (20, 50)).astype(F)).cuda()
    _o, a, _w = pair(50, 30, **io)
    _o, b, _w = pair(50, 30, **io)
    _o, c, _w = pair(50, 30, construction_seed=8, **io)
    for direction, n in (("fwd", 30), ("bwd", 50)):
        for kind in KINDS:
            va, vb, vc = (lines_of(t, direction, kind) for t in (a, b, c))
            assert va.size == n and np.array_equal(va, vb)
            assert not np.array_equal(va, vc) or kind == "out_noise_values"      # out_noise = 0 here: all levels are 0
    ya = a.forward(x).cpu().numpy()
    assert np.array_equal(ya, b.forward(x).cpu().numpy()) and not np.array_equal(ya, c.forward(x).cpu().numpy())
    assert np.array_equal(copy.deepcopy(a).forward(x).cpu().numpy(), ya)
    c.load_extra(a.dump_extra(), True)                            # the lines of another tile
    assert np.array_equal(c.forward(x).cpu().numpy(), ya)
    # set from outside: no offsets, no non-linearity -> the plain product times the calibration factor
    state = a.dump_extra()
    for k in state:
        if "v_offset_" in k or "out_nonlinearity_" in k:
            state[k] = 0
    a.load_extra(state, True)
    w = a.get_weights().numpy()
    np.testing.assert_allclose(a.forward(x).cpu().numpy(), x.cpu().numpy() @ w.T, rtol=1e-5, atol=1e-6)


def test_line_terms_are_refused_where_they_are_not_provided(gpu_device):
    from helpers import soft_bounds, transfer_param
    tr = transfer_param([soft_bounds(), soft_bounds()])
    tr.transfer_forward.mv_type = PNS
    tr.transfer_forward.w_read_asymmetry_dtod = 0.1
    with pytest.raises(Exception, match="not provided for the read of a transfer"):
        make_meta().create_array(8, 8, tr)
    with pytest.raises(Exception, match="AnalogMVType not implemented"):
        pair(8, 8, mv_type=4)                                       # SplitMode
