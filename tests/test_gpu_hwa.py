"""GPU parity of the hardware-aware-training helpers of a tile (weight remapping, weight modifier, device-level
power-law drift, pulse counters) against the numpy restatement, through the Python mirror over the C ABI."""
import numpy as np
import pytest
import torch

import hwa_oracle as ho
from aihwkit_amd.rpu_base import devices as dv
from aihwkit_amd.rpu_base import tiles
from helpers import make_meta, noise_free_io, soft_bounds

pytestmark = pytest.mark.gpu
F = np.float32


def hidden(tile):
    names = tile.get_hidden_parameter_names()
    values = tile.get_hidden_parameters().numpy()
    return {name: values[k] for k, name in enumerate(names)}


def pulsed_tile(x_size=37, d_size=23, pulse_type=dv.PulseType.StochasticCompressed, drift=None, **device):
    meta = make_meta(noise_free_io(), noise_free_io(), pulse_type=pulse_type, desired_bl=31)
    dev = soft_bounds(construction_seed=5, **device)
    for name, value in (drift or {}).items():
        setattr(dev.drift, name, value)
    host = meta.create_array(x_size, d_size, dev)
    rng = np.random.default_rng(0)
    host.set_weights(torch.from_numpy(rng.uniform(-0.5, 0.5, (d_size, x_size)).astype(F)))
    return tiles.CudaAnalogTile(host)


def fp_tile(x_size=37, d_size=23, scale=0.3, weights=None, drift=None):
    meta = dv.FloatingPointTileParameter()
    for name, value in (drift or {}).items():
        setattr(meta.drift, name, value)
    host = meta.create_array(x_size, d_size)
    rng = np.random.default_rng(0)
    w = rng.normal(0.01, scale, (d_size, x_size)).astype(F) if weights is None else np.asarray(weights, dtype=F)
    host.set_weights(torch.from_numpy(w))
    return tiles.CudaFloatingPointTile(host)


def remap_par(kind, **kw):
    par = tiles.WeightRemapParameter()
    par.type = kind
    for name, value in kw.items():
        setattr(par, name, value)
    return par


def modifier_par(kind, **kw):
    par = tiles.WeightModifierParameter()
    par.type = kind
    for name, value in kw.items():
        setattr(par, name, value)
    return par


# ---- remap --------------------------------------------------------------------------------------------------------

def test_remap_golden_vectors_of_the_reference_tests(gpu_device):
    # tests/test_inference_tiles.py:215-275 of the reference
    w = np.array([[0.1, 0.2, 0.3, -0.1], [0.4, 0.5, 0.6, -0.3]], dtype=F)
    tile = fp_tile(4, 2, weights=w)
    scales = torch.ones(2, device="cuda")
    assert tile.remap_weights(remap_par(tiles.WeightRemapType.LayerwiseSymmetric), scales) is scales
    np.testing.assert_allclose(tile.get_weights().numpy(), w / F(0.6), rtol=1e-6)
    np.testing.assert_allclose(scales.cpu().numpy(), [0.6, 0.6], rtol=1e-6)
    w = np.array([[-0.7, 0.2, 0.3, -0.1], [0.4, 0.5, 0.6, -0.3]], dtype=F)
    tile = fp_tile(4, 2, weights=w)
    scales = torch.ones(2, device="cuda")
    tile.remap_weights(remap_par(tiles.WeightRemapType.ChannelwiseSymmetric), scales)
    np.testing.assert_allclose(scales.cpu().numpy(), [0.7, 0.6], rtol=1e-6)
    np.testing.assert_allclose(tile.get_weights().numpy(), w / np.array([[0.7], [0.6]], dtype=F), rtol=1e-6)


@pytest.mark.parametrize("shape", [(37, 23), (1000, 300)])
def test_remap_against_the_oracle(gpu_device, shape):
    x_size, d_size = shape
    rng = np.random.default_rng(3)
    cases = [
        (tiles.WeightRemapType.LayerwiseSymmetric, dict(remapped_wmax=0.8)),
        (tiles.WeightRemapType.ChannelwiseSymmetric, dict()),
        (tiles.WeightRemapType.ChannelwiseSymmetric, dict(remapped_wmax=0.7)),
        (tiles.WeightRemapType.ChannelwiseSymmetric, dict(max_scale_range=1.5)),
        (tiles.WeightRemapType.ChannelwiseSymmetric, dict(max_scale_range=1.3, max_scale_ref=1.1)),
        (tiles.WeightRemapType.ChannelwiseNorm, dict(row_norm=2.0, clip_if=False)),
        (tiles.WeightRemapType.ChannelwiseNorm, dict(row_norm=2.0, clip_if=True)),
        (tiles.WeightRemapType.NONE, dict()),
    ]
    for kind, kw in cases:
        tile = fp_tile(x_size, d_size)
        w = tile.get_weights().numpy()
        w[3] = 0.0
        tile.set_weights(torch.from_numpy(w))
        s0 = rng.uniform(0.5, 2.0, d_size).astype(F)
        scales = torch.from_numpy(s0).cuda()
        tile.remap_weights(remap_par(kind, **kw), scales)
        want_w, want_s = ho.remap(w, s0, int(kind), **kw)
        # tolerance: 1e-6 relative (a division and a product in float32; the row norm sums in another order)
        np.testing.assert_allclose(scales.cpu().numpy(), want_s, rtol=2e-6)
        np.testing.assert_allclose(tile.get_weights().numpy(), want_w, rtol=2e-6, atol=1e-9)


def test_remap_on_a_pulsed_tile_and_its_errors(gpu_device):
    tile = pulsed_tile()
    w = tile.get_weights().numpy()
    scales = torch.ones(23, device="cuda")
    tile.remap_weights(remap_par(tiles.WeightRemapType.LayerwiseSymmetric, remapped_wmax=0.3), scales)
    want_w, want_s = ho.remap(w, np.ones(23, dtype=F), ho.REMAP_LAYERWISE_SYMMETRIC, remapped_wmax=0.3)
    np.testing.assert_allclose(tile.get_weights().numpy(), want_w, rtol=2e-6)
    np.testing.assert_allclose(scales.cpu().numpy(), want_s, rtol=2e-6)
    with pytest.raises(RuntimeError, match="Invalid scales dimensions"):
        tile.remap_weights(remap_par(tiles.WeightRemapType.LayerwiseSymmetric), torch.ones(22, device="cuda"))
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        tile.remap_weights(remap_par(tiles.WeightRemapType.LayerwiseSymmetric), torch.ones(23))
    with pytest.raises(RuntimeError, match="biases"):
        tile.remap_weights(remap_par(tiles.WeightRemapType.ChannelwiseAsymmetric), scales)
    with pytest.raises(RuntimeError, match="not implemented"):
        tile.remap_weights(remap_par(tiles.WeightRemapType.ChannelwiseExceeded), scales)
    with pytest.raises(RuntimeError, match="remapped_wmax to be 1"):
        tile.remap_weights(remap_par(tiles.WeightRemapType.ChannelwiseSymmetric, max_scale_range=2.0,
                                     remapped_wmax=0.5), scales)
    with pytest.raises(RuntimeError, match="row_norm"):
        tile.remap_weights(remap_par(tiles.WeightRemapType.ChannelwiseNorm, row_norm=0.0), scales)


# ---- modifier -----------------------------------------------------------------------------------------------------

def test_modifier_deterministic_types_against_the_oracle(gpu_device):
    T = tiles.WeightModifierType
    cases = [
        (T.Copy, dict()),
        (T.Discretize, dict(res=0.132)),
        (T.Discretize, dict(res=0.132, rel_to_actual_wmax=False, assumed_wmax=0.7)),
        (T.Discretize, dict(res=0.05, copy_last_column=True)),
        (T.Discretize, dict(res=0.0)),                                           # no resolution: a plain copy
        (T.DoReFa, dict(res=0.1, dorefa_clip=0.6)),
        (T.DoReFa, dict(res=0.07, dorefa_clip=0.9, copy_last_column=True)),
        (T.AddNormal, dict(std_dev=0.0)),                                        # no noise: a plain copy
        (T.DropConnect, dict(pdrop=0.0)),
    ]
    for shape in ((37, 23), (1000, 300)):
        tile = fp_tile(*shape)
        w = tile.get_weights().numpy()
        for kind, kw in cases:
            tile.modify_weights(modifier_par(kind, **kw))
            got = tile.get_modified_weights().numpy()
            want = ho.modify(w, int(kind), **kw)
            # values that sit on a rounding boundary within float32 accuracy may round either way
            step = kw.get("res", 0.0) * (np.abs(w).max() if kw.get("rel_to_actual_wmax", True) else kw.get("assumed_wmax"))
            off = np.abs(got - want) > 1e-6
            if kind == T.DoReFa:
                step = kw["res"]
            assert off.mean() < 1e-3 and (np.abs(got - want)[off] <= step * (1 + 1e-5)).all(), (kind, kw)
            assert np.array_equal(tile.get_weights().numpy(), w)                  # the weights themselves stay
            if kw.get("copy_last_column"):
                assert np.array_equal(got[:, -1], w[:, -1])


def test_modified_weights_are_what_forward_and_backward_contract_with(gpu_device):
    # the behaviour the reference tests for every modifier type (tests/test_inference_tiles.py:336-395): training
    # passes see the modified weights, evaluation and the weights that are read out do not
    tile = fp_tile(37, 23)
    w = tile.get_weights().numpy()
    rng = np.random.default_rng(1)
    x = torch.from_numpy(rng.uniform(-1, 1, (11, 37)).astype(F)).cuda()
    d = torch.from_numpy(rng.uniform(-1, 1, (11, 23)).astype(F)).cuda()
    plain = tile.forward(x).cpu().numpy()
    np.testing.assert_allclose(plain, x.cpu().numpy() @ w.T, atol=2e-5)
    with pytest.raises(RuntimeError, match="No modified weights"):
        tile.get_modified_weights()
    tile.modify_weights(modifier_par(tiles.WeightModifierType.Discretize, res=0.132))
    wm = tile.get_modified_weights().numpy()
    assert np.abs(wm - w).max() > 0.01
    np.testing.assert_allclose(tile.forward(x).cpu().numpy(), x.cpu().numpy() @ wm.T, atol=2e-5)
    np.testing.assert_allclose(tile.forward(x, is_test=True).cpu().numpy(), plain, atol=1e-6)
    np.testing.assert_allclose(tile.backward(d).cpu().numpy(), d.cpu().numpy() @ wm, atol=2e-5)
    # the update works on the real weights; the modified copy stays until the next modify_weights
    tile.set_learning_rate(0.1)
    tile.update(x, d, False)
    w_new = tile.get_weights().numpy()
    np.testing.assert_allclose(w_new, w - 0.1 * d.cpu().numpy().T @ x.cpu().numpy(), atol=2e-5)
    assert np.array_equal(tile.get_modified_weights().numpy(), wm)
    tile.modify_weights(modifier_par(tiles.WeightModifierType.Discretize, res=0.132, enable_during_test=True))
    wm2 = tile.get_modified_weights().numpy()
    np.testing.assert_allclose(tile.forward(x, is_test=True).cpu().numpy(), x.cpu().numpy() @ wm2.T, atol=2e-5)
    # a copy of the tile carries the modified weights along
    import copy
    twin = copy.deepcopy(tile)
    assert np.array_equal(twin.get_modified_weights().numpy(), wm2)
    np.testing.assert_allclose(twin.forward(x, is_test=True).cpu().numpy(), x.cpu().numpy() @ wm2.T, atol=2e-5)
    with pytest.raises(RuntimeError, match="not implemented"):
        tile.modify_weights(modifier_par(tiles.WeightModifierType.PCMNoise))
    with pytest.raises(RuntimeError, match="Per batch sample"):
        tile.modify_weights(modifier_par(tiles.WeightModifierType.AddNormal, per_batch_sample=True))


def test_modifier_noise_types_with_replayed_draws(gpu_device):
    # AddNormal with unit scale shows the normal draws; replaying the random stream (load_extra) gives every other
    # type the same draws, which the oracle then takes as its input
    T = tiles.WeightModifierType
    tile = fp_tile(128, 64)
    tile.set_seed(77)
    w = tile.get_weights().numpy()
    state = tile.dump_extra()
    base = dict(rel_to_actual_wmax=False, assumed_wmax=1.0)
    tile.modify_weights(modifier_par(T.AddNormal, std_dev=1.0, **base))
    z = (tile.get_modified_weights().numpy().astype(np.float64) - w).astype(F)
    n = z.size
    assert abs(z.mean()) < 4 / np.sqrt(n) and abs(z.std() - 1) < 4 / np.sqrt(2 * n)
    assert abs((z ** 3).mean()) < 4 * np.sqrt(15 / n) and abs((z ** 4).mean() - 3) < 4 * np.sqrt(96 / n)
    tile.modify_weights(modifier_par(T.AddNormal, std_dev=1.0, **base))             # the next call draws anew
    z_next = tile.get_modified_weights().numpy() - w
    assert abs(np.corrcoef(z.ravel(), z_next.ravel())[0, 1]) < 4 / np.sqrt(n)
    cases = [
        (T.AddNormal, dict(std_dev=0.3)),                                          # relative to the actual maximum
        (T.MultNormal, dict(std_dev=0.2, **base)),
        (T.Poly, dict(std_dev=0.1, coeffs=[1.0, 3.0], **base)),
        (T.Poly, dict(std_dev=0.1, coeffs=[0.1, 0.2, 0.2, 0.3])),
        (T.ProgNoise, dict(std_dev=0.5, coeffs=[0.1, 0.2, 0.2, 0.3], g_max=2.0)),
        (T.DiscretizeAddNormal, dict(std_dev=0.1, res=0.132, **base)),
        (T.AddNormal, dict(std_dev=0.3, copy_last_column=True)),
    ]
    for kind, kw in cases:
        tile.load_extra(state, True)
        tile.modify_weights(modifier_par(kind, **kw))
        got = tile.get_modified_weights().numpy()
        want = ho.modify(w, int(kind), normals=z, **kw)
        # z is known to about 1e-7 (it was read off a float32 sum), its products to a few 1e-7
        np.testing.assert_allclose(got, want, atol=3e-6, err_msg=str((kind, kw)))
    # dropped connections: the expected share, and the same connections for every type under the same draws
    tile.load_extra(state, True)
    tile.modify_weights(modifier_par(T.DropConnect, pdrop=0.3))
    dropped = tile.get_modified_weights().numpy() == 0
    assert abs(dropped.mean() - 0.3) < 4 * np.sqrt(0.21 / n)
    assert np.array_equal(tile.get_modified_weights().numpy()[~dropped], w[~dropped])
    tile.load_extra(state, True)
    tile.modify_weights(modifier_par(T.AddNormal, std_dev=0.3, pdrop=0.3))
    got = tile.get_modified_weights().numpy()
    assert np.array_equal(got == 0, dropped)
    np.testing.assert_allclose(got[~dropped], ho.modify(w, ho.MOD_ADD_NORMAL, normals=z, std_dev=0.3)[~dropped], atol=3e-6)
    assert abs(np.corrcoef(dropped.ravel(), z.ravel())[0, 1]) < 4 / np.sqrt(n)      # its own random word
    # stochastic rounding: the two neighbours on the grid, up with the probability of the remainder
    tile.modify_weights(modifier_par(T.Discretize, res=0.25, sto_round=True, **base))
    got = tile.get_modified_weights().numpy().astype(np.float64)
    q = w.astype(np.float64) / 0.25
    assert np.isin(np.round(got / 0.25), np.stack([np.floor(q), np.ceil(q)])).all()
    assert np.abs(got / 0.25 - np.round(got / 0.25)).max() < 1e-5
    went_up = got / 0.25 > q
    frac = q - np.floor(q)
    assert abs((went_up - frac).mean()) < 4 * np.sqrt((frac * (1 - frac)).mean() / n)
    assert abs(np.corrcoef(went_up.ravel() - frac.ravel(), z.ravel())[0, 1]) < 4 / np.sqrt(n)


# ---- device-level drift -------------------------------------------------------------------------------------------

def test_drift_golden_vector_of_the_reference_test(gpu_device):
    # tests/test_bindings_tiles.py:118-131 of the reference: nu = 0.1, t_0 = 1, delta_t = 2
    for tile in (pulsed_tile(drift=dict(nu=0.1, t_0=1.0, nu_dtod=0.0, nu_std=0.0, w_noise_std=0.0)),
                 fp_tile(drift=dict(nu=0.1))):
        w = tile.get_weights().numpy()
        tile.drift_weights(2.0)
        np.testing.assert_allclose(tile.get_weights().numpy(), w * 2.0 ** (-0.1), rtol=2e-6)
    still = pulsed_tile()                                         # a pulsed device without nu does not drift
    w = still.get_weights().numpy()
    still.drift_weights(5.0)
    assert np.array_equal(still.get_weights().numpy(), w)
    assert float(np.abs(hidden(still)["drift_nu"]).max()) == 0.0


def test_drift_sequence_against_the_oracle(gpu_device):
    drift = dict(nu=0.08, nu_dtod=0.3, t_0=2.0, wg_ratio=0.5, g_offset=0.2, w_offset=-0.05, reset_tol=1e-6)
    tile = pulsed_tile(drift=drift, w_max=0.4, w_min=-0.4, w_max_dtod=0.1, w_min_dtod=0.1)
    par = hidden(tile)
    nu = par["drift_nu"]
    assert abs(nu.mean() - 0.08) < 0.004 and 0.015 < nu.std() < 0.035
    oracle = ho.Drifter(nu, t0=2.0, wg_ratio=0.5, g_offset=0.2, w_offset=-0.05, reset_tol=1e-6)
    bounds = dict(w_min=par["min_bound"], w_max=par["max_bound"])
    rng = np.random.default_rng(2)
    x = torch.from_numpy(rng.uniform(-1, 1, (4, 37)).astype(F)).cuda()
    d = torch.from_numpy((rng.uniform(-1, 1, (4, 23)) * (rng.random((4, 23)) < 0.3)).astype(F)).cuda()
    tile.set_learning_rate(0.02)
    w = tile.get_weights().numpy()
    for step, dt in enumerate((1.0, 3.0, 4.0, 20.0, 100.0)):
        if step == 2:
            tile.update(x, d, False)                              # some weights change: their clocks restart
            w_new = tile.get_weights().numpy()
            changed = np.abs(w_new - w) > 1e-6
            assert 0.02 < changed.mean() < 0.9 and np.array_equal(changed, w_new != w)
            w = w_new
        tile.drift_weights(dt)
        w = oracle.apply(w, dt, **bounds)
        got = tile.get_weights().numpy()
        # tolerance: powf against a float64 power, rounded once
        np.testing.assert_allclose(got, w, rtol=3e-6, atol=1e-7, err_msg="step %d" % step)
        w = got
        oracle.prev = got.copy()
    assert np.array_equal(oracle.t != 0, changed)                 # exactly the updated weights restarted
    # new drift coefficients through the hidden parameters are used from the next call on
    names = tile.get_hidden_parameter_names()
    values = tile.get_hidden_parameters()
    values[names.index("drift_nu")] = 0.2
    tile.set_hidden_parameters(values)
    oracle.nu = np.full_like(nu, 0.2)
    w = tile.get_weights().numpy()                                # the new bounds clip at once; here they are the same
    tile.drift_weights(50.0)
    np.testing.assert_allclose(tile.get_weights().numpy(), oracle.apply(w, 50.0, **bounds), rtol=3e-6, atol=1e-7)
    # a copy drifts on from the same clocks
    import copy
    twin = copy.deepcopy(tile)
    tile.drift_weights(10.0)
    twin.drift_weights(10.0)
    assert np.array_equal(tile.get_weights().numpy(), twin.get_weights().numpy())


def test_drift_with_conductance_dependent_nu_and_noise(gpu_device):
    rng = np.random.default_rng(4)
    w0 = (np.abs(rng.normal(0, 0.3, (64, 128))) + 0.05).astype(F)
    drift = dict(nu=0.05, nu_k=0.02, log_g0=float(np.log(0.5)))
    tile = fp_tile(128, 64, weights=w0, drift=drift)
    oracle = ho.Drifter(0.05, nu_k=0.02, log_g0=np.log(0.5))
    tile.drift_weights(7.0)
    np.testing.assert_allclose(tile.get_weights().numpy(), oracle.apply(w0, 7.0), rtol=3e-6)
    # variation of nu from call to call and read noise: N(0, 1) draws that enter as the oracle says
    tile = fp_tile(128, 64, weights=w0, drift=dict(nu=0.1, nu_std=0.3))
    tile.drift_weights(8.0)
    z = (np.log(tile.get_weights().numpy().astype(np.float64) / w0) / (-np.log(8.0)) - 0.1) / 0.03
    n = z.size
    assert abs(z.mean()) < 4 / np.sqrt(n) and abs(z.std() - 1) < 4 / np.sqrt(2 * n)
    tile.drift_weights(8.0)                                       # redrawn at every call, from w0 at the new time
    z2 = (np.log(tile.get_weights().numpy().astype(np.float64) / w0) / (-np.log(16.0)) - 0.1) / 0.03
    assert abs(z2.std() - 1) < 4 / np.sqrt(2 * n) and abs(np.corrcoef(z.ravel(), z2.ravel())[0, 1]) < 4 / np.sqrt(n)
    tile = fp_tile(128, 64, weights=w0, drift=dict(nu=0.1, w_noise_std=0.01))
    tile.drift_weights(8.0)
    r = (tile.get_weights().numpy().astype(np.float64) - w0 * 8.0 ** (-0.1)) / 0.01
    assert abs(r.mean()) < 4 / np.sqrt(n) and abs(r.std() - 1) < 4 / np.sqrt(2 * n)


# ---- pulse counters -----------------------------------------------------------------------------------------------

def test_pulse_counters_of_stochastic_updates(gpu_device):
    rng = np.random.default_rng(6)
    x = torch.from_numpy(rng.uniform(-1, 1, (40, 37)).astype(F)).cuda()
    d = torch.from_numpy(rng.normal(0, 0.4, (40, 23)).astype(F)).cuda()
    tile = pulsed_tile(count_pulses=True)
    plain = pulsed_tile()
    assert plain.get_pulse_counters().numel() == 0
    for t in (tile, plain):
        t.set_learning_rate(0.05)
        t.set_seed(9)
    assert tile.get_pulse_counters().shape == (2, 23, 37) and int(tile.get_pulse_counters().sum()) == 0
    total = np.zeros((2, 23, 37), dtype=np.int64)
    for _ in range(2):
        tile.update(x, d, False)
        plain.update(x, d, False)
        x_words, d_words, _bl = tile.get_update_words(40)
        total += ho.pulse_counts(x_words.numpy().view(np.uint32), d_words.numpy().view(np.uint32))
        assert np.array_equal(tile.get_pulse_counters().numpy(), total)
    assert total[0].sum() > 1000 and total[1].sum() > 1000
    assert torch.equal(tile.get_weights(), plain.get_weights())   # counting changes nothing else
    # words made elsewhere are counted too
    xw = torch.from_numpy(rng.integers(0, 2 ** 31, (5, 37)).astype(np.int32)).cuda()
    dw = torch.from_numpy(rng.integers(0, 2 ** 31, (5, 23)).astype(np.int32)).cuda()
    tile.update_with_words(xw, dw)
    total += ho.pulse_counts(xw.cpu().numpy().view(np.uint32), dw.cpu().numpy().view(np.uint32))
    assert np.array_equal(tile.get_pulse_counters().numpy(), total)
    import copy
    twin = copy.deepcopy(tile)
    assert np.array_equal(twin.get_pulse_counters().numpy(), total)


def test_pulse_counters_of_implicit_updates(gpu_device):
    rng = np.random.default_rng(7)
    x = torch.from_numpy(rng.uniform(-1, 1, (12, 37)).astype(F)).cuda()
    d = torch.from_numpy(rng.normal(0, 0.4, (12, 23)).astype(F)).cuda()
    tile = pulsed_tile(pulse_type=dv.PulseType.DeterministicImplicit, count_pulses=True)
    tile.set_learning_rate(0.05)
    tile.update(x, d, False)
    n = tile.get_implicit_counts(12).numpy().astype(np.int64)
    want = np.stack([np.where(n > 0, n, 0).sum(axis=0), np.where(n < 0, -n, 0).sum(axis=0)])
    assert want[0].sum() > 100 and want[1].sum() > 100
    assert np.array_equal(tile.get_pulse_counters().numpy(), want)


# ---- write noise (persistent weights) -------------------------------------------------------------------------------

def test_write_noise_persistent_weights(gpu_device):
    """SoftBounds with write_noise_std: the pulses and the maintenance act on the persistent weights, which follow the
    trajectory of the same device without write noise (oracle and GPU, deterministic pulses); the shown weights are those
    plus N(0, (write_noise_std dw_min)^2), redrawn where a pulse landed, for all after maintenance and set_weights."""
    from helpers import build_pair

    rng = np.random.default_rng(5)
    x_size, d_size, batch = 70, 45, 8
    sigma = 5.0 * 0.002
    for pulse_type in (dv.PulseType.DeterministicImplicit, dv.PulseType.StochasticCompressed):
        meta = make_meta(noise_free_io(), noise_free_io(), pulse_type=pulse_type, desired_bl=31)
        kw = dict(dw_min=0.002, dw_min_std=0.0, construction_seed=3, lifetime=40.0)
        host, orc, noisy = build_pair(meta, soft_bounds(write_noise_std=5.0, **kw), x_size, d_size)
        _h, _o, plain = build_pair(meta, soft_bounds(**kw), x_size, d_size)
        names = noisy.get_hidden_parameter_names()
        assert names.index("persistent_weights") == 8 and names[-2:] == ["slope_up", "slope_down"] and len(names) == 11
        persistent = lambda: noisy.get_hidden_parameters()[8].numpy()       # noqa: E731
        w = rng.uniform(-0.3, 0.3, (d_size, x_size)).astype(F)
        for t in (noisy, plain):
            t.set_weights(torch.from_numpy(w))
            t.set_learning_rate(0.05)
            t.set_seed(31)
        shown0 = noisy.get_weights().numpy()
        assert np.array_equal(persistent(), plain.get_weights().numpy())
        z = (shown0 - persistent()) / sigma
        assert abs(z.mean()) < 4 / np.sqrt(z.size) and abs(z.std() - 1) < 4 / np.sqrt(2 * z.size)
        x = rng.uniform(-1, 1, (batch, x_size)).astype(F)
        x[:, :12] = 0.0                                           # columns that see no pulse
        d = rng.normal(0, 0.3, (batch, d_size)).astype(F)
        xg, dg = torch.from_numpy(x).cuda(), torch.from_numpy(d).cuda()
        noisy.update(xg, dg, False)
        plain.update(xg, dg, False)
        assert np.array_equal(persistent(), plain.get_weights().numpy())    # same seed, same pulses, same steps
        touched = plain.get_weights().numpy() != np.clip(w, hidden(plain)["min_bound"], hidden(plain)["max_bound"])
        assert not touched[:, :12].any() and 0.2 < touched.mean() < 0.95
        shown1 = noisy.get_weights().numpy()
        assert np.array_equal(shown1[:, :12], shown0[:, :12])    # no pulse, no new noise
        z1 = ((shown1 - persistent()) / sigma)[touched]
        assert abs(z1.mean()) < 4 / np.sqrt(z1.size) and abs(z1.std() - 1) < 4 / np.sqrt(2 * z1.size)
        assert abs(np.corrcoef(z1, z[touched])[0, 1]) < 4 / np.sqrt(z1.size)   # redrawn
        if pulse_type == dv.PulseType.DeterministicImplicit:     # the oracle walks the same deterministic pulses
            orc.set_weights(w)
            orc.set_learning_rate(0.05)
            orc.update(x, d)
            assert np.abs(orc.get_persistent() - persistent()).max() <= 1e-5
        # forward contracts with the shown weights
        y = noisy.forward(xg).cpu().numpy()
        assert np.abs(y - plain.forward(xg).cpu().numpy()).max() > 1e-3
        # maintenance acts on the persistent weights and redraws every shown one
        noisy.decay_weights(1.0)
        plain.decay_weights(1.0)
        assert np.abs(persistent() - plain.get_weights().numpy()).max() <= 1e-7
        shown2 = noisy.get_weights().numpy()
        z2 = (shown2 - persistent()) / sigma
        assert abs(z2.std() - 1) < 4 / np.sqrt(2 * z2.size) and abs(np.corrcoef(z2.ravel(), z.ravel())[0, 1]) < 4 / np.sqrt(z2.size)
        assert not np.array_equal(shown2[:, :12], shown1[:, :12])
        # a copy carries both matrices
        import copy
        twin = copy.deepcopy(noisy)
        assert np.array_equal(twin.get_hidden_parameters()[8].numpy(), persistent())
        assert np.array_equal(twin.get_weights().numpy(), shown2)
    # without apply_write_noise_on_set the given weights are shown as they are
    _h, _o, quiet = build_pair(meta, soft_bounds(write_noise_std=5.0, apply_write_noise_on_set=False, **kw), x_size, d_size)
    quiet.set_weights(torch.from_numpy(w))
    assert np.array_equal(quiet.get_weights().numpy(), quiet.get_hidden_parameters()[8].numpy())
