"""Pins of the IR-drop and output-referred weight-noise restatement in oracle/rpu_oracle.cpp: closed forms on tiles
whose sums can be written down, the position dependence of the drop, and the variance laws of the two noise types."""
import numpy as np

from aihwkit_amd.rpu_base import devices as dv
from helpers import constant_step, io_params, make_meta
from oracle_lib import OracleTile

F = np.float32


def oracle_tile(x_size, d_size, w, **io):
    # no quantization, no clipping, no scaling: the inputs reach the array as they are
    base = dict(out_noise=0.0, inp_noise=0.0, inp_res=-1.0, out_res=-1.0, out_bound=1e6,
                noise_management=dv.NoiseManagementType.NONE, bound_management=dv.BoundManagementType.NONE)
    base.update(io)
    meta = make_meta(io_params(**base), io_params(**base))
    dev = constant_step(w_max=10.0, w_min=-10.0, w_max_dtod=0.0, w_min_dtod=0.0, construction_seed=1)
    tile = OracleTile(x_size, d_size, meta._config(dev))
    tile.set_weights(np.asarray(w, dtype=F))
    return tile


def drop_factor(a):
    return a * (a * (0.05 * a - 0.2) + 0.5)


def test_ir_drop_closed_form_on_a_constant_tile():
    for n, d, w, v, ratio, scale in ((8, 3, 0.5, 0.7, 40.0, 1.0), (20, 2, -0.3, 0.9, 150.0, 2.5), (5, 4, 0.4, -1.0, 10.0, 0.5)):
        tile = oracle_tile(n, d, np.full((d, n), w), ir_drop=scale, ir_drop_g_ratio=ratio)
        y = tile.forward(np.full((1, n), v, dtype=F))[0]
        a = n / ratio * (n * abs(w) * abs(v))                    # total current, scaled by n / (Gw / g_max)
        s = sum(1.0 - (1.0 - j / n) ** 2 for j in range(n))      # sum of the position weights
        want = n * w * v - scale * drop_factor(a) * w * v * s
        np.testing.assert_allclose(y, np.full(d, want), rtol=2e-6)
        assert abs(want - n * w * v) > 1e-3 * abs(n * w * v)     # the drop is visible in this setting


def test_ir_drop_depends_on_the_position_of_the_input_line():
    n, ratio = 10, 8.0
    w = np.linspace(0.2, 0.9, 3 * n).reshape(3, n).astype(F) * np.array([[1], [-1], [1]], dtype=F)
    tile = oracle_tile(n, 3, w, ir_drop=1.0, ir_drop_g_ratio=ratio)
    for j in (0, 1, 5, 9):
        x = np.zeros((1, n), dtype=F)
        x[0, j] = -0.8
        y = tile.forward(x)[0].astype(np.float64)
        a = n / ratio * np.abs(w[:, j].astype(np.float64)) * 0.8
        want = w[:, j] * -0.8 * (1.0 - drop_factor(a) * (1.0 - (1.0 - j / n) ** 2))
        np.testing.assert_allclose(y, want, rtol=3e-6)
    x = np.zeros((1, n), dtype=F)
    x[0, 0] = 1.0                                                # the line next to the output sees no drop at all
    np.testing.assert_array_equal(tile.forward(x)[0], w[:, 0])
    # backward: the same law on the transposed matrix (n = d_size input lines)
    dvec = np.zeros((1, 3), dtype=F)
    dvec[0, 2] = 0.5
    got = tile.backward(dvec)[0].astype(np.float64)
    a = 3 / ratio * np.abs(w[2].astype(np.float64)) * 0.5
    want = w[2] * 0.5 * (1.0 - drop_factor(a) * (1.0 - (1.0 - 2 / 3) ** 2))
    np.testing.assert_allclose(got, want, rtol=3e-6)


def test_weight_noise_variance_laws():
    rng = np.random.default_rng(0)
    n, d, m = 16, 400, 50
    x = rng.uniform(-1, 1, (m, n)).astype(F)
    # additive constant: sigma = w_noise |x|_2 for every output, whatever the weights
    tile = oracle_tile(n, d, np.zeros((d, n)), w_noise=0.05, w_noise_type=dv.WeightNoiseType.AdditiveConstant)
    tile.set_seed(3)
    y = tile.forward(x).astype(np.float64)
    z = y / (0.05 * np.linalg.norm(x.astype(np.float64), axis=1))[:, None]
    assert abs(z.mean()) < 4 / np.sqrt(z.size) and abs(z.std() - 1) < 4 / np.sqrt(2 * z.size)
    assert abs(np.corrcoef(z[:, :-1].ravel(), z[:, 1:].ravel())[0, 1]) < 4 / np.sqrt(z.size)
    # PCM read noise: sigma_i^2 = w_noise^2 sum_j |w_ij| x_j^2
    w = rng.uniform(-0.6, 0.6, (d, n)).astype(F)
    w[:50] *= 0.01                                               # rows of small conductance are quiet
    tile = oracle_tile(n, d, w, w_noise=0.1, w_noise_type=dv.WeightNoiseType.PCMRead)
    tile.set_seed(4)
    y = tile.forward(x).astype(np.float64)
    clean = x.astype(np.float64) @ w.T.astype(np.float64)
    sigma = 0.1 * np.sqrt((x.astype(np.float64) ** 2) @ np.abs(w.T.astype(np.float64)))
    z = (y - clean) / sigma
    assert abs(z.mean()) < 4 / np.sqrt(z.size) and abs(z.std() - 1) < 4 / np.sqrt(2 * z.size)
    assert abs(z[:, :50].std() - 1) < 4 / np.sqrt(2 * 50 * m)    # the law holds on the quiet rows as well
    assert (y - clean)[:, :50].std() < 0.2 * (y - clean)[:, 50:].std()
    # backward uses the transposed matrix: sigma_j^2 = w_noise^2 sum_i |w_ij| d_i^2
    dm = rng.uniform(-1, 1, (m, d)).astype(F)
    got = tile.backward(dm).astype(np.float64)
    sigma = 0.1 * np.sqrt((dm.astype(np.float64) ** 2) @ np.abs(w.astype(np.float64)))
    z = (got - dm.astype(np.float64) @ w.astype(np.float64)) / sigma
    assert abs(z.mean()) < 4 / np.sqrt(z.size) and abs(z.std() - 1) < 4 / np.sqrt(2 * z.size)


def test_running_average_noise_management_closed_form():
    """AverageAbsMax: the first sample sets the scale, every further one moves it by nm_decay towards its own largest
    absolute input; forward and backward share the one value and it lives on between calls.  With an identity tile and
    the DAC clipping at 1 the largest output of a sample whose input exceeds the scale is the scale itself.  Maxima
    1, 2, 2, 2, ... with nm_decay = 0.5 give 2 - 2^-b."""
    n = 6
    io = dict(noise_management=dv.NoiseManagementType.AverageAbsMax, nm_decay=0.5, inp_bound=1.0)
    tile = oracle_tile(n, n, np.eye(n), **io)
    x = np.zeros((5, n), dtype=F)
    x[:, 0] = [1.0, 2.0, 2.0, 2.0, 2.0]
    x[:, 1] = [0.5, -0.25, 0.125, 1.0, -2.0]                     # smaller entries pass through unchanged
    y = tile.forward(x)
    want = 2.0 - 0.5 ** np.arange(5)
    np.testing.assert_allclose(y[:, 0], want, rtol=1e-6)
    np.testing.assert_allclose(y[:3, 1], x[:3, 1], rtol=1e-6)
    np.testing.assert_allclose(y[4, 1], -want[4], rtol=1e-6)      # clipped on the negative side as well
    d = np.zeros((2, n), dtype=F)
    d[:, 3] = [-2.0, 2.0]                                         # the backward pass continues the same average
    g = tile.backward(d)
    np.testing.assert_allclose(np.abs(g[:, 3]), 2.0 - 0.5 ** np.arange(5, 7), rtol=1e-6)
    y = tile.forward(x[1:2])                                      # and the next forward call goes on from there
    np.testing.assert_allclose(y[0, 0], 2.0 - 0.5 ** 7, rtol=1e-6)
    fresh = oracle_tile(n, n, np.eye(n), **io)                    # another tile starts from its own first sample
    np.testing.assert_allclose(fresh.forward(x[1:3])[:, 0], [2.0, 2.0], rtol=1e-6)
    # a sample below the average is scaled by the average, not by its own maximum: nothing clips, the value survives
    low = np.zeros((1, n), dtype=F)
    low[0, 2] = 0.01
    np.testing.assert_allclose(fresh.forward(low)[0, 2], 0.01, rtol=1e-5)


def test_mean_count_and_none_with_device_updates_closed_form():
    """MeanCount: every line gets round(BL p) pulses, a cross-point round(d_count / BL * x_count) steps of dw_min (no
    variation here); NoneWithDevice: the floating-point outer product, then the device bounds."""
    from oracle_lib import OracleTile

    dev = constant_step(dw_min=0.01, dw_min_dtod=0.0, dw_min_std=0.0, up_down_dtod=0.0, w_max=0.3, w_min=-0.3, w_max_dtod=0.0,
                        w_min_dtod=0.0, construction_seed=1)
    meta = make_meta(pulse_type=dv.PulseType.MeanCount, desired_bl=10, update_management=False, update_bl_management=False,
                     fixed_bl=True)
    tile = OracleTile(3, 2, meta._config(dev))
    tile.set_weights(np.zeros((2, 3), dtype=F))
    tile.set_learning_rate(0.1)
    # lr / (dw_min BL) = 1: A = B = 1, so p = |value|; counts round(10 p): x -> 10, 5, 0(-), d -> 8, -4 (round half even)
    x = np.array([[1.0, 0.5, -0.04]], dtype=F)
    d = np.array([[0.8, -0.35]], dtype=F)
    counts = tile.implicit_counts(x, d)[0]
    # rintf(d_count / 10 * x_count): [8, 4, 0] and [-4, -2, 0]
    np.testing.assert_array_equal(counts, [[8, 4, 0], [-4, -2, 0]])
    tile.update(x, d)
    np.testing.assert_allclose(tile.get_weights(), [[-0.08, -0.04, 0.0], [0.04, 0.02, 0.0]], atol=1e-7)   # w -= lr d x^T
    x2 = np.array([[0.25, -1.0, 0.0]], dtype=F)                   # 2.5 rounds to 2 (half to even), negative input
    np.testing.assert_array_equal(tile.implicit_counts(x2, d)[0], [[2, -8, 0], [-1, 4, 0]])
    # NoneWithDevice
    meta = make_meta(pulse_type=dv.PulseType.NoneWithDevice)
    tile = OracleTile(3, 2, meta._config(dev))
    w0 = np.array([[0.25, 0.0, -0.29], [0.0, 0.1, 0.2]], dtype=F)
    tile.set_weights(w0)
    tile.set_learning_rate(0.5)
    xs = np.array([[1.0, 0.5, -1.0], [0.5, 0.0, 1.0]], dtype=F)
    ds = np.array([[-0.4, 0.2], [0.1, -0.3]], dtype=F)
    tile.update(xs, ds)
    want = np.clip(np.clip(w0 - 0.5 * np.outer(ds[0], xs[0]), -0.3, 0.3) - 0.5 * np.outer(ds[1], xs[1]), -0.3, 0.3)
    np.testing.assert_allclose(tile.get_weights(), want, atol=1e-6)
    assert (np.abs(w0 - 0.5 * ds.T @ xs) > 0.3).any()             # the example does reach the bounds


def test_write_noise_persistent_weights_in_the_oracle():
    """With write noise the pulses act on persistent weights, which follow exactly the trajectory of a device without
    it; the shown weights are those plus N(0, (write_noise_std dw_min)^2), redrawn only where a pulse landed."""
    from oracle_lib import OracleTile

    rng = np.random.default_rng(5)
    x_size, d_size, batch = 40, 30, 6
    meta = make_meta(pulse_type=dv.PulseType.DeterministicImplicit, desired_bl=31)
    kw = dict(dw_min=0.002, dw_min_std=0.0, construction_seed=3)
    from helpers import soft_bounds
    noisy = OracleTile(x_size, d_size, meta._config(soft_bounds(write_noise_std=5.0, **kw)))
    plain = OracleTile(x_size, d_size, meta._config(soft_bounds(**kw)))
    w = rng.uniform(-0.3, 0.3, (d_size, x_size)).astype(F)
    noisy.set_seed(11)
    noisy.set_weights(w)
    plain.set_weights(w)
    shown0 = noisy.get_weights()
    np.testing.assert_array_equal(noisy.get_persistent(), plain.get_weights())
    z = (shown0 - noisy.get_persistent()) / (5.0 * 0.002)       # apply_write_noise_on_set: all redrawn
    assert abs(z.mean()) < 4 / np.sqrt(z.size) and abs(z.std() - 1) < 4 / np.sqrt(2 * z.size)
    x = rng.uniform(-1, 1, (batch, x_size)).astype(F)
    x[:, :10] = 0.0                                              # columns that see no pulse
    d = rng.normal(0, 0.3, (batch, d_size)).astype(F)
    for t in (noisy, plain):
        t.set_learning_rate(0.05)
        t.update(x, d)
    np.testing.assert_array_equal(noisy.get_persistent(), plain.get_weights())
    counts = np.abs(plain.implicit_counts(x, d)).sum(axis=0)
    shown1 = noisy.get_weights()
    untouched = counts == 0
    assert untouched[:, :10].all() and 0.2 < (~untouched).mean() < 0.9
    np.testing.assert_array_equal(shown1[untouched], shown0[untouched])
    z = ((shown1 - noisy.get_persistent()) / (5.0 * 0.002))[~untouched]
    assert abs(z.mean()) < 4 / np.sqrt(z.size) and abs(z.std() - 1) < 4 / np.sqrt(2 * z.size)
    assert abs(np.corrcoef(z, ((shown0 - plain.get_weights()) / 0.01)[~untouched])[0, 1]) < 0.3   # redrawn, not shifted
