"""Pins of the per-line periphery terms in oracle/rpu_oracle.cpp: voltage offsets with and without a reference line,
series resistance, output non-linearity with its slope calibration, per-line output noise, the order of these steps
among IR drop / weight noise / ADC, and the laws the per-line values are drawn from.  Expected values are worked out
by hand on tiles whose sums can be written down."""
import numpy as np

from aihwkit_amd.rpu_base import devices as dv
from test_oracle_nonideal_pins import oracle_tile

F = np.float32


def test_output_nonlinearity_and_its_slope_calibration():
    n = 4
    # without calibration: y / (1 + nl_i |y|) with the given coefficients
    tile = oracle_tile(n, n, np.eye(n), out_nonlinearity=1.0, slope_calibration=0.0, out_bound=12.0)
    tile.set_lines(0, 1, [0.0, 0.1, 0.5, 1.0])
    assert tile.nl_factor(0) == 1.0
    y = tile.forward(np.array([[0.5, -0.5, 1.0, -1.0]], dtype=F))[0]
    np.testing.assert_allclose(y, [0.5, -0.5 / 1.05, 1.0 / 1.5, -1.0 / 2.0], rtol=1e-6)
    # drawn without spread: nl = out_nonlinearity / out_bound = 0.1 on every line; f = 1 + nl c out_bound = 1.6
    tile = oracle_tile(n, n, 10.0 * np.eye(n), out_nonlinearity=1.2, slope_calibration=0.5, out_bound=12.0)
    np.testing.assert_allclose(tile.get_lines(0, 1), np.full(n, 0.1), rtol=1e-6)
    assert abs(tile.nl_factor(0) - 2.56) < 1e-5
    y = tile.forward(np.array([[0.05, 0.0, 0.0, -0.2]], dtype=F))[0]
    np.testing.assert_allclose(y, [2.56 * 0.5 / 1.05, 0.0, 0.0, -2.56 * 2.0 / 1.2], rtol=1e-6)
    # what the calibration is for: slope 1 at y = slope_calibration * out_bound = 6 (x = 0.6 through weights of 10)
    lo = tile.forward(np.array([[0.599, 0, 0, 0]], dtype=F))[0, 0]
    hi = tile.forward(np.array([[0.601, 0, 0, 0]], dtype=F))[0, 0]
    assert abs((hi - lo) / 0.02 - 1.0) < 2e-3
    # the backward pass has its own lines, of the other length
    tile = oracle_tile(3, 5, np.zeros((5, 3)), out_nonlinearity=0.6, out_nonlinearity_std=0.0)
    assert tile.get_lines(0, 1).shape == (5,) and tile.get_lines(1, 1).shape == (3,)
    assert tile.get_lines(0, 0).size == 0 and tile.get_lines(0, 2).size == 0


def test_voltage_offsets_and_series_resistance():
    n = 3
    x = np.array([[0.8, -0.4, 0.5]], dtype=F)
    vo = np.array([0.0, 0.1, 0.25], dtype=F)
    # offsets alone: (1 - vo_i) y_i
    tile = oracle_tile(n, n, np.eye(n), v_offset_std=0.1)
    tile.set_lines(0, 0, vo)
    np.testing.assert_allclose(tile.forward(x)[0], x[0] * (1 - vo), rtol=1e-6)
    # series resistance: (1 - vo_i) y_i / (1 + min(rs |y_i|, cap)); it also switches the slope calibration on
    for cap, c in ((3.4028234e38, 0.0), (0.1, 0.0), (3.4028234e38, 0.5)):
        tile = oracle_tile(n, n, np.eye(n), v_offset_std=0.1, r_series=0.5, r_series_max_total=cap, slope_calibration=c,
                           out_bound=12.0)
        tile.set_lines(0, 0, vo)
        f = (1.0 + 0.5 * c * 12.0) ** 2
        assert abs(tile.nl_factor(0) - f) < 1e-5
        np.testing.assert_array_equal(tile.get_lines(0, 1), np.zeros(n, dtype=F))
        want = f * (1 - vo) * x[0] / (1 + np.minimum(0.5 * np.abs(x[0]), cap))
        np.testing.assert_allclose(tile.forward(x)[0], want, rtol=1e-6)
    # with a reference line of conductance w_min = -1: y_ref = sum_j x_j = 0.9
    tile = oracle_tile(n, n, np.eye(n), v_offset_std=0.1, v_offset_w_min=-1.0)
    tile.set_lines(0, 0, vo)
    np.testing.assert_allclose(tile.forward(x)[0], x[0] * (1 - vo) - vo * 2 * 0.9, rtol=1e-6)
    tile = oracle_tile(n, n, np.eye(n), v_offset_std=0.1, v_offset_w_min=-1.0, r_series=0.5, slope_calibration=0.0)
    tile.set_lines(0, 0, vo)
    y_pos = x[0] + 0.9
    want = (1 - vo) * y_pos / (1 + 0.5 * np.abs(y_pos)) - (1 + vo) * 0.9 / (1 + 0.5 * 0.9)
    np.testing.assert_allclose(tile.forward(x)[0], want, rtol=1e-6)
    # backward uses the lines of its own direction on the transposed matrix
    w = np.array([[1.0, 2.0, 0.0], [0.0, 1.0, 0.5]], dtype=F)
    tile = oracle_tile(3, 2, w, v_offset_std=0.1)
    tile.set_lines(1, 0, vo)
    tile.set_lines(0, 0, [0.5, 0.5])
    d = np.array([[1.0, -1.0]], dtype=F)
    np.testing.assert_allclose(tile.backward(d)[0], (d @ w)[0] * (1 - vo), rtol=1e-6)
    np.testing.assert_allclose(tile.forward(x)[0], 0.5 * (x @ w.T)[0], rtol=1e-6)


def test_order_of_the_periphery_steps():
    """IR drop, then offsets, then weight noise, then non-linearity, asymmetry, output noise, ADC."""
    n, d, m = 8, 300, 40
    rng = np.random.default_rng(2)
    x = rng.uniform(0.2, 1.0, (m, n)).astype(F)
    # offsets halve the mean but not the weight noise added after them
    tile = oracle_tile(n, d, np.full((d, n), 0.3), v_offset_std=0.1, w_noise=0.05,
                       w_noise_type=dv.WeightNoiseType.AdditiveConstant)
    tile.set_lines(0, 0, np.full(d, 0.5))
    tile.use_gauss_table(False)                                  # the table of 32768 normals has a mean of its own
    y = tile.forward(x).astype(np.float64)
    mean = 0.5 * 0.3 * x.astype(np.float64).sum(axis=1)
    z = (y - mean[:, None]) / (0.05 * np.linalg.norm(x.astype(np.float64), axis=1))[:, None]
    assert abs(z.mean()) < 4 / np.sqrt(z.size) and abs(z.std() - 1) < 4 / np.sqrt(2 * z.size)
    # the offsets act on the sums after the IR drop: (1 - vo) (y - drop)
    plain = oracle_tile(n, 2, np.full((2, n), 0.3), ir_drop=1.0, ir_drop_g_ratio=20.0)
    both = oracle_tile(n, 2, np.full((2, n), 0.3), ir_drop=1.0, ir_drop_g_ratio=20.0, v_offset_std=0.1)
    both.set_lines(0, 0, [0.25, 0.0])
    a, b = plain.forward(x), both.forward(x)
    assert np.abs(a[:, 0] - 0.3 * x.sum(axis=1)).max() > 1e-3
    np.testing.assert_allclose(b, a * np.array([0.75, 1.0], dtype=F), rtol=1e-6)
    # asymmetry after the non-linearity, output noise after both (not compressed), then the ADC grid
    tile = oracle_tile(2, 2, np.eye(2), out_nonlinearity=1.0, slope_calibration=0.0, out_asymmetry=0.5)
    tile.set_lines(0, 1, [1.0, 1.0])
    np.testing.assert_allclose(tile.forward(np.array([[1.0, -1.0]], dtype=F))[0], [0.5, -0.25], rtol=1e-6)
    tile = oracle_tile(1, 2000, np.ones((2000, 1)), out_nonlinearity=1.0, slope_calibration=0.0, out_noise=0.2)
    tile.set_lines(0, 1, np.full(2000, 1.0))
    tile.use_gauss_table(False)
    y = tile.forward(np.ones((20, 1), dtype=F)).astype(np.float64)
    assert abs(y.mean() - 0.5) < 4 * 0.2 / np.sqrt(y.size) and abs(y.std() / 0.2 - 1) < 4 / np.sqrt(2 * y.size)
    tile = oracle_tile(2, 2, np.eye(2), v_offset_std=0.1, out_res=0.25, out_bound=1.0)   # absolute step 0.5
    tile.set_lines(0, 0, [0.3, 0.0])
    np.testing.assert_array_equal(tile.forward(np.array([[1.0, 1.0]], dtype=F))[0], [0.5, 1.0])


def test_per_line_output_noise_levels():
    d, m = 5, 4000
    tile = oracle_tile(1, d, np.zeros((d, 1)), out_noise=0.1, out_noise_std=0.3)
    levels = np.array([0.0, 0.02, 0.1, 0.5, 1.0], dtype=F)
    tile.set_lines(0, 2, levels)
    tile.use_gauss_table(False)
    y = tile.forward(np.ones((m, 1), dtype=F)).astype(np.float64)
    assert np.all(y[:, 0] == 0.0)
    z = y[:, 1:] / levels[1:]
    assert np.abs(z.mean(axis=0)).max() < 4 / np.sqrt(m) and np.abs(z.std(axis=0) - 1).max() < 4 / np.sqrt(2 * m)


def test_laws_of_the_drawn_line_values():
    d = 20000
    tile = oracle_tile(2, d, np.zeros((d, 2)), v_offset_std=0.2, out_nonlinearity=0.6, out_nonlinearity_std=0.25,
                       out_noise=0.1, out_noise_std=0.5, out_bound=12.0, slope_calibration=0.5)
    vo, nl, noise = (tile.get_lines(0, k).astype(np.float64) for k in range(3))
    # max(0.2 xi, 0): half of the lines have none, the others a half normal
    assert abs((vo == 0).mean() - 0.5) < 4 * 0.5 / np.sqrt(d) and vo.min() == 0.0
    pos = vo[vo > 0] / 0.2
    assert abs(pos.mean() - np.sqrt(2 / np.pi)) < 4 * np.sqrt(1 - 2 / np.pi) / np.sqrt(pos.size)
    assert abs((pos ** 2).mean() - 1.0) < 4 * np.sqrt(2.0 / pos.size)
    # |0.6 / 12 (1 + 0.25 xi)|: four sigma away from a sign change
    r = nl / 0.05
    assert abs(r.mean() - 1.0) < 4 * 0.25 / np.sqrt(d) and abs(r.std() / 0.25 - 1) < 4 / np.sqrt(2 * d) and nl.min() > 0
    r = noise / 0.1
    assert abs(r.mean() - 1.0) < 4 * 0.5 / np.sqrt(d) and noise.min() >= 0      # folding at 2 sigma moves the mean by 0.0085
    f = 1.0 + nl.astype(F).sum(dtype=np.float64) / d * 0.5 * 12.0
    assert abs(tile.nl_factor(0) / f ** 2 - 1.0) < 1e-4
    assert len({tuple(np.round(v[:50], 7)) for v in (vo, nl, noise)}) == 3      # separate draws
    assert tile.get_lines(1, 0).shape == (2,)


def test_pos_neg_separate_passes():
    """Negative and positive inputs see the array one after the other; what is not linear in the inputs differs."""
    pns = dv.AnalogMVType.PosNegSeparate
    rng = np.random.default_rng(7)
    # everything linear: the two passes add up to the one pass
    w = rng.uniform(-0.6, 0.6, (5, 9)).astype(F)
    x = rng.uniform(-1, 1, (6, 9)).astype(F)
    one, two = oracle_tile(9, 5, w), oracle_tile(9, 5, w, mv_type=pns)
    np.testing.assert_allclose(two.forward(x), one.forward(x), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(two.forward(x), x @ w.T, rtol=1e-5, atol=1e-6)
    # series resistance acts on the current of each pass: w = [1, 1], x = [0.8, -0.3]
    kw = dict(r_series=0.5, slope_calibration=0.0)
    xs = np.array([[0.8, -0.3]], dtype=F)
    assert abs(oracle_tile(2, 1, [[1.0, 1.0]], **kw).forward(xs)[0, 0] - 0.5 / 1.25) < 1e-6
    want = 0.8 / 1.4 - 0.3 / 1.15
    assert abs(oracle_tile(2, 1, [[1.0, 1.0]], mv_type=pns, **kw).forward(xs)[0, 0] - want) < 1e-6
    # IR drop of a constant tile with the first h lines at +v and the others at -v: each pass has its own total current
    n, h, wv, v, ratio = 10, 4, 0.5, 0.8, 30.0
    xs = np.full((1, n), -v, dtype=F)
    xs[0, :h] = v
    pos_w = np.array([1.0 - (1.0 - j / n) ** 2 for j in range(n)])

    def drop(a):
        return a * (a * (0.05 * a - 0.2) + 0.5)

    a_pos, a_neg = n / ratio * wv * v * h, n / ratio * wv * v * (n - h)
    want = (wv * v * h - drop(a_pos) * wv * v * pos_w[:h].sum()) + (-wv * v * (n - h) + drop(a_neg) * wv * v * pos_w[h:].sum())
    got = oracle_tile(n, 2, np.full((2, n), wv), mv_type=pns, ir_drop=1.0, ir_drop_g_ratio=ratio).forward(xs)[0]
    np.testing.assert_allclose(got, [want, want], rtol=3e-6)
    a_all = n / ratio * wv * v * n
    want_one = wv * v * (2 * h - n) - drop(a_all) * wv * v * (pos_w[:h].sum() - pos_w[h:].sum())
    got_one = oracle_tile(n, 2, np.full((2, n), wv), ir_drop=1.0, ir_drop_g_ratio=ratio).forward(xs)[0]
    np.testing.assert_allclose(got_one, [want_one, want_one], rtol=3e-6)
    assert abs(want - want_one) > 1e-2
    # one ADC for the sum: clipping and the non-linearity see both passes together
    t = oracle_tile(2, 1, [[1.0, 1.0]], mv_type=pns, out_bound=0.4, out_nonlinearity=0.4, slope_calibration=0.0)
    np.testing.assert_allclose(t.forward(np.array([[0.9, -0.7]], dtype=F))[0, 0], 0.2 / 1.2, rtol=1e-6)   # nl = 1
    t = oracle_tile(2, 1, [[1.0, 1.0]], mv_type=pns, out_bound=0.4)
    assert abs(t.forward(np.array([[0.9, -0.7]], dtype=F))[0, 0] - 0.2) < 1e-6   # each pass alone is beyond the bound
    assert t.forward(np.array([[0.9, -0.1]], dtype=F))[0, 0] == F(0.4)
    # weight noise is drawn for each pass: the variances of the passes add to the one-pass law
    d = 4000
    t = oracle_tile(3, d, np.zeros((d, 3)), mv_type=pns, w_noise=0.1, w_noise_type=dv.WeightNoiseType.AdditiveConstant)
    t.use_gauss_table(False)
    y = t.forward(np.array([[0.6, -0.8, 0.0]] * 10, dtype=F)).astype(np.float64) / 0.1
    assert abs(y.mean()) < 4 / np.sqrt(y.size) and abs(y.std() - 1) < 4 / np.sqrt(2 * y.size)
    # backward takes the same path
    t = oracle_tile(1, 2, [[1.0], [1.0]], mv_type=pns, **kw)
    assert abs(t.backward(np.array([[0.8, -0.3]], dtype=F))[0, 0] - (0.8 / 1.4 - 0.3 / 1.15)) < 1e-6


def test_pos_neg_separate_digital_sum():
    """Each pass through its own ADC stage, converted values added (R/rpu_forward_backward_pass.cpp:861-877): hand
    values where the analog sum and the digital sum differ."""
    pnsd = dv.AnalogMVType.PosNegSeparateDigitalSum
    pns = dv.AnalogMVType.PosNegSeparate
    # clipping per pass: 0.9 -> 0.4, -0.7 -> -0.4, sum 0 (the analog sum 0.2 fits the bound)
    xs = np.array([[0.9, -0.7]], dtype=F)
    assert oracle_tile(2, 1, [[1.0, 1.0]], mv_type=pnsd, out_bound=0.4).forward(xs)[0, 0] == 0.0
    assert abs(oracle_tile(2, 1, [[1.0, 1.0]], mv_type=pns, out_bound=0.4).forward(xs)[0, 0] - 0.2) < 1e-6
    # quantization per pass with step 0.25 (1 / 32 of the range of 8): 0.9 -> 1.0 and -0.3 -> -0.25 give 0.75; the analog sum 0.6 gives 0.5
    xs = np.array([[0.9, -0.3]], dtype=F)
    assert oracle_tile(2, 1, [[1.0, 1.0]], mv_type=pnsd, out_bound=4.0, out_res=1 / 32).forward(xs)[0, 0] == F(0.75)
    assert oracle_tile(2, 1, [[1.0, 1.0]], mv_type=pns, out_bound=4.0, out_res=1 / 32).forward(xs)[0, 0] == F(0.5)
    # the non-linearity acts on each pass: 0.9 / (1 + 0.4 * 0.9) - 0.7 / (1 + 0.4 * 0.7)
    xs = np.array([[0.9, -0.7]], dtype=F)
    t = oracle_tile(2, 1, [[1.0, 1.0]], mv_type=pnsd, out_bound=1.0, out_nonlinearity=0.4, slope_calibration=0.0)
    np.testing.assert_allclose(t.forward(xs)[0, 0], 0.9 / 1.36 - 0.7 / 1.28, rtol=1e-6)
    # bound management: a pass that saturates alone fails the test although the sum fits; with the upper bound only
    # tested (bm_test_negative_bound off) a negative pass beyond the lower bound does not
    bm = dict(out_bound=0.4, bound_management=dv.BoundManagementType.Iterative, noise_management=dv.NoiseManagementType.NONE)
    t = oracle_tile(2, 1, [[1.0, 1.0]], mv_type=pnsd, **bm)
    np.testing.assert_allclose(t.forward(np.array([[0.7, -0.6]], dtype=F))[0, 0], 0.1, atol=1e-6)   # 0.35 - 0.3 at half range, x 2
    assert t.bm_rounds(1)[0] == 2
    t = oracle_tile(2, 1, [[1.0, 1.0]], mv_type=pns, **bm)
    np.testing.assert_allclose(t.forward(np.array([[0.7, -0.6]], dtype=F))[0, 0], 0.1, atol=1e-6)
    assert t.bm_rounds(1)[0] == 1
    t = oracle_tile(2, 1, [[1.0, 1.0]], mv_type=pnsd, **bm)
    np.testing.assert_allclose(t.forward(np.array([[0.3, -0.7]], dtype=F))[0, 0], 2 * (0.15 - 0.35), atol=1e-6)
    assert t.bm_rounds(1)[0] == 2                                  # the negative pass failed the lower bound
    t = oracle_tile(2, 1, [[1.0, 1.0]], mv_type=pnsd, bm_test_negative_bound=False, **bm)
    np.testing.assert_allclose(t.forward(np.array([[0.3, -0.7]], dtype=F))[0, 0], 0.3 - 0.4, atol=1e-6)   # lower bound not tested
    assert t.bm_rounds(1)[0] == 1
    # output noise is drawn for each pass
    d = 4000
    t = oracle_tile(3, d, np.zeros((d, 3)), mv_type=pnsd, out_noise=0.1)
    t.use_gauss_table(False)
    y = t.forward(np.array([[0.6, -0.8, 0.0]] * 10, dtype=F)).astype(np.float64) / (0.1 * np.sqrt(2.0))
    assert abs(y.mean()) < 4 / np.sqrt(y.size) and abs(y.std() - 1) < 4 / np.sqrt(2 * y.size)


def test_read_asymmetry_of_the_negative_pass():
    pns = dv.AnalogMVType.PosNegSeparate
    # w = [1, 1], factors [2, 3], x = [0.8, -0.3]: only the negative input reads its weight through the factor
    t = oracle_tile(2, 1, [[1.0, 1.0]], mv_type=pns, w_read_asymmetry_dtod=0.1)
    assert t.get_lines(0, 3).shape == (2,) and t.get_lines(1, 3).shape == (2,)
    t.set_lines(0, 3, [2.0, 3.0])
    assert abs(t.forward(np.array([[0.8, -0.3]], dtype=F))[0, 0] - (0.8 - 0.9)) < 1e-6
    assert abs(t.forward(np.array([[-0.8, 0.3]], dtype=F))[0, 0] - (-1.6 + 0.3)) < 1e-6
    # the IR drop of the negative pass sees the scaled conductances too: one line, closed form with w -> 2 w
    n, ratio = 4, 10.0
    t = oracle_tile(n, 1, np.full((1, n), 0.5), mv_type=pns, w_read_asymmetry_dtod=0.1, ir_drop=1.0, ir_drop_g_ratio=ratio)
    t.set_lines(0, 3, np.full(n, 2.0))
    x = np.zeros((1, n), dtype=F)
    x[0, 2] = -0.6
    a = n / ratio * 1.0 * 0.6
    want = -0.6 * (1.0 - a * (a * (0.05 * a - 0.2) + 0.5) * (1.0 - (1.0 - 2 / n) ** 2))
    assert abs(t.forward(x)[0, 0] - want) < 1e-6
    # one pass does not read the factors; the drawn ones are 1 + dtod xi, both directions their own
    t = oracle_tile(2, 1, [[1.0, 1.0]], w_read_asymmetry_dtod=0.1)
    t.set_lines(0, 3, [2.0, 3.0])
    assert abs(t.forward(np.array([[0.8, -0.3]], dtype=F))[0, 0] - 0.5) < 1e-6
    t = oracle_tile(100, 100, np.zeros((100, 100)), mv_type=pns, w_read_asymmetry_dtod=0.2)
    f, b = t.get_lines(0, 3).astype(np.float64), t.get_lines(1, 3).astype(np.float64)
    assert abs(f.mean() - 1) < 4 * 0.2 / 100 + 0.2 * 0.03 and abs(f.std() / 0.2 - 1) < 0.05 and not np.array_equal(f, b)
    # backward: the factors keep the layout of the weights
    t = oracle_tile(1, 2, [[1.0], [1.0]], mv_type=pns, w_read_asymmetry_dtod=0.1)
    t.set_lines(1, 3, [2.0, 3.0])
    assert abs(t.backward(np.array([[0.8, -0.3]], dtype=F))[0, 0] - (0.8 - 0.9)) < 1e-6
