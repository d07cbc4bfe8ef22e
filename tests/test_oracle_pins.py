"""Pins the CPU oracle (oracle/rpu_oracle.cpp) to facts that do not come from the oracle itself:
hand-derived values, closed forms, textbook routines (numpy matmul), brute force on tiny cases and the
expected values the reference's own tests compute (cited per test).  Each case is chosen so that a
plausible slip (dropped term, wrong sign / index, transposed operand, wrong rounding) fails it.
"""
import numpy as np
import pytest

from aihwkit_amd.rpu_base import devices as dv
from helpers import constant_step, io_params, make_meta, noise_free_io, soft_bounds
from oracle_lib import OracleTile

NM, BM = dv.NoiseManagementType, dv.BoundManagementType


def orc_tile(meta, dev, x_size, d_size, w=None, lr=None):
    t = OracleTile(x_size, d_size, meta._config(dev))
    if w is not None:
        t.set_weights(np.asarray(w, np.float32))
    if lr is not None:
        t.set_learning_rate(lr)
    return t


def wide_device(**kw):
    base = dict(w_max=100.0, w_min=-100.0, w_max_dtod=0.0, w_min_dtod=0.0, dw_min_dtod=0.0, up_down_dtod=0.0,
                dw_min_std=0.0, construction_seed=1)
    base.update(kw)
    return constant_step(**base)


# ------------------------------------------------------------------------------------------------
# forward: DAC / ADC / noise management / bound management


def test_perfect_io_is_a_plain_matmul():
    # reference: tests/test_bindings_tiles.py:133-169 (forward = x W^T, backward = d W)
    rng = np.random.default_rng(0)
    meta = make_meta(io_params(is_perfect=True, out_scale=1.0), io_params(is_perfect=True))
    w = rng.standard_normal((6, 5)).astype(np.float32)
    t = orc_tile(meta, dv.IdealResistiveDeviceParameter(), 5, 6, w)
    x = rng.uniform(-1.2, 1.2, (4, 5)).astype(np.float32)
    d = rng.uniform(-0.1, 0.1, (4, 6)).astype(np.float32)
    assert np.allclose(t.forward(x), x @ w.T, atol=1e-6)
    assert np.allclose(t.backward(d), d @ w, atol=1e-6)
    # transposed layouts address the same numbers
    assert np.allclose(t.forward(np.ascontiguousarray(x.T), x_trans=True, d_trans=True), (x @ w.T).T, atol=1e-6)


@pytest.mark.parametrize("inp_bound,out_bound,inp_res,out_res,bm,want", [
    # x = 10, w = 1, no noise management (the reference's 1x1 case, tests/test_torch_tiles.py:232-272).
    # DAC: step = res*2*bound; 10 saturates at inp_bound.  ADC step = out_res*2*out_bound.
    (1.0, 10.0, 4, 4, BM.NONE, 0.0),        # y=1, ADC step 5: rint(0.2)=0
    (1.0, 10.0, 4, 16, BM.NONE, 1.25),      # ADC step 1.25: rint(0.8)=1
    (1.0, 1.0, -1, -1, BM.NONE, 1.0),       # no quantization, no clipping needed
    (10.0, 1.0, -1, -1, BM.NONE, 1.0),      # xq = 10, output clipped to out_bound
    (10.0, 0.1, 16, -1, BM.NONE, 0.1),
    (0.1, 10.0, -1, 16, BM.NONE, 0.0),      # y = 0.1, ADC step 1.25: rint(0.08) = 0
    # iterative BM: inp_res = 1/4 of range 2*10 -> step 5; limit = 0.25/5 < 1: a single round, clipped
    (10.0, 1.0, 4, -1, BM.Iterative, 1.0),
    # no DAC quantization (no resolution limit): halve until rint fits: 10 -> 5 -> 2.5 -> 1.25 -> 0.625 <= 1
    # result is rescaled by the reduction 16: 0.625 * 16 = 10
    (10.0, 1.0, -1, -1, BM.Iterative, 10.0),
    # same with a 16-level ADC on [-1, 1] (step 0.125): 0.625 is on the grid
    (10.0, 1.0, -1, 16, BM.Iterative, 10.0),
])
def test_one_by_one_tile_hand_values(inp_bound, out_bound, inp_res, out_res, bm, want):
    f_io = noise_free_io(inp_bound=inp_bound, out_bound=out_bound, inp_res=inp_res, out_res=out_res,
                         noise_management=NM.NONE, bound_management=bm)
    t = orc_tile(make_meta(f_io), wide_device(), 1, 1, [[1.0]])
    assert t.forward(np.array([[10.0]], np.float32))[0, 0] == pytest.approx(want, abs=1e-6)


def test_dac_rounds_half_to_even_and_clips_after_rounding():
    # step = (1/8) * 2 * 2 = 0.5 ; identity weights expose the quantized inputs
    f_io = noise_free_io(inp_bound=2.0, inp_res=1 / 8.0, out_res=-1, out_bound=100.0, noise_management=NM.NONE)
    t = orc_tile(make_meta(f_io), wide_device(), 6, 6, np.eye(6))
    x = np.array([[1.25, 0.75, -1.25, 1.76, 5.0, -0.24]], np.float32)
    #            2.5->2   1.5->2  -2.5->-2  3.52->4  clip  -0.48->0
    assert np.array_equal(t.forward(x)[0], np.array([1.0, 1.0, -1.0, 2.0, 2.0, -0.0], np.float32))


def test_abs_max_noise_management_scales_in_and_out():
    # y_i = nm * q(x_i / nm), q = 7-bit DAC on [-1, 1]; brute force in float64 away from rounding edges
    f_io = noise_free_io(out_res=-1, out_bound=1e6, noise_management=NM.AbsMax)
    t = orc_tile(make_meta(f_io), wide_device(), 4, 4, np.eye(4))
    x = np.array([[0.5, -2.0, 1.0, 0.2], [0.0, 0.0, 0.0, 0.0], [3.0, 3.0, -3.0, 1.4]], np.float32)
    step = 2.0 / 126.0
    want = np.zeros_like(x, dtype=np.float64)
    for b in range(3):
        nm = np.abs(x[b]).max()
        if nm > 0:
            want[b] = np.rint(x[b] / nm / step) * step * nm
    assert np.allclose(t.forward(x), want, atol=1e-6)
    assert np.array_equal(t.forward(x)[1], np.zeros(4, np.float32))  # zero input short-cut
    # nm_thres caps the scale: inputs above it saturate at +-1 * thres
    f_io2 = noise_free_io(out_res=-1, out_bound=1e6, noise_management=NM.AbsMax, nm_thres=1.0)
    t2 = orc_tile(make_meta(f_io2), wide_device(), 4, 4, np.eye(4))
    assert np.allclose(t2.forward(x)[2], [1.0, 1.0, -1.0, 1.0], atol=1e-6)
    # constant and max variants (tests/test_torch_tiles.py:438-485 sweeps the same modes)
    f_io3 = noise_free_io(out_res=-1, out_bound=1e6, noise_management=NM.Constant, nm_thres=2.0)
    t3 = orc_tile(make_meta(f_io3), wide_device(), 4, 4, np.eye(4))
    assert np.allclose(t3.forward(x)[0], np.rint(x[0] / 2.0 / step) * step * 2.0, atol=1e-6)
    f_io4 = noise_free_io(out_res=-1, out_bound=1e6, noise_management=NM.Max)
    t4 = orc_tile(make_meta(f_io4), wide_device(), 4, 4, np.eye(4))
    assert np.allclose(t4.forward(x)[0], np.clip(np.rint(x[0] / 1.0 / step) * step, -1, 1), atol=1e-6)


def test_contraction_is_w_times_x_not_its_transpose():
    rng = np.random.default_rng(1)
    f_io = noise_free_io(inp_res=-1, out_res=-1, out_bound=1e6, inp_bound=1.0, noise_management=NM.AbsMax)
    meta = make_meta(f_io, noise_free_io(inp_res=-1, out_res=-1, out_bound=1e6, noise_management=NM.AbsMax))
    w = rng.standard_normal((3, 7)).astype(np.float32)
    t = orc_tile(meta, wide_device(), 7, 3, w)
    x = rng.uniform(-1, 1, (5, 7)).astype(np.float32)
    d = rng.uniform(-1, 1, (5, 3)).astype(np.float32)
    assert np.allclose(t.forward(x), x @ w.T, atol=1e-5)
    assert np.allclose(t.backward(d), d @ w, atol=1e-5)
    xb = np.concatenate([x[:, :6], np.ones((5, 1), np.float32)], axis=1)
    assert np.allclose(t.forward(x[:, :6], bias=True), xb @ w.T, atol=1e-5)
    assert np.allclose(t.backward(d, bias=True), (d @ w)[:, :6], atol=1e-5)


def test_iterative_bound_management_rounds_and_limits():
    # W = 4 * ones(1, 4), x = ones: y = 16 * scale ; out_bound 12 ; DAC step 1/64 (exact in binary).
    f_io = noise_free_io(noise_management=NM.AbsMax, bound_management=BM.Iterative, out_res=-1, inp_res=1 / 128.0)
    t = orc_tile(make_meta(f_io), wide_device(), 4, 1, np.full((1, 4), 4.0))
    x = np.ones((1, 4), np.float32)
    y = t.forward(x)
    # round 1: 16 > 12 fails; round 2: x/2 = 0.5 is on the DAC grid -> y = 8 ok; rescaled by the reduction 2
    assert t.bm_rounds(1)[0] == 2
    assert y[0, 0] == pytest.approx(16.0, abs=1e-5)
    # a sample that can never fit stops when the reduction exceeds max_bm_res / inp_step = 16: rounds with
    # reduction 1, 2, 4, 8, 16, 32 = 6 rounds, output = clip * 32
    t2 = orc_tile(make_meta(f_io), wide_device(), 4, 1, np.full((1, 4), 900.0))
    y2 = t2.forward(x)
    assert t2.bm_rounds(1)[0] == 6
    assert y2[0, 0] == pytest.approx(12.0 * 32.0, abs=1e-4)
    # with the default 7-bit DAC (step 2/126) the limit is 15.75: reductions 1 .. 16 = 5 rounds
    f_io7 = noise_free_io(noise_management=NM.AbsMax, bound_management=BM.Iterative, out_res=-1)
    t7 = orc_tile(make_meta(f_io7), wide_device(), 4, 1, np.full((1, 4), 900.0))
    assert t7.forward(x)[0, 0] == pytest.approx(12.0 * 16.0, abs=1e-4) and t7.bm_rounds(1)[0] == 5
    # max_bm_factor caps the reduction when there is no DAC resolution: (int) red > 2 stops at red = 4
    f_io3 = noise_free_io(noise_management=NM.AbsMax, bound_management=BM.Iterative, out_res=-1, inp_res=-1,
                          max_bm_factor=2)
    t3 = orc_tile(make_meta(f_io3), wide_device(), 4, 1, np.full((1, 4), 90.0))
    y3 = t3.forward(x)
    assert t3.bm_rounds(1)[0] == 3
    assert y3[0, 0] == pytest.approx(12.0 * 4.0, abs=1e-4)
    # the negative bound also triggers, unless bm_test_negative_bound is off
    t4 = orc_tile(make_meta(f_io), wide_device(), 4, 1, np.full((1, 4), -4.0))
    t4.forward(x)
    assert t4.bm_rounds(1)[0] == 2
    f_io5 = noise_free_io(noise_management=NM.AbsMax, bound_management=BM.Iterative, out_res=-1,
                          bm_test_negative_bound=False)
    t5 = orc_tile(make_meta(f_io5), wide_device(), 4, 1, np.full((1, 4), -4.0))
    assert t5.forward(x)[0, 0] == pytest.approx(-12.0, abs=1e-5)
    assert t5.bm_rounds(1)[0] == 1


def test_backward_never_iterates_and_rescales_by_the_abs_max():
    b_io = noise_free_io(noise_management=NM.AbsMax, bound_management=BM.Iterative, out_res=-1)
    t = orc_tile(make_meta(None, b_io), wide_device(), 1, 4, np.full((4, 1), 4.0))
    d = np.full((1, 4), 2.0, np.float32)
    # d / 2 = 1 -> exact on the DAC grid; sum = 16 clipped to 12; times nm = 2
    assert t.backward(d)[0, 0] == pytest.approx(24.0, abs=1e-5)


def test_output_noise_statistics_and_out_scale():
    # no quantization: y = out_scale * nm * (w.x/nm + out_noise * xi)
    f_io = io_params(out_noise=0.1, inp_res=-1, out_res=-1, out_bound=1e6, noise_management=NM.AbsMax, out_scale=3.0)
    t = orc_tile(make_meta(f_io), wide_device(), 2, 1, [[0.5, 0.25]])
    t.use_gauss_table(False)
    t.set_seed(5)
    x = np.tile(np.array([[2.0, -1.0]], np.float32), (20000, 1))
    y = t.forward(x)[:, 0]
    assert y.mean() == pytest.approx(3.0 * (0.5 * 2.0 - 0.25), abs=4 * 0.6 / np.sqrt(20000))
    assert y.std() == pytest.approx(3.0 * 2.0 * 0.1, rel=0.03)


# ------------------------------------------------------------------------------------------------
# update


def test_bl_and_probability_scales_closed_form():
    meta = make_meta(desired_bl=31, update_management=False, update_bl_management=False)
    t = orc_tile(meta, wide_device(dw_min=0.001), 4, 3, lr=0.01)
    x = np.array([[1.0, -0.5, 0.25, 0.0], [0.0, 0.0, 0.0, 0.0]], np.float32)
    d = np.array([[0.16, -0.08, 0.0], [0.1, 0.1, 0.1]], np.float32)
    bl, a, b = t.update_bl_ab(x, d)
    assert list(bl) == [31, 31]
    assert a[0] == pytest.approx(np.sqrt(0.01 / (0.001 * 31)), rel=1e-6) and b[0] == a[0]
    # update management + BL management (rpu_pulsed_meta_parameter.cpp:183-236):
    # k = lr*xmax*dmax/dw_min = 1.6 -> BL = 2 ; A = sqrt(lr/(dw_min*BL)) * sqrt(xmax/dmax), B likewise inverted
    meta2 = make_meta(desired_bl=31, update_management=True, update_bl_management=True)
    t2 = orc_tile(meta2, wide_device(dw_min=0.001), 4, 3, lr=0.01)
    bl, a, b = t2.update_bl_ab(x, d)
    assert list(bl) == [2, 0]  # a zero x sample sends no pulses
    assert a[0] == pytest.approx(np.sqrt(5.0) * 2.5, rel=1e-5)
    assert b[0] == pytest.approx(np.sqrt(5.0) * 0.4, rel=1e-5)
    # probabilities at the abs-max entries: B*xmax * A*dmax * BL = k  (expected coincidences = lr*x*d/dw_min)
    assert a[0] * 0.16 * b[0] * 1.0 * 2 == pytest.approx(1.6, rel=1e-5)
    # k > max BL: the d side is clipped so that the x probability stays <= 1
    t3 = orc_tile(meta2, wide_device(dw_min=0.001), 4, 3, lr=1.0)
    bl, a, b = t3.update_bl_ab(x, d)
    assert bl[0] == 31
    assert b[0] * 1.0 == pytest.approx(1.0, rel=1e-5)  # p(x_max) = 1
    assert a[0] * 0.16 == pytest.approx(160.0 / 31.0, rel=1e-5)


def test_all_ones_update_is_deterministic():
    # tests/test_bindings_tiles.py:307-373 protocol: x = d = 1, lr = 1, noise-free ConstantStep, UM + UBLM:
    # every pulse probability is >= 1, so each sample gives BL coincidences, all "down".
    in_size, out_size, m_batch, bl = 32, 16, 128, 31
    meta = make_meta(io_params(is_perfect=True), io_params(is_perfect=True), desired_bl=bl)
    dev = constant_step(dw_min=2 / 12000, w_max=1.0, w_min=-1.0, w_max_dtod=0.0, w_min_dtod=0.0, up_down_dtod=0.0,
                        dw_min_dtod=0.0, dw_min_std=0.0, construction_seed=3)
    t = orc_tile(meta, dev, in_size, out_size, np.zeros((out_size, in_size)), lr=1.0)
    t.update(np.ones((m_batch, in_size), np.float32), np.ones((m_batch, out_size), np.float32))
    assert np.allclose(t.get_weights(), -bl * m_batch * (2 / 12000), atol=1e-4)  # 3968 fp32 additions
    # and it saturates at the lower bound
    for _ in range(2):
        t.update(np.ones((m_batch, in_size), np.float32), np.ones((m_batch, out_size), np.float32))
    assert np.allclose(t.get_weights(), -1.0, atol=1e-6)


def _reference_scalar_word_model(x_words, d_words):
    """Coincidences and direction of one sample as the reference's test model computes them
    (src/rpucuda/cuda/pulsed_weight_updater_test.cpp:51-69): n = popcount(x & d) minus the shared sign bit,
    direction = xor of the sign bits."""
    xw = x_words.astype(np.int64)[None, :]
    dw = d_words.astype(np.int64)[:, None]
    both = xw & dw
    n = np.zeros(both.shape, np.int64)
    for bit in range(32):
        n += (both >> bit) & 1
    n -= both & 1
    negative = (xw ^ dw) & 1
    return n, negative


def test_packed_words_drive_constant_step_like_the_scalar_model():
    rng = np.random.default_rng(4)
    x_size, d_size, batch = 9, 7, 6
    meta = make_meta(desired_bl=31)
    dev = wide_device(dw_min=0.01)
    w0 = rng.uniform(-0.3, 0.3, (d_size, x_size)).astype(np.float32)
    t = orc_tile(meta, dev, x_size, d_size, w0, lr=0.1)
    xw = rng.integers(0, 2**32, (batch, x_size), dtype=np.uint64).astype(np.uint32)
    dw = rng.integers(0, 2**32, (batch, d_size), dtype=np.uint64).astype(np.uint32)
    bl = np.full(batch, 31, np.int32)
    t.update_with_words(xw, dw, bl)
    want = w0.astype(np.float64)
    for b in range(batch):
        n, negative = _reference_scalar_word_model(xw[b], dw[b])
        # negative (signs differ) steps up, otherwise down (w -= lr x d for same-sign x and d)
        want += np.where(negative == 1, 1.0, -1.0) * n * 0.01
    assert np.allclose(t.get_weights(), want, atol=1e-5)
    # a shorter BL ignores the higher pulse bits
    t2 = orc_tile(meta, dev, x_size, d_size, w0, lr=0.1)
    t2.update_with_words(xw, dw, np.full(batch, 3, np.int32))
    want = w0.astype(np.float64)
    for b in range(batch):
        n, negative = _reference_scalar_word_model(xw[b] & np.uint32(0xF), dw[b] & np.uint32(0xF))
        want += np.where(negative == 1, 1.0, -1.0) * n * 0.01
    assert np.allclose(t2.get_weights(), want, atol=1e-5)


def test_negative_learning_rate_flips_the_direction():
    meta = make_meta(desired_bl=31)
    t = orc_tile(meta, wide_device(dw_min=0.01), 1, 1, [[0.0]], lr=-0.1)
    t.update_with_words(np.array([[0b1110]], np.uint32), np.array([[0b0110]], np.uint32), np.array([31], np.int32))
    assert t.get_weights()[0, 0] == pytest.approx(+0.02, abs=1e-6)  # 2 coincidences, same signs, lr < 0: up


def test_stochastic_update_mean_is_the_sgd_step():
    # E[coincidences] = BL * (B|x|) * (A|d|) = lr |x d| / dw_min  =>  E[dW] = -lr * d x^T for a noise-free
    # ConstantStep device with probabilities below 1.
    rng = np.random.default_rng(2)
    x_size, d_size = 5, 4
    meta = make_meta(desired_bl=31, update_management=False, update_bl_management=False)
    t = orc_tile(meta, wide_device(dw_min=0.001), x_size, d_size, np.zeros((d_size, x_size)), lr=0.01)
    t.set_seed(12)
    x = rng.uniform(-1, 1, (1, x_size)).astype(np.float32)
    d = rng.uniform(-1, 1, (1, d_size)).astype(np.float32)
    reps = 4000
    t.update(np.repeat(x, reps, 0), np.repeat(d, reps, 0))
    got = t.get_weights() / reps
    want = -0.01 * d.T @ x
    # one sample: BL Bernoulli(p) trials; std of the mean is below dw_min * sqrt(BL * 0.25 / reps)
    assert np.abs(got - want).max() < 5 * 0.001 * np.sqrt(31 * 0.25 / reps)


def test_soft_bounds_noise_free_run_is_geometric():
    # up pulses: w += scale_up (1 - w / w_max)  =>  (w_max - w_n) = (w_max - w_0) (1 - scale_up / w_max)^n
    meta = make_meta(desired_bl=31)
    dev = soft_bounds(dw_min=0.01, dw_min_dtod=0.0, dw_min_std=0.0, up_down_dtod=0.0, w_max=0.6, w_min=-0.6,
                      w_max_dtod=0.0, w_min_dtod=0.0, construction_seed=2)
    t = orc_tile(meta, dev, 1, 1, [[0.1]], lr=0.1)
    hidden = t.get_hidden()
    assert hidden[8, 0, 0] == pytest.approx(-0.01 / 0.6, rel=1e-6)   # slope_up = -scale_up / w_max
    assert hidden[9, 0, 0] == pytest.approx(-0.01 / -0.6, rel=1e-6)  # slope_down = -scale_down / w_min
    up = (np.array([[0xFFFFFFFE]], np.uint32), np.array([[0xFFFFFFFF]], np.uint32))  # signs differ: up
    t.update_with_words(*up, np.array([31], np.int32))
    assert t.get_weights()[0, 0] == pytest.approx(0.6 - 0.5 * (1 - 0.01 / 0.6) ** 31, abs=1e-6)
    w1 = float(t.get_weights()[0, 0])
    down = (np.array([[0xFFFFFFFE]], np.uint32), np.array([[0x000000FE]], np.uint32))  # same signs: 7 down
    t.update_with_words(*down, np.array([31], np.int32))
    assert t.get_weights()[0, 0] == pytest.approx(-0.6 + (w1 + 0.6) * (1 - 0.01 / 0.6) ** 7, abs=1e-6)


def test_constant_step_clips_at_the_device_bounds_and_set_weights_clips():
    meta = make_meta(desired_bl=31)
    dev = constant_step(dw_min=0.1, dw_min_dtod=0.0, dw_min_std=0.0, up_down_dtod=0.0, w_max=0.6, w_min=-0.6,
                        w_max_dtod=0.0, w_min_dtod=0.0, construction_seed=2)
    t = orc_tile(meta, dev, 2, 1, [[5.0, -5.0]], lr=0.1)
    assert np.allclose(t.get_weights(), [[0.6, -0.6]])
    t.update_with_words(np.array([[0xFFFFFFFE, 0xFFFFFFFE]], np.uint32), np.array([[0xFFFFFFFE]], np.uint32),
                        np.array([31], np.int32))
    assert np.allclose(t.get_weights(), [[-0.6, -0.6]])  # 31 down steps of 0.1 from 0.6 end at the bound


def test_cycle_to_cycle_noise_moments():
    # n pulses of size scale * (1 + std * xi): mean n * scale, variance n * (scale * std)^2
    meta = make_meta(desired_bl=31)
    dev = wide_device(dw_min=0.01, dw_min_std=0.3)
    n_dev = 4000
    t = orc_tile(meta, dev, n_dev, 1, np.zeros((1, n_dev)), lr=0.1)
    t.use_gauss_table(False)
    t.set_seed(9)
    xw = np.full((1, n_dev), 0x000003FE, np.uint32)  # 9 pulses
    t.update_with_words(xw, np.array([[0xFFFFFFFF]], np.uint32), np.array([31], np.int32))
    w = t.get_weights()[0]
    assert w.mean() == pytest.approx(9 * 0.01, abs=4 * 0.009 / np.sqrt(n_dev))
    assert w.std() == pytest.approx(np.sqrt(9) * 0.01 * 0.3, rel=0.06)


def test_deterministic_implicit_counts_brute_force():
    # n_ij = rint((dv_i * BL) * xv_j) with xv = clip(disc(|x| B), 0, 1) * sign (dense_bit_line_maker.cpp:209-264)
    meta = make_meta(desired_bl=10, pulse_type=dv.PulseType.DeterministicImplicit, update_management=False,
                     update_bl_management=False, x_res_implicit=0.25, d_res_implicit=0.5)
    lr, dw_min = 0.1, 0.01  # A = B = sqrt(lr / (dw_min * BL)) = 1
    t = orc_tile(meta, wide_device(dw_min=dw_min), 4, 3, np.zeros((3, 4)), lr=lr)
    x = np.array([[0.6, -0.3, 2.0, 0.1]], np.float32)   # -> 0.5, -0.25, 1 (clipped), 0
    d = np.array([[0.7, -0.2, 1.3]], np.float32)        # -> 0.5, 0 (rint(0.4)=0), 1 (2.6 -> rint 3 -> 1.5 -> clip 1)
    counts = t.implicit_counts(x, d)[0]
    xv = np.array([0.5, -0.25, 1.0, 0.0])
    dvv = np.array([0.5, 0.0, 1.0])
    want = np.rint((dvv[:, None] * 10) * xv[None, :]).astype(np.int32)  # 2.5 -> 2, -1.25 -> -1, 5, 0 / 5, -2 (2.5 -> -2), 10
    assert np.array_equal(counts, want)
    assert counts[0, 0] == 2 and counts[2, 1] == -2 and counts[2, 2] == 10  # half-to-even
    t.update(x, d)
    assert np.allclose(t.get_weights(), -want * dw_min, atol=1e-6)  # positive count = down


def test_floating_point_update_is_rank_b_sgd():
    # tests/test_bindings_tiles.py:161-167: W <- W - lr d^T x
    rng = np.random.default_rng(6)
    meta = make_meta(io_params(is_perfect=True), io_params(is_perfect=True), pulse_type=dv.PulseType.NONE)
    w = rng.standard_normal((6, 5)).astype(np.float32)
    t = orc_tile(meta, dv.IdealResistiveDeviceParameter(), 5, 6, w, lr=0.1)
    x = rng.uniform(-1.2, 1.2, (4, 5)).astype(np.float32)
    d = rng.uniform(-0.1, 0.1, (4, 6)).astype(np.float32)
    t.update(x, d)
    assert np.allclose(t.get_weights(), w - 0.1 * d.T @ x, atol=1e-6)


# ------------------------------------------------------------------------------------------------
# device construction (the draw order is pinned in test_draw_order_pins.py; these pin distributions and relations)


def test_populated_arrays_have_the_configured_distributions_and_relations():
    meta = make_meta()
    dev = soft_bounds(construction_seed=123, enforce_consistency=True)
    t = orc_tile(meta, dev, 300, 200)
    h = t.get_hidden()
    w_max, w_min, up, down, decay, diff, reset, nu, slope_up, slope_down = h
    n = w_max.size
    # w_max = |0.6 (1 + 0.3 xi)|: mean 0.6, std 0.18 (folding at 0 is a 3.3 sigma event)
    assert w_max.mean() == pytest.approx(0.6, abs=5 * 0.18 / np.sqrt(n)) and w_max.std() == pytest.approx(0.18, rel=0.03)
    assert w_min.mean() == pytest.approx(-0.6, abs=5 * 0.18 / np.sqrt(n)) and np.all(w_min <= 0) and np.all(w_max >= 0)
    # scale_up/down = dw_min (1 + 0.3 xi +- 0.01 xi'): mean 1e-3, std 3e-4, difference std 2e-5
    assert up.mean() == pytest.approx(1e-3, abs=5 * 3e-4 / np.sqrt(n)) and up.std() == pytest.approx(3e-4, rel=0.03)
    assert (up - down).std() == pytest.approx(2e-5, rel=0.05) and np.all(up >= 0) and np.all(down >= 0)
    assert np.all(decay == 1.0) and np.all(diff == 0.0) and np.all(reset == 0.0) and np.all(nu == 0.0)
    assert np.allclose(slope_up, -up / w_max, rtol=1e-6) and np.allclose(slope_down, -down / w_min, rtol=1e-6)
    # the four draws of a cross-point are independent
    assert abs(np.corrcoef(w_max.ravel(), up.ravel())[0, 1]) < 0.03
    # same seed, same arrays; other seed, other arrays
    assert np.array_equal(orc_tile(meta, dev, 300, 200).get_hidden(), h)
    assert not np.array_equal(orc_tile(meta, soft_bounds(construction_seed=124, enforce_consistency=True), 300, 200).get_hidden(), h)


def test_inconsistent_bounds_collapse_without_enforce_consistency():
    dev = constant_step(w_max=0.01, w_max_dtod=5.0, w_min=-0.01, w_min_dtod=5.0, construction_seed=8, enforce_consistency=False)
    h = orc_tile(make_meta(), dev, 50, 50).get_hidden()
    assert np.all(h[1] <= h[0])  # w_min <= w_max everywhere: crossed draws collapse onto their midpoint
    assert (h[1] == h[0]).mean() > 0.2
