"""Pins of the transfer-compound oracle (oracle/transfer_oracle.py) by closed forms and invariants; CPU only.

A dropped sign, a wrong column, a transposed read, a counter that is off by one or a mixed-up learning
rate each fail one of these."""
import numpy as np
import pytest

from aihwkit_amd.rpu_base import devices as dv
from helpers import build_transfer_pair, constant_step, make_meta, noise_free_io, transfer_param

PT = dv.PulseType


def quiet_device(**kw):
    base = dict(dw_min=0.01, dw_min_dtod=0.0, dw_min_std=0.0, up_down_dtod=0.0, w_max_dtod=0.0, w_min_dtod=0.0,
                w_max=1.0, w_min=-1.0, reset_std=0.0, construction_seed=1)
    base.update(kw)
    return constant_step(**base)


def exact_transfer(x_size=4, d_size=3, bl=10, **kw):
    """Deterministic pulses, no variation, perfect read: a transfer adds lr_t * column exactly (in dw_min steps)."""
    meta = make_meta(noise_free_io(), noise_free_io(), pulse_type=PT.DeterministicImplicit, desired_bl=bl,
                     update_management=False, update_bl_management=False)
    tr = transfer_param([quiet_device(), quiet_device()], **kw)
    tr.transfer_forward.is_perfect = True
    tr.transfer_update.pulse_type = PT.DeterministicImplicit
    tr.transfer_update.desired_bl = bl
    tr.transfer_update.update_management = False
    tr.transfer_update.update_bl_management = False
    _, orc, _ = build_transfer_pair(meta, tr, x_size, d_size, gpu=False)
    return orc


def test_gradient_goes_to_the_first_device_only_and_hidden_weights_stay():
    orc = exact_transfer(transfer_every=1000.0)
    orc.set_learning_rate(0.1)  # = dw_min * BL: A = B = 1, n = rint(|d| BL |x|)
    x = np.array([[1.0, 0.0, -0.5, 0.0]], np.float32)
    d = np.array([[0.4, -0.2, 0.0]], np.float32)
    orc.update(x, d)
    want = -0.1 * np.outer(d[0], x[0])  # SGD: W -= lr d x^T, here exactly on the dw_min grid
    assert np.allclose(orc.device_weights(0), want, atol=1e-6)
    assert np.all(orc.device_weights(1) == 0) and np.all(orc.get_weights() == 0)  # gamma = 0: only C is visible


def test_transfer_adds_the_read_column_times_lr_and_nothing_else():
    orc = exact_transfer(transfer_every=1.0, transfer_lr=1.0, scale_transfer_lr=False)
    a = np.array([[0.3, -0.2, 0.1, 0.0], [0.5, 0.4, -0.3, 0.2], [-0.1, 0.0, 0.2, -0.4]], np.float32)
    orc.set_device_weights(0, a)
    orc.set_learning_rate(0.1)
    zeros_x, zeros_d = np.zeros((1, 4), np.float32), np.zeros((1, 3), np.float32)
    # lr_t = 1 with dw_min * BL = 0.1: BL management off -> A = B = sqrt(1 / 0.1), clipped probabilities;
    # use lr_t = 0.1 instead through the vector of learning rates
    orc.lr_vec = [0.1, 0.1]
    orc.update(zeros_x, zeros_d)  # one vector, no gradient: counter 1 -> transfer of column 0
    c = orc.device_weights(1)
    assert np.allclose(c[:, 0], 0.1 * a[:, 0], atol=1e-6)  # + lr_t * A[:, 0]: sign and column
    assert np.all(c[:, 1:] == 0)
    assert np.array_equal(orc.device_weights(0), a)        # reading does not change A
    assert np.array_equal(orc.get_weights(), c)            # fully hidden: the tile's weights are C
    orc.update(zeros_x, zeros_d)
    c = orc.device_weights(1)
    assert np.allclose(c[:, 1], 0.1 * a[:, 1], atol=1e-6) and np.all(c[:, 2:] == 0)
    assert orc.slice_idx[0] == 2 and orc.update_idx == 2


def test_row_transfer_reads_rows_with_the_backward_pass():
    orc = exact_transfer(transfer_every=1.0, transfer_columns=False)
    a = np.array([[0.3, -0.2, 0.1, 0.0], [0.5, 0.4, -0.3, 0.2], [-0.1, 0.0, 0.2, -0.4]], np.float32)
    orc.set_device_weights(0, a)
    orc.set_learning_rate(0.1)
    orc.lr_vec = [1.0, 1.0]  # scaled by the current lr 0.1
    orc.update(np.zeros((1, 4), np.float32), np.zeros((1, 3), np.float32))
    c = orc.device_weights(1)
    assert np.allclose(c[0], 0.1 * a[0], atol=1e-6) and np.all(c[1:] == 0)


@pytest.mark.parametrize("units_in_mbatch,every,batch,n_updates,expected_transfers", [
    (False, 3.0, 4, 3, 4),   # 12 vectors, one transfer every 3
    (True, 2.0, 4, 5, 2),    # every 2 mini-batches of 4 = 8 vectors: after 8 and 16 of 20
    (True, 0.5, 4, 2, 4),    # every half mini-batch = ceil(0.5 * 4) = 2 vectors
])
def test_transfer_schedule_counts_update_vectors(units_in_mbatch, every, batch, n_updates, expected_transfers):
    orc = exact_transfer(x_size=5, transfer_every=every, units_in_mbatch=units_in_mbatch, n_reads_per_transfer=2)
    orc.set_learning_rate(0.1)
    rng = np.random.default_rng(0)
    for _ in range(n_updates):
        orc.update(rng.uniform(-1, 1, (batch, 5)).astype(np.float32), rng.uniform(-1, 1, (batch, 3)).astype(np.float32))
    assert orc.update_idx == batch * n_updates
    assert orc.slice_idx[0] == (2 * expected_transfers) % 5   # two columns per transfer, cyclic
    assert orc.slice_idx[1] == 0                               # the last device does not transfer onto itself


def test_gamma_mixes_the_devices_and_set_weights_resets():
    orc = exact_transfer(transfer_every=2.0, gamma=0.5)
    assert [float(g) for g in orc.gamma_vec] == [0.5, 1.0] and not orc.fully_hidden
    orc.set_learning_rate(0.1)
    x = np.array([[1.0, 0.0, 0.0, 1.0]], np.float32)
    d = np.array([[0.5, 0.0, -0.5]], np.float32)
    orc.update(x, d)
    a, c = orc.device_weights(0), orc.device_weights(1)
    assert np.allclose(orc.get_weights(), 0.5 * a + c, atol=1e-7) and np.abs(a).max() > 0
    w = np.full((3, 4), 0.25, np.float32)
    w[0, 0] = 5.0
    orc.set_weights(w)
    assert np.all(orc.device_weights(0) == 0)
    c = orc.device_weights(1)
    assert c[0, 0] == 1.0 and np.all(c.flatten()[1:] == 0.25)   # W / gamma_last, clipped into the device bounds
    assert orc.update_idx == 0 and orc.slice_idx == [0, 0]


def test_fast_learning_rate_options():
    for fast_lr, scale, expected in [(0.0, True, 0.1), (0.5, True, 0.05), (0.2, False, 0.2)]:
        orc = exact_transfer(transfer_every=1000.0, fast_lr=fast_lr, scale_fast_lr=scale, bl=20)
        orc.set_learning_rate(0.1)
        orc.update(np.array([[1.0, 0, 0, 0]], np.float32), np.array([[1.0, 0, 0]], np.float32))
        # BL management off: A = B = sqrt(lr / (dw_min BL)), n = rint(BL A B) = lr / dw_min pulses of dw_min
        assert orc.device_weights(0)[0, 0] == pytest.approx(-expected, abs=1e-6)


def test_random_selection_and_reset_after_a_transfer():
    """random_selection: the transfer starts at column floor(u * in_size), clamped, and the running index follows it
    (R/rpu_transfer_device.cpp:486-488, 515).  with_reset_prob: when the lottery wins, the columns that were read are
    back at their reset values on the source device AFTER the destination took the values they had
    (C/rpucuda_transfer_device.cu:320-324); the other columns and a lost lottery change nothing."""
    a = np.array([[0.3, -0.2, 0.1, 0.0], [0.5, 0.4, -0.3, 0.2], [-0.1, 0.0, 0.2, -0.4]], np.float32)
    zeros_x, zeros_d = np.zeros((1, 4), np.float32), np.zeros((1, 3), np.float32)
    for u, start in ((0.0, 0), (0.5, 2), (0.74, 2), (0.75, 3), (0.99999994, 3)):
        orc = exact_transfer(transfer_every=1.0, scale_transfer_lr=False, random_selection=True, n_reads_per_transfer=2)
        orc.select = lambda idx, frm, u=u: u
        orc.set_device_weights(0, a)
        orc.set_learning_rate(0.1)
        orc.lr_vec = [0.1, 0.1]
        orc.update(zeros_x, zeros_d)
        c = orc.device_weights(1)
        cols = [start, (start + 1) % 4]
        rest = [j for j in range(4) if j not in cols]
        assert np.allclose(c[:, cols], 0.1 * a[:, cols], atol=1e-6) and np.all(c[:, rest] == 0), (u, c)
        assert orc.slice_idx[0] == (start + 2) % 4
    for lottery, wins in ((0.2, True), (0.3, False)):
        orc = exact_transfer(transfer_every=1.0, scale_transfer_lr=False, with_reset_prob=0.3, n_reads_per_transfer=2)
        asked = []
        orc.reset_lottery = lambda idx, frm, v=lottery: asked.append((idx, frm)) or v
        orc.set_device_weights(0, a)
        orc.set_learning_rate(0.1)
        orc.lr_vec = [0.1, 0.1]
        orc.update(zeros_x, zeros_d)
        assert asked == [(1, 0)]                                    # one draw per transfer, none for the last device
        assert np.allclose(orc.device_weights(1)[:, :2], 0.1 * a[:, :2], atol=1e-6)   # read before the reset
        want = a.copy()
        if wins:
            want[:, :2] = 0.0                                       # reset bias 0, no reset noise
        assert np.array_equal(orc.device_weights(0), want)
    with pytest.raises(RuntimeError, match="column-transfer"):
        exact_transfer(transfer_every=1.0, with_reset_prob=0.3, transfer_columns=False)
