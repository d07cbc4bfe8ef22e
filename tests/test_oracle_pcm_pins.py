"""Pins of the PCM noise oracle (oracle/pcm_oracle.py) by closed forms; CPU only."""
import numpy as np
import pytest
from scipy.stats import norm

from pcm_oracle import PcmOracle


def test_conductance_pair_round_trip_and_mapping():
    orc = PcmOracle(prog_noise_scale=0.0, g_min=0.0)
    w = np.array([[0.5, -0.25, 0.0, -0.5]], np.float32)
    (gp, gm), ratio = orc.to_conductances(w)
    assert ratio == pytest.approx(50.0)                      # max |w| -> g_max = 25 uS
    assert np.allclose(gp, [[25.0, 0.0, 0.0, 0.0]]) and np.allclose(gm, [[0.0, 12.5, 0.0, 25.0]])
    prog, nu = orc.apply_programming_noise(w)
    assert np.allclose(prog, w, atol=1e-7) and len(nu) == 2 and nu[0].shape == w.shape
    (gp, gm), _ = PcmOracle(g_min=2.0).to_conductances(w)   # zero weight sits at g_min on both devices
    assert gp[0, 2] == 2.0 and gm[0, 2] == 2.0 and gp[0, 0] == 25.0


def test_programming_noise_sigma_polynomial_and_clamp():
    orc = PcmOracle(seed=1)
    n = 200000
    for g, sigma in [(25.0, 0.26348 + 1.9650 - 1.1731), (12.5, 0.26348 + 1.9650 * 0.5 - 1.1731 * 0.25)]:
        noisy = orc.program_conductance(np.full(n, g, np.float32))
        assert noisy.mean() == pytest.approx(g, abs=4 * sigma / np.sqrt(n))
        assert noisy.std() == pytest.approx(sigma, rel=0.01)
    at_zero = orc.program_conductance(np.zeros(n, np.float32))
    assert at_zero.min() == 0.0                                        # no negative conductances
    assert at_zero.mean() == pytest.approx(0.26348 / np.sqrt(2 * np.pi), rel=0.02)  # half-normal mean
    half = PcmOracle(g_max=12.5, seed=2).program_conductance(np.full(n, 12.5, np.float32))
    assert half.std() == pytest.approx(0.5 * (0.26348 + 1.9650 - 1.1731), rel=0.01)  # coefficients refer to 25 uS


def test_drift_coefficient_distribution_limits():
    orc = PcmOracle(seed=3)
    n = 200000
    top = orc.drift_coefficients(np.full(n, 25.0, np.float32))        # ln(1) = 0: mu, sigma at their lower clips
    assert top.mean() == pytest.approx(0.049, rel=0.01) and top.std() == pytest.approx(0.008, rel=0.02)
    low = orc.drift_coefficients(np.full(n, 0.025, np.float32))       # ln(1e-3): both at their upper clips
    assert low.mean() == pytest.approx(0.1, rel=0.02) and low.std() == pytest.approx(0.045, rel=0.03)
    mid = orc.drift_coefficients(np.full(n, 2.5, np.float32))
    assert mid.mean() == pytest.approx(-0.0155 * np.log(0.1) + 0.0244, rel=0.01)
    assert PcmOracle(seed=3, drift_scale=2.0).drift_coefficients(np.full(10, 25.0, np.float32)).mean() > 0.08


def test_drift_power_law_and_read_noise():
    orc = PcmOracle(read_noise_scale=0.0)
    g = np.array([25.0, 10.0, 1.0], np.float32)
    nu = np.array([0.05, 0.06, 0.1], np.float32)
    t = 86400.0
    assert np.allclose(orc.drift_conductance(g, nu, t), g * ((t + 20.0) / 20.0) ** (-nu), rtol=1e-5)
    assert np.array_equal(orc.drift_conductance(g, nu, 0.0), g)       # t = t_0: no drift yet
    noisy = PcmOracle(seed=4).drift_conductance(np.full(200000, 25.0, np.float32), np.zeros(200000, np.float32), t)
    sigma = 0.0088 * np.sqrt(np.log((t + 20.0 + 250e-9) / (2 * 250e-9)))
    assert noisy.std() == pytest.approx(25.0 * sigma, rel=0.02) and noisy.mean() == pytest.approx(25.0, rel=1e-3)
    small = PcmOracle(seed=5).drift_conductance(np.full(200000, 0.001, np.float32), np.zeros(200000, np.float32), t)
    # q_s saturates at 0.2: relative noise s = 0.2 * sqrt(ln(..)) ~ 1.02, and max(1 + s xi, 0) is a clamped normal
    s_rel = 0.2 * sigma / 0.0088
    cdf, pdf = norm.cdf(1 / s_rel), norm.pdf(1 / s_rel)
    mean = cdf + s_rel * pdf
    second = (1 + s_rel ** 2) * cdf + s_rel * pdf
    assert small.mean() / 0.001 == pytest.approx(mean, rel=0.01)
    assert small.std() / 0.001 == pytest.approx(np.sqrt(second - mean ** 2), rel=0.02)


def test_weights_shrink_with_time_and_sign_is_kept():
    orc = PcmOracle(seed=6)
    w = np.random.default_rng(0).uniform(-1, 1, (64, 64)).astype(np.float32)
    prog, nu = orc.apply_programming_noise(w)
    day = orc.apply_drift_noise(prog, nu, 86400.0)
    year = orc.apply_drift_noise(prog, nu, 86400.0 * 365)
    assert np.abs(prog).mean() > np.abs(day).mean() > np.abs(year).mean()
    strong = np.abs(w) > 0.5
    assert np.all(np.sign(day[strong]) == np.sign(w[strong]))
    assert np.abs(day).mean() / np.abs(prog).mean() == pytest.approx((86420.0 / 20.0) ** -0.06, rel=0.1)
