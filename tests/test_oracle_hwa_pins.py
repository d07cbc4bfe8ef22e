"""Pins of oracle/hwa_oracle.py (weight remapping, weight modifier, device drift, pulse counters): the golden vectors
of the reference's own tests for these calls, closed forms and brute force on tiny inputs."""
import math

import numpy as np

from oracle import hwa_oracle as ho

F = np.float32


def test_remap_golden_vectors_of_the_reference_tests():
    # tests/test_inference_tiles.py:215-243 (layerwise, analog bias in the last column): weights / 0.6, scales 0.6
    w = np.array([[0.1, 0.2, 0.3, -0.1], [0.4, 0.5, 0.6, -0.3]], dtype=F)
    out, scales = ho.remap(w, np.ones(2, dtype=F), ho.REMAP_LAYERWISE_SYMMETRIC)
    np.testing.assert_allclose(out, w / F(0.6), rtol=1e-6)
    np.testing.assert_allclose(scales, [0.6, 0.6], rtol=1e-6)
    # tests/test_inference_tiles.py:245-275 (channelwise): scales [0.7, 0.6]
    w = np.array([[-0.7, 0.2, 0.3, -0.1], [0.4, 0.5, 0.6, -0.3]], dtype=F)
    out, scales = ho.remap(w, np.ones(2, dtype=F), ho.REMAP_CHANNELWISE_SYMMETRIC)
    np.testing.assert_allclose(scales, [0.7, 0.6], rtol=1e-6)
    np.testing.assert_allclose(out, w / np.array([[0.7], [0.6]], dtype=F), rtol=1e-6)


def test_remap_invariants():
    rng = np.random.default_rng(0)
    w = (rng.standard_normal((9, 14)) * 0.4).astype(F)
    w[3] = 0.0                                                   # an empty row keeps its scale
    s0 = rng.uniform(0.5, 2.0, 9).astype(F)
    for kind, kw in ((ho.REMAP_LAYERWISE_SYMMETRIC, dict(remapped_wmax=0.8)),
                     (ho.REMAP_CHANNELWISE_SYMMETRIC, dict(remapped_wmax=0.8)),
                     (ho.REMAP_CHANNELWISE_SYMMETRIC, dict(max_scale_range=1.5)),
                     (ho.REMAP_CHANNELWISE_SYMMETRIC, dict(max_scale_range=1.5, max_scale_ref=1.0)),
                     (ho.REMAP_CHANNELWISE_NORM, dict(row_norm=0.9, clip_if=False))):
        out, s = ho.remap(w, s0, kind, **kw)
        # the product of scale and row is what it was
        np.testing.assert_allclose(out * s[:, None], w * s0[:, None], rtol=2e-6, atol=1e-7)
        assert not out[3].any()
        if kind == ho.REMAP_CHANNELWISE_SYMMETRIC and "max_scale_range" not in kw:
            assert s[3] == s0[3]
        if kind == ho.REMAP_LAYERWISE_SYMMETRIC:
            assert abs(np.abs(out).max() - 0.8) < 1e-6
            np.testing.assert_allclose(s / s0, np.abs(w).max() / 0.8, rtol=1e-6)
        elif "max_scale_range" in kw:
            floor = max(s0.min(), kw.get("max_scale_ref", 0.0))
            assert s.max() <= floor * 1.5 * (1 + 1e-6)
            free = (np.abs(w).max(axis=1) * s0 < floor * 1.5) & (np.abs(w).max(axis=1) > 0)
            np.testing.assert_allclose(np.abs(out[free]).max(axis=1), 1.0, rtol=1e-6)   # unbounded rows map to 1
            assert (~free).sum() >= 2                                                   # and some rows are bounded
        elif kind == ho.REMAP_CHANNELWISE_SYMMETRIC:
            np.testing.assert_allclose(np.abs(np.delete(out, 3, 0)).max(axis=1), 0.8, rtol=1e-6)
        else:
            norms = np.linalg.norm(out.astype(np.float64), axis=1)
            assert norms.max() <= 0.9 * (1 + 1e-6)
            small = np.linalg.norm(w.astype(np.float64), axis=1) <= 0.9
            np.testing.assert_array_equal(out[small], w[small])                         # short rows are left alone
    # clip_if: rows are scaled down but the scales do not take the factor up
    out, s = ho.remap(w, s0, ho.REMAP_CHANNELWISE_NORM, row_norm=0.9, clip_if=True)
    np.testing.assert_array_equal(s, s0)
    assert np.linalg.norm(out.astype(np.float64), axis=1).max() <= 0.9 * (1 + 1e-6)
    out, s = ho.remap(w, s0, ho.REMAP_NONE)
    np.testing.assert_array_equal(out, w)


def test_modifier_known_answers():
    w = np.array([[0.5, -0.5, 0.24, 1.0], [0.26, -0.74, 0.0, -2.0]], dtype=F)
    # round half away from zero (roundf), not half to even: 0.5 / 1.0 -> 1, -0.5 -> -1
    out = ho.modify(w, ho.MOD_DISCRETIZE, res=0.5, rel_to_actual_wmax=False, assumed_wmax=2.0)
    np.testing.assert_array_equal(out, np.array([[1.0, -1.0, 0.0, 1.0], [0.0, -1.0, 0.0, -2.0]], dtype=F))
    # relative to the largest absolute weight (2): the same grid
    np.testing.assert_array_equal(ho.modify(w, ho.MOD_DISCRETIZE, res=0.5), out)
    # copy_last_column: amax comes from the other columns (0.74) and the last column is kept
    out = ho.modify(w, ho.MOD_DISCRETIZE, res=0.5, copy_last_column=True)
    np.testing.assert_allclose(out, np.array([[0.37, -0.37, 0.37, 1.0], [0.37, -0.74, 0.0, -2.0]], dtype=F), rtol=1e-6)
    # stochastic rounding: u = 0 rounds v / res - 0.5, u -> 1 rounds v / res + 0.5
    v = np.array([[0.3]], dtype=F)
    lo = ho.modify(v, ho.MOD_DISCRETIZE, res=1.0, sto_round=True, uniforms=np.array([[0.1]], dtype=F),
                   rel_to_actual_wmax=False)
    hi = ho.modify(v, ho.MOD_DISCRETIZE, res=1.0, sto_round=True, uniforms=np.array([[0.9]], dtype=F),
                   rel_to_actual_wmax=False)
    assert lo[0, 0] == 0.0 and hi[0, 0] == 1.0                   # P(up) = 0.3: u > 0.7 goes up
    # DoReFa: round(tanh(w) * clip / tanh(amax) / res) * res
    out = ho.modify(w, ho.MOD_DOREFA, res=0.1, dorefa_clip=0.6)
    scale = 0.6 / math.tanh(2.0)
    want = [[math.floor(abs(math.tanh(x)) * scale / 0.1 + 0.5) * 0.1 * (1 if x >= 0 else -1) for x in row] for row in w]
    np.testing.assert_allclose(out, np.array(want, dtype=F), atol=1e-6)
    assert abs(out).max() <= 0.6 + 1e-6
    z = np.array([[1.0, -2.0, 0.5, 0.0], [3.0, 1.0, -1.0, 2.0]], dtype=F)
    kw = dict(normals=z, std_dev=0.1, rel_to_actual_wmax=False, assumed_wmax=2.0)
    np.testing.assert_allclose(ho.modify(w, ho.MOD_ADD_NORMAL, **kw), w + 0.2 * z, rtol=1e-6)
    np.testing.assert_allclose(ho.modify(w, ho.MOD_MULT_NORMAL, **kw), w * (1 + 0.2 * z), rtol=1e-6)
    # Poly: sigma = std (c0 + c1 |w| / amax + c2 (|w| / amax)^2), noise amax sigma z
    sig = 0.1 * (1.0 + 3.0 * np.abs(w) / 2.0 + 0.5 * (np.abs(w) / 2.0) ** 2)
    np.testing.assert_allclose(ho.modify(w, ho.MOD_POLY, coeffs=(1.0, 3.0, 0.5), **kw), w + 2.0 * sig * z, rtol=1e-6)
    # ProgNoise: std / g_max, and the sign of a weight survives (zero counts as positive)
    out = ho.modify(w, ho.MOD_PROG_NOISE, coeffs=(1.0, 3.0, 0.5), g_max=0.05, **kw)
    noisy = w + 2.0 * (sig / 0.05) * z
    np.testing.assert_allclose(out, np.where(w < 0, -np.abs(noisy), np.abs(noisy)), rtol=1e-5)
    assert (np.sign(out) == np.sign(noisy)).mean() < 1.0         # the example does flip some
    assert ((out < 0) == (w < 0)).all()
    # discretize, then noise that is not discretized
    out = ho.modify(w, ho.MOD_DISCRETIZE_ADD_NORMAL, res=0.5, **kw)
    np.testing.assert_allclose(out, np.array([[1.0, -1.0, 0.0, 1.0], [0.0, -1.0, 0.0, -2.0]]) + 0.2 * z, rtol=1e-6)
    # dropped connections and the copy
    drop = np.array([[0.1, 0.9, 0.49, 0.5], [0.0, 0.7, 0.2, 0.3]], dtype=F)
    out = ho.modify(w, ho.MOD_DROP_CONNECT, pdrop=0.5, drop_uniforms=drop)
    np.testing.assert_array_equal(out, np.where(drop < 0.5, 0, w))
    np.testing.assert_array_equal(ho.modify(w, ho.MOD_COPY), w)
    out = ho.modify(w, ho.MOD_ADD_NORMAL, pdrop=0.5, drop_uniforms=drop, copy_last_column=True, **kw)
    np.testing.assert_array_equal(out[:, -1], w[:, -1])          # the last column is neither noisy nor dropped


def test_drift_golden_vector_and_clock():
    rng = np.random.default_rng(1)
    w = (rng.standard_normal((6, 5)) * 0.3).astype(F)
    # tests/test_bindings_tiles.py:118-131: nu = 0.1, t_0 = 1, one call with delta_t = 2 -> w 2^(-0.1)
    d = ho.Drifter(0.1)
    out = d.apply(w, 2.0)
    np.testing.assert_allclose(out, w * 2.0 ** (-0.1), rtol=1e-6)
    # the clock runs on: after 2 + 3 the weights are w0 5^(-nu), not the product of the two steps
    out2 = d.apply(out, 3.0)
    np.testing.assert_allclose(out2, w * 5.0 ** (-0.1), rtol=1e-6)
    # a weight that was changed from outside restarts from its new value at the current time
    moved = out2.copy()
    moved[0, 0] += 0.05
    out3 = d.apply(moved, 4.0)
    assert out3[0, 0] == moved[0, 0]
    np.testing.assert_allclose(out3.ravel()[1:], (w * 9.0 ** (-0.1)).ravel()[1:], rtol=1e-6)
    out4 = d.apply(out3, 5.0)                                    # 5 time units after its restart
    np.testing.assert_allclose(out4[0, 0], moved[0, 0] * 5.0 ** (-0.1), rtol=1e-6)
    # less than t_0 since the (re)start: no drift yet; t_0 scales the time
    d = ho.Drifter(0.1, t0=10.0)
    np.testing.assert_array_equal(d.apply(w, 5.0), w)
    np.testing.assert_allclose(d.apply(w, 35.0), w * 4.0 ** (-0.1), rtol=1e-6)
    # per-weight nu, conductance offset: w -> w0 s + a (s - 1) with a = g_offset wg_ratio + w_offset
    nu = rng.uniform(0.01, 0.2, w.shape).astype(F)
    d = ho.Drifter(nu, wg_ratio=0.5, g_offset=0.2, w_offset=-0.3)
    s = 3.0 ** (-nu.astype(np.float64))
    np.testing.assert_allclose(d.apply(w, 3.0), w * s + (0.2 * 0.5 - 0.3) * (s - 1), rtol=1e-5, atol=1e-7)
    # nu depends on the conductance: nu - k log((w - w_offset) / wg_ratio + g_offset) + k log G0
    wp = np.abs(w) + F(0.1)
    d = ho.Drifter(0.05, nu_k=0.02, log_g0=math.log(0.5))
    nu_w = 0.05 - 0.02 * np.log(wp.astype(np.float64)) + 0.02 * math.log(0.5)
    np.testing.assert_allclose(d.apply(wp, 7.0), wp * 7.0 ** (-nu_w), rtol=1e-5)
    # variation of nu and read noise enter linearly; the bounds saturate both the weight and its memory
    z = rng.standard_normal(w.shape).astype(F)
    d = ho.Drifter(0.1, nu_std=0.3, w_read_std=0.01)
    out = d.apply(w, 2.0, nu_normals=z, read_normals=-z, w_min=-0.2 * np.ones_like(w), w_max=0.2 * np.ones_like(w))
    want = np.clip(w * 2.0 ** (-(0.1 + 0.03 * z.astype(np.float64))) - 0.01 * z, -0.2, 0.2)
    np.testing.assert_allclose(out, want, rtol=1e-5, atol=1e-7)
    np.testing.assert_array_equal(d.prev, out)
    # a device whose sampled bounds cross (min above max): the saturation applies the lower bound first, the upper wins
    d = ho.Drifter(0.1)
    out = d.apply(np.array([[0.3, 0.3]], dtype=F), 2.0, w_min=np.array([[0.5, -1.0]], dtype=F),
                  w_max=np.array([[0.1, 1.0]], dtype=F))
    np.testing.assert_allclose(out, [[0.1, 0.3 * 2.0 ** (-0.1)]], rtol=1e-6)


def test_pulse_counts_against_brute_force():
    rng = np.random.default_rng(2)
    x_words = rng.integers(0, 2 ** 32, (5, 4), dtype=np.uint64).astype(np.uint32)
    d_words = rng.integers(0, 2 ** 32, (5, 3), dtype=np.uint64).astype(np.uint32)
    got = ho.pulse_counts(x_words, d_words)
    want = np.zeros((2, 3, 4), dtype=np.int64)
    for b in range(5):
        for i in range(3):
            for j in range(4):
                n = sum(1 for k in range(1, 32) if (int(x_words[b, j]) >> k) & (int(d_words[b, i]) >> k) & 1)
                differ = (int(x_words[b, j]) ^ int(d_words[b, i])) & 1
                want[differ, i, j] += n
    np.testing.assert_array_equal(got, want)
    assert got[0].sum() > 0 and got[1].sum() > 0
