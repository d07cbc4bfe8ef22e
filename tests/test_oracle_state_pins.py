"""Pins of the weight-maintenance oracle against closed forms, numpy routines and brute force."""
import numpy as np

import state_oracle as so

F = np.float32


def test_decay_is_geometric_towards_the_reset_bias():
    rng = np.random.default_rng(0)
    w = rng.uniform(-0.5, 0.5, (7, 9)).astype(F)
    scale = rng.uniform(0.9, 0.99, w.shape).astype(F)
    bias = rng.normal(0, 0.05, w.shape).astype(F)
    wide = np.full(w.shape, 10.0, F)
    out = w
    for _ in range(20):
        out = so.decay_device(out, scale, bias, -wide, wide)
    assert np.allclose(out, bias + (w - bias) * scale.astype(np.float64) ** 20, atol=2e-6)
    # alpha interpolates the decay scale towards 1; alpha = 0 is the identity
    assert np.allclose(so.decay_device(w, scale, bias, -wide, wide, alpha=0.0), w, atol=1e-7)   # (w - b) + b in fp32
    half = so.decay_device(w, scale, bias, -wide, wide, alpha=0.5)
    assert np.allclose(half, bias + (w - bias) * (1 + 0.5 * (scale - 1)), atol=1e-7)
    # the bias column stays; the bounds hold afterwards
    kept = so.decay_device(w, scale, bias, -wide, wide, bias_no_decay=True)
    assert np.allclose(kept[:, -1], w[:, -1], atol=1e-7) and np.abs(kept[:, :-1] - w[:, :-1]).max() > 1e-3
    tight = np.full(w.shape, 0.1, F)
    assert np.abs(so.decay_device(w, scale, bias, -tight, tight)).max() <= 0.1
    # simple device: w * (1 - alpha / lifetime), nothing for a lifetime <= 1
    assert np.allclose(so.decay_simple(w, 50.0, 2.0), w * (1 - 2.0 / 50.0), atol=1e-7)
    assert np.array_equal(so.decay_simple(w, 1.0), w)
    assert np.array_equal(so.decay_simple(w, 50.0, bias_no_decay=True)[:, -1], w[:, -1])


def test_clip_values_against_numpy():
    rng = np.random.default_rng(1)
    w = rng.normal(0.02, 0.3, (13, 21)).astype(F)
    assert np.isclose(so.clip_value_layer_gaussian(w, 2.5), 2.5 * np.std(w.astype(np.float64), ddof=1), rtol=1e-9)
    assert so.clip_value_layer_gaussian(w, 2.5, fixed_value=0.1) == 0.1
    assert np.isclose(so.clip_value_average_channel_max(w), np.abs(w).max(axis=1).mean(), rtol=1e-6)
    assert so.clip_value_average_channel_max(w, fixed_value=0.2) == 0.2
    clipped = so.clip_with_value(w, 0.25)
    assert clipped.max() == F(0.25) and clipped.min() == F(-0.25)
    assert np.array_equal(so.clip_with_value(clipped, 0.25), clipped)            # idempotent
    assert np.array_equal(so.clip_with_value(w, -1.0), w)                        # no value, no clipping
    w_max = rng.uniform(0.1, 0.4, w.shape).astype(F)
    w_min = -rng.uniform(0.1, 0.4, w.shape).astype(F)
    both = so.clip_fixed(w, 0.3, w_min, w_max)
    assert np.array_equal(both, np.clip(np.clip(w, w_min, w_max), -0.3, 0.3).astype(F))
    assert np.array_equal(so.clip_fixed(w, -1.0, w_min, w_max), np.clip(w, w_min, w_max))
    assert np.array_equal(so.clip_fixed(w, 0.3), np.clip(w, -0.3, 0.3))


def test_reset_columns_wrap_around_and_values():
    for x_size, start, n in [(10, 2, 3), (10, 8, 5), (10, 0, 10), (10, 9, 1), (7, 3, -1), (10, 4, 0)]:
        want = np.zeros(x_size, bool)
        for t in range(n if n >= 0 else x_size):
            want[(start + t) % x_size] = True
        assert np.array_equal(so.reset_column_mask(x_size, start, n), want), (x_size, start, n)
    rng = np.random.default_rng(2)
    w = rng.uniform(-0.5, 0.5, (6, 10)).astype(F)
    bias = rng.normal(0, 0.1, w.shape).astype(F)
    normals = rng.normal(0, 1, w.shape).astype(F)
    wide = np.full(w.shape, 10.0, F)
    out = so.reset_cols(w, bias, -wide, wide, 0.01, 8, 5, normals)
    cols = [8, 9, 0, 1, 2]
    rest = [j for j in range(10) if j not in cols]
    assert np.array_equal(out[:, rest], w[:, rest])
    assert np.allclose(out[:, cols], (bias + F(0.01) * normals)[:, cols], atol=1e-7)
    lottery = rng.uniform(0, 1, w.shape).astype(F)
    part = so.reset_cols(w, bias, -wide, wide, 0.0, 0, -1, normals, lottery, 0.3)
    assert np.array_equal(part != w, (lottery < 0.3) & (bias != w))
    assert np.array_equal(part[lottery < 0.3], bias[lottery < 0.3])
    plain = so.reset_cols(w, None, None, None, 0.5, 1, 2, normals)
    assert np.allclose(plain[:, 1:3], 0.5 * normals[:, 1:3], atol=1e-7)


def test_delta_weights_bookkeeping():
    rng = np.random.default_rng(3)
    w_old = rng.normal(0, 0.3, (4, 5)).astype(F)
    w_new = (w_old + rng.normal(0, 0.01, w_old.shape)).astype(F)
    lr = 0.05
    restored, delta = so.get_and_reset_weight_update(w_new, w_old, -1.0 / lr)
    assert np.array_equal(restored, w_old)
    assert np.allclose(w_old - lr * delta, w_new, atol=1e-7)
