"""Pins the ORDER in which the device-to-device parameters are drawn at construction
(src/rpucuda/rpu_pulsed_device.cpp:593-733, src/rpucuda/rpu_linearstep_device.cpp:20-74, generator of
src/rpucuda/rng.h:45-61) without going through the oracle's or the library's own sampling code.

`tests/rawstream.cpp` prints the raw libstdc++ stream (one engine, one persistent normal distribution, one
uniform distribution) for a given pattern of draws.  The expected arrays are assembled here in numpy from
those raw numbers, following the reference's loops as read from its source: column-major walk (x outer, d
inner) with the draws [w_max, w_min, gain, up/down, corrupt-uniform (+1 uniform if corrupt), diffusion,
reset, (lifetime only if lifetime > 0)] per cross-point, then a row-major walk with [gamma_up, gamma_down].
One `*_dtod` is non-zero at a time, so each array is a function of exactly one slot of the stream: a swapped
loop, a dropped or additional draw, or a distribution object made afresh per call moves the numbers to
other cross-points and fails the comparison.  Both the oracle and the library's host code are checked."""
import os
import subprocess

import numpy as np
import pytest

from aihwkit_amd.rpu_base import devices as dv
from helpers import constant_step, make_meta
from oracle_lib import OracleTile

HERE = os.path.dirname(os.path.abspath(__file__))
X, D = 4, 5  # x_size, d_size
SEED = 4711
F = np.float32


@pytest.fixture(scope="module")
def rawstream(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("rawstream") / "rawstream")
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-o", exe, os.path.join(HERE, "rawstream.cpp")])

    def draw(pattern, threshold=0.0, seed=SEED):
        out = subprocess.check_output([exe, str(seed), pattern, "1", repr(float(threshold))], text=True)
        rows = [line.split() for line in out.splitlines()]
        tags = [r[0] for r in rows]
        vals = np.array([int(r[1], 16) for r in rows], dtype=np.uint32).view(np.float32)
        return tags, vals

    return draw


def cells_pass1(per_cell, lifetime=False):
    """Stream offsets of the first pass: cell (row i, column j) is number j*D + i, `per_cell` draws each."""
    off = np.zeros((D, X), dtype=np.int64)
    for j in range(X):
        for i in range(D):
            off[i, j] = (j * D + i) * per_cell
    return off


def hidden_of(kind, dev):
    """Hidden-parameter arrays [n, D, X] of the oracle and of the library for the same parameters."""
    meta = make_meta()
    host = meta.create_array(X, D, dev)
    orc = OracleTile(X, D, meta._config(dev))
    names = host.get_hidden_parameter_names()
    return names, orc.get_hidden(), host.get_hidden_parameters().numpy()


def quiet(cls=dv.ConstantStepResistiveDeviceParameter, **kw):
    """Device with every device-to-device spread at zero except what `kw` turns on."""
    dev = cls()
    base = dict(construction_seed=SEED, enforce_consistency=False, w_max=0.6, w_min=-0.6, w_max_dtod=0.0, w_min_dtod=0.0,
                dw_min=0.001, dw_min_dtod=0.0, dw_min_std=0.0, up_down=0.0, up_down_dtod=0.0, diffusion=0.0,
                diffusion_dtod=0.0, reset=0.0, reset_dtod=0.0, lifetime=0.0, lifetime_dtod=0.0)
    base.update(kw)
    for k, v in base.items():
        setattr(dev, k, v)
    return dev


def both(names, orc, lib, name, expected):
    k = names.index(name)
    assert np.array_equal(orc[k], expected), ("oracle", name, orc[k], expected)
    assert np.array_equal(lib[k], expected), ("library", name, lib[k], expected)


@pytest.mark.parametrize("lifetime", [0.0, 50.0])
def test_each_bound_and_scale_comes_from_its_own_slot_of_the_column_major_walk(rawstream, lifetime):
    per_cell = 8 if lifetime > 0 else 7
    pattern = ("NNNNUNN" + ("N" if lifetime > 0 else "")) * (X * D) + "NN" * (X * D)
    tags, g = rawstream(pattern)
    off = cells_pass1(per_cell)
    one = F(1.0)

    # slot 0: upper bound
    names, orc, lib = hidden_of("c", quiet(w_max_dtod=0.3, lifetime=lifetime))
    both(names, orc, lib, "max_bound", F(0.6) * (one + F(0.3) * g[off + 0]))
    both(names, orc, lib, "min_bound", np.full((D, X), F(-0.6)))
    # slot 1: lower bound
    names, orc, lib = hidden_of("c", quiet(w_min_dtod=0.3, lifetime=lifetime))
    both(names, orc, lib, "min_bound", F(-0.6) * (one + F(0.3) * g[off + 1]))
    both(names, orc, lib, "max_bound", np.full((D, X), F(0.6)))
    # slot 2: step gain (both directions share it)
    names, orc, lib = hidden_of("c", quiet(dw_min_dtod=0.3, lifetime=lifetime))
    gain = one + F(0.3) * g[off + 2]
    both(names, orc, lib, "dwmin_up", (F(0.0) + gain + F(0.0)) * F(0.001))
    both(names, orc, lib, "dwmin_down", (F(0.0) + gain - F(0.0)) * F(0.001))
    # slot 2, log-normal form
    names, orc, lib = hidden_of("c", quiet(dw_min_dtod=0.3, dw_min_dtod_log_normal=True, lifetime=lifetime))
    k = names.index("dwmin_up")
    expect = np.exp(F(0.3) * g[off + 2]).astype(F) * F(0.001)
    assert np.allclose(orc[k], expect, rtol=2e-7, atol=0) and np.allclose(lib[k], expect, rtol=2e-7, atol=0)
    # slot 3: up/down asymmetry enters the two directions with opposite signs
    names, orc, lib = hidden_of("c", quiet(up_down_dtod=0.1, lifetime=lifetime))
    r = F(0.1) * g[off + 3]
    both(names, orc, lib, "dwmin_up", (F(0.0) + one + r) * F(0.001))
    both(names, orc, lib, "dwmin_down", (F(0.0) + one - r) * F(0.001))
    # slot 4 is the uniform of the corrupt-device test (next test); slot 5: diffusion, slot 6: reset
    assert tags[4] == "U"
    names, orc, lib = hidden_of("c", quiet(diffusion=0.1, diffusion_dtod=0.4, lifetime=lifetime))
    both(names, orc, lib, "diffusion_rates", np.abs(F(0.1) * (one + F(0.4) * g[off + 5])))
    names, orc, lib = hidden_of("c", quiet(reset=0.05, reset_dtod=0.2, lifetime=lifetime))
    both(names, orc, lib, "reset_bias", F(0.05) + F(0.2) * g[off + 6])
    if lifetime > 0:
        # slot 7 exists only with a lifetime
        names, orc, lib = hidden_of("c", quiet(lifetime=lifetime, lifetime_dtod=0.2))
        t = F(lifetime) * (one + F(0.2) * g[off + 7])
        both(names, orc, lib, "decay_scales", np.where(t > 1, one - one / t, F(0.0)).astype(F))
    else:
        names, orc, lib = hidden_of("c", quiet(lifetime_dtod=0.2))
        both(names, orc, lib, "decay_scales", np.ones((D, X), F))


def test_all_spreads_together_are_the_same_slots(rawstream):
    """Every spread on at once (the configuration of the benchmark): no slot moves when the others are in use."""
    _, g = rawstream("NNNNUNN" * (X * D))
    off = cells_pass1(7)
    one = F(1.0)
    dev = quiet(w_max_dtod=0.3, w_min_dtod=0.3, dw_min_dtod=0.3, up_down_dtod=0.01, enforce_consistency=True)
    names, orc, lib = hidden_of("c", dev)
    hi = F(0.6) * (one + F(0.3) * g[off + 0])
    lo = F(-0.6) * (one + F(0.3) * g[off + 1])
    swap = lo > hi
    hi, lo = np.where(swap, lo, hi), np.where(swap, hi, lo)
    both(names, orc, lib, "max_bound", np.abs(hi))
    both(names, orc, lib, "min_bound", -np.abs(lo))
    gain = one + F(0.3) * g[off + 2]
    r = F(0.01) * g[off + 3]
    both(names, orc, lib, "dwmin_up", np.abs((F(0.0) + gain + r) * F(0.001)))
    both(names, orc, lib, "dwmin_down", np.abs((F(0.0) + gain - r) * F(0.001)))


def test_corrupt_devices_take_a_second_uniform_only_when_corrupt(rawstream):
    prob = 0.5
    tags, g = rawstream("NNNNCNN" * (X * D), threshold=prob)
    assert 3 <= tags.count("V") <= X * D - 3  # both branches occur with this seed
    dev = quiet(w_max_dtod=0.3, corrupt_devices_prob=prob, corrupt_devices_range=0.25, reset=0.05, reset_dtod=0.2)
    names, orc, lib = hidden_of("c", dev)
    hi_e, lo_e, up_e, reset_e = (np.zeros((D, X), F) for _ in range(4))
    pos = 0
    for j in range(X):
        for i in range(D):
            hi = F(0.6) * (F(1.0) + F(0.3) * g[pos])
            lo = F(-0.6)
            up = F(0.001)
            assert tags[pos + 4] == "C"
            pos_after = pos + 5
            if g[pos + 4] < F(prob):
                assert tags[pos + 5] == "V"
                a = max(min(hi, lo), F(-0.25))
                b = min(max(hi, lo), F(0.25))
                hi = lo = F(a + (b - a) * g[pos + 5])
                up = F(0.0)
                pos_after += 1
            hi_e[i, j], lo_e[i, j], up_e[i, j] = hi, lo, up
            reset_e[i, j] = F(0.05) + F(0.2) * g[pos_after + 1]  # diffusion draw, then reset draw
            pos = pos_after + 2
    assert pos == len(g)
    both(names, orc, lib, "max_bound", hi_e)
    both(names, orc, lib, "min_bound", lo_e)
    both(names, orc, lib, "dwmin_up", up_e)
    both(names, orc, lib, "reset_bias", reset_e)


@pytest.mark.parametrize("lifetime", [0.0, 50.0])
def test_linear_step_slopes_are_drawn_row_major_after_the_first_pass(rawstream, lifetime):
    per_cell = 8 if lifetime > 0 else 7
    n1 = per_cell * X * D
    _, g = rawstream(("NNNNUNN" + ("N" if lifetime > 0 else "")) * (X * D) + "NN" * (X * D))
    off2 = n1 + 2 * np.arange(D * X).reshape(D, X)  # row-major: cell (i, j) is number i*X + j
    # mean-bound reference: slope = -(gamma + dtod xi) * scale / w_max with constant scale and bound
    for which, slot, bound in (("up", 0, F(0.6)), ("down", 1, F(-0.6))):
        kw = dict(gamma_up=0.3, gamma_down=0.2, gamma_up_dtod=0.0, gamma_down_dtod=0.0, mean_bound_reference=True,
                  allow_increasing=True, lifetime=lifetime)
        kw["gamma_%s_dtod" % which] = 0.4
        dev = quiet(dv.LinearStepResistiveDeviceParameter, **kw)
        names, orc, lib = hidden_of("l", dev)
        gamma = F(0.3 if which == "up" else 0.2)
        expect = -(gamma + F(0.4) * g[off2 + slot]) * F(0.001) / bound
        both(names, orc, lib, "slope_%s" % which, expect.astype(F))
        other = "down" if which == "up" else "up"
        k = names.index("slope_%s" % other)
        assert np.unique(orc[k]).size == 1 and np.array_equal(orc[k], lib[k])
    # without allow_increasing the drawn decrease is folded to positive before use
    dev = quiet(dv.LinearStepResistiveDeviceParameter, gamma_up=0.0, gamma_up_dtod=1.0, gamma_down=0.2, gamma_down_dtod=0.0,
                mean_bound_reference=True, allow_increasing=False, lifetime=lifetime)
    names, orc, lib = hidden_of("l", dev)
    both(names, orc, lib, "slope_up", (-np.abs(F(0.0) + F(1.0) * g[off2]) * F(0.001) / F(0.6)).astype(F))


def test_soft_bounds_draws_the_two_slope_normals_although_they_are_unused(rawstream):
    """A second device sampled from the same generator (a transfer chain) starts after ALL draws of the
    first one: 7 per cross-point plus the two slope normals of a SoftBounds device."""
    from helpers import soft_bounds, transfer_param

    _, g = rawstream("NNNNUNN" * (X * D) + "NN" * (X * D) + "NNNNUNN" * (X * D))
    first = quiet(dv.SoftBoundsResistiveDeviceParameter, construction_seed=0)
    second = quiet(dv.SoftBoundsResistiveDeviceParameter, construction_seed=0, w_max_dtod=0.3)
    tr = transfer_param([first, second], construction_seed=SEED, gamma=0.0)
    host = make_meta().create_array(X, D, tr)
    names = host.get_hidden_parameter_names()
    hidden = host.get_hidden_parameters().numpy()
    k = names.index("max_bound_1")
    off = 9 * X * D + cells_pass1(7)
    assert np.array_equal(hidden[k], F(0.6) * (F(1.0) + F(0.3) * g[off]))


def test_the_normal_distribution_object_is_persistent(rawstream):
    """libstdc++'s normal_distribution makes two values per round and keeps the second: with an odd number of
    normals per cross-point (7 draws = 6 normals + 1 uniform is even; with a lifetime it is 7) a fresh object
    per call or per cross-point would give another stream.  The helper's stream itself shows the cache: the
    uniform drawn between two normals does not disturb the pair."""
    _, a = rawstream("NN")
    _, b = rawstream("NUN")
    assert a[0] == b[0] and a[1] == b[2]
