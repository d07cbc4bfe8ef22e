"""CPU-side checks: the C ABI library loads and exports every declared symbol, the host tile classes
behave like the reference bindings (shapes, errors, parameter plumbing), and the device arrays the
library samples equal the oracle's for the same construction seed.  No GPU compute here."""
import copy
import os
import re
import subprocess
import sys

import numpy as np
import pytest
import torch

from aihwkit_amd import _cabi
from aihwkit_amd.rpu_base import cuda, devices as dv, tiles
from helpers import config2, constant_step, io_params, make_meta, soft_bounds
from oracle_lib import OracleTile

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "rpu_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rpu_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = declared_functions()
    assert len(names) >= 25
    lib = _cabi.lib()
    for name in names:
        assert hasattr(lib, name), name
    # and the ctypes table covers exactly the header
    assert sorted(_cabi.SYMBOLS) == names
    assert lib.rpu_abi_version() == 1
    assert cuda.is_compiled()


def test_struct_sizes_match_the_header_layout():
    # plain 4-byte fields only: a mismatch in field count shows up as a size difference
    text = open(os.path.join(ROOT, "include", "rpu_amd.h")).read()
    for struct, cls in (("rpu_io_params", _cabi.IOParams), ("rpu_update_params", _cabi.UpdateParams),
                        ("rpu_device_params", _cabi.DeviceParams)):
        body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (struct, struct), text, flags=re.S).group(1)
        body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
        fields = re.findall(r"\b(?:int32_t|uint32_t|float)\s+([a-z0-9_]+)\s*;", body)
        assert fields == [f[0] for f in cls._fields_], struct


def test_defaults_from_the_library_equal_the_python_mirror():
    cfg = _cabi.TileConfig()
    _cabi.check(_cabi.lib().rpu_tile_config_default(cfg, 3))
    meta = dv.AnalogTileParameter()
    mine = meta._config(dv.SoftBoundsResistiveDeviceParameter())
    for part in ("f_io", "b_io", "up", "device"):
        a, b = getattr(cfg, part), getattr(mine, part)
        for name, _ in a._fields_:
            assert getattr(a, name) == pytest.approx(getattr(b, name)), (part, name)


@pytest.mark.parametrize("kind", ["constant", "soft", "linear"])
@pytest.mark.parametrize("consistent", [True, False])
def test_sampled_device_arrays_equal_the_oracle(kind, consistent):
    kw = dict(construction_seed=321, enforce_consistency=consistent, lifetime=100.0, lifetime_dtod=0.1,
              diffusion=0.01, diffusion_dtod=0.2, reset_dtod=0.1, up_down=0.02)
    if kind == "constant":
        dev = constant_step(**kw)
    elif kind == "soft":
        dev = soft_bounds(**kw)
    else:
        dev = dv.LinearStepResistiveDeviceParameter()
        for k, v in dict(kw, gamma_up=0.3, gamma_down=0.1, mean_bound_reference=True).items():
            setattr(dev, k, v)
    meta = make_meta()
    host = meta.create_array(37, 23, dev)
    orc = OracleTile(37, 23, meta._config(dev))
    assert host.get_hidden_parameter_names()[:4] == ["max_bound", "min_bound", "dwmin_up", "dwmin_down"]
    assert np.array_equal(host.get_hidden_parameters().numpy(), orc.get_hidden())


def test_host_tile_state_surface():
    meta, dev = config2()
    tile = meta.create_array(20, 10, dev)
    assert (tile.get_x_size(), tile.get_d_size()) == (20, 10)
    assert tile.get_learning_rate() == 0.0  # RPUAbstract default
    tile.set_learning_rate(0.05)
    assert tile.get_learning_rate() == pytest.approx(0.05)
    w = torch.full((10, 20), 5.0)
    tile.set_weights(w)
    hidden = tile.get_hidden_parameters()
    assert torch.equal(tile.get_weights(), hidden[0])  # clipped into the per-device upper bounds
    with pytest.raises(RuntimeError, match="Invalid weights dimensions"):
        tile.set_weights(torch.zeros(20, 10))
    # new bounds clip the stored weights at once
    before = tile.get_weights()
    hidden[0].fill_(0.1)
    tile.set_hidden_parameters(hidden)
    assert torch.equal(tile.get_weights(), torch.minimum(before, torch.tensor(0.1)))
    clone = copy.deepcopy(tile)
    clone.set_weights(torch.zeros(10, 20))
    assert torch.equal(tile.get_weights(), torch.minimum(before, torch.tensor(0.1)))
    assert clone.get_learning_rate() == pytest.approx(0.05)
    with pytest.raises(RuntimeError, match="do not compute"):
        tile.forward(torch.zeros(1, 20))


def test_unsupported_parameters_fail_loudly():
    dev = soft_bounds()
    with pytest.raises(RuntimeError, match="expects bound==1"):
        make_meta(io_params(inp_bound=2.0)).create_array(4, 4, dev)
    with pytest.raises(RuntimeError, match="not implemented"):
        make_meta(io_params(mv_type=4)).create_array(4, 4, dev)                   # SplitMode
    # per-line periphery values are drawn at creation and are part of the extra state of a host tile too
    host = make_meta(io_params(out_noise_std=0.1, v_offset_std=0.1, r_series=0.01, out_nonlinearity=0.3)).create_array(4, 6, dev)
    names = [k for k in host.dump_extra() if k.startswith("rpu.fwd.")]
    assert len(names) == 3 * 6 and "rpu.fwd.v_offset_5.bits" in names and "rpu.fwd.out_noise_values_0.bits" in names
    assert not any(k.startswith("rpu.bwd.") for k in host.dump_extra())
    make_meta(io_params(ir_drop=1.0, w_noise_type=dv.WeightNoiseType.PCMRead, w_noise=0.1)).create_array(4, 4, dev)
    with pytest.raises(RuntimeError, match="desired_bl"):
        make_meta(desired_bl=1000).create_array(4, 4, dev)
    with pytest.raises(RuntimeError, match="not supported"):
        make_meta(pulse_type=17).create_array(4, 4, dev)
    make_meta(pulse_type=dv.PulseType.Stochastic).create_array(4, 4, dev)
    make_meta(pulse_type=dv.PulseType.MeanCount).create_array(4, 4, dev)
    make_meta(pulse_type=dv.PulseType.NoneWithDevice).create_array(4, 4, dev)
    bad = soft_bounds()
    bad.gamma_up = 0.5
    with pytest.raises(RuntimeError, match="SoftBounds set to wrong values"):
        make_meta().create_array(4, 4, bad)
    with pytest.raises(RuntimeError, match="needs to contain 0"):
        make_meta().create_array(4, 4, constant_step(w_min=0.1))
    with pytest.raises(AttributeError):
        dev.no_such_field = 1
    make_meta().create_array(4, 4, soft_bounds(write_noise_std=0.1))    # LinearStep / SoftBounds implement write noise
    cfg = make_meta()._config(constant_step())                          # ConstantStep does not (through the C ABI)
    cfg.device.write_noise_std = 0.1
    import ctypes
    handle = ctypes.c_void_p()
    assert _cabi.lib().rpu_tile_create(ctypes.byref(handle), 4, 4, ctypes.byref(cfg)) != 0
    assert b"write noise" in _cabi.lib().rpu_last_error()


def test_enums_have_the_reference_values():
    assert int(dv.PulseType.StochasticCompressed) == 1 and int(dv.PulseType.DeterministicImplicit) == 5
    assert int(getattr(dv.PulseType, "None")) == 0
    assert int(dv.NoiseManagementType.AbsMax) == 1 and int(dv.NoiseManagementType.Constant) == 4
    assert int(dv.BoundManagementType.Iterative) == 1 and int(dv.AnalogMVType.OnePass) == 1


def test_gpu_tile_needs_a_gpu():
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    meta, dev = config2()
    with pytest.raises(RuntimeError, match="No GPU"):
        tiles.CudaAnalogTile(meta.create_array(8, 8, dev))
    # the C ABI itself refuses compute on a tile that is not resident
    tile = meta.create_array(8, 8, dev)
    rc = _cabi.lib().rpu_tile_forward(tile._h, 1, 1, 1, 0, 0, 0, 0, None)
    assert rc != 0 and b"not resident" in _cabi.lib().rpu_last_error()


def test_philox_known_answers_on_host():
    import ctypes as C

    out = (C.c_uint32 * 4)()
    _cabi.check(_cabi.lib().rpu_philox4x32_10((C.c_uint32 * 4)(0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344),
                                              (C.c_uint32 * 2)(0xA4093822, 0x299F31D0), out))
    assert list(out) == [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]  # Random123 kat_vectors


def test_bench_refuses_more_than_one_gpu():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert proc.returncode == 2 and "one GPU" in proc.stderr


def test_product_does_not_touch_the_oracle():
    for base, _, files in os.walk(os.path.join(ROOT, "aihwkit_amd")):
        for name in files:
            if name.endswith((".py", ".cpp", ".hip", ".h", "Makefile")):
                assert "oracle" not in open(os.path.join(base, name), errors="ignore").read().lower(), name


def test_extra_state_and_maintenance_calls_on_a_host_tile():
    """dump_extra / load_extra work without a GPU; the weight maintenance calls compute on the GPU only and say so."""
    import ctypes as C

    from aihwkit_amd._cabi import lib
    from aihwkit_amd.rpu_base import devices as dv

    meta = dv.AnalogTileParameter()
    tile = meta.create_array(6, 4, dv.ConstantStepResistiveDeviceParameter())
    tile.set_seed(77)
    state = tile.dump_extra()
    assert state["rpu.seed"] == 77 and state["rpu.call"] == 0 and set(state) >= {"rpu.update_calls", "rpu.transfer.update_idx"}
    other = meta.create_array(6, 4, dv.ConstantStepResistiveDeviceParameter())
    other.load_extra({"rpu.seed": 5, "rpu.call": 9}, False)
    assert other.dump_extra()["rpu.seed"] == 5 and other.dump_extra()["rpu.call"] == 9
    with pytest.raises(RuntimeError, match="Cannot find the key"):
        other.load_extra({"rpu.seed": 5}, True)
    other.load_extra(state, True)
    assert other.dump_extra() == state
    # a transfer compound carries its counters
    tr = dv.TransferResistiveDeviceParameter()
    tr.append_parameter(dv.SoftBoundsResistiveDeviceParameter())
    tr.append_parameter(dv.SoftBoundsResistiveDeviceParameter())
    compound = meta.create_array(6, 4, tr)
    assert any(name.startswith("rpu.transfer.slice_idx_") for name in compound.dump_extra())
    with pytest.raises(RuntimeError):
        compound.load_extra(state, True)                       # another layout: the slice counters are missing
    # no CPU compute path: maintenance needs the tile on a GPU
    for call in (lambda: lib().rpu_tile_decay_weights(tile._h, C.c_float(1.0), 0, None),
                 lambda: lib().rpu_tile_diffuse_weights(tile._h, None),
                 lambda: lib().rpu_tile_clip_weights(tile._h, 1, C.c_float(0.1), C.c_float(2.5), None),
                 lambda: lib().rpu_tile_reset_columns(tile._h, 0, 1, C.c_float(1.0), None)):
        assert call() != 0 and b"GPU" in lib().rpu_last_error()
    assert not tile.get_shared_weights_if()


def test_parameter_accessors_and_random_weights_on_a_host_tile():
    import copy

    import torch

    from aihwkit_amd.rpu_base import devices as dv

    meta = dv.AnalogTileParameter()
    meta.forward_io.out_noise = 0.01
    dev = dv.SoftBoundsResistiveDeviceParameter()
    dev.dw_min = 0.002
    tile = meta.create_array(7, 5, dev)
    assert tile.get_meta_parameters().forward_io.out_noise == 0.01 and tile.get_parameters().dw_min == 0.002
    meta.forward_io.out_noise = 0.5                                     # the tile keeps what it was built from
    assert tile.get_meta_parameters().forward_io.out_noise == 0.01
    assert copy.deepcopy(tile).get_parameters().dw_min == 0.002
    torch.manual_seed(0)
    tile.set_weights_uniform_random(-0.2, 0.1)
    w = tile.get_weights()
    assert w.min() >= -0.2 and w.max() <= 0.1 and w.std() > 0.03
    hidden = dict(zip(tile.get_hidden_parameter_names(), tile.get_hidden_parameters()))
    assert (w <= hidden["max_bound"]).all() and (w >= hidden["min_bound"]).all()
    for name in ("drift_weights", "remap_weights", "modify_weights"):       # they work on the matrix in HBM
        with pytest.raises(RuntimeError, match="Host tiles do not compute"):
            getattr(tile, name)()
    assert tile.get_pulse_counters().numel() == 0                           # count_pulses is off
    dev.count_pulses = True
    dev.drift.nu = 0.05
    dev.drift.nu_dtod = 0.1
    counting = meta.create_array(7, 5, dev)
    assert counting.get_pulse_counters().shape == (2, 5, 7) and counting.get_pulse_counters().sum() == 0
    nu = dict(zip(counting.get_hidden_parameter_names(), counting.get_hidden_parameters()))["drift_nu"]
    assert abs(float(nu.mean()) - 0.05) < 0.005 and 0.002 < float(nu.std()) < 0.01   # nu (1 + nu_dtod N(0, 1))
    assert float(hidden["drift_nu"].abs().max()) == 0.0                     # no drifter: zeros, as the reference
    assert dv.SoftBoundsResistiveDeviceParameter().drift.nu == 0.0          # a struct of its own per object
    fp = dv.FloatingPointTileParameter().create_array(3, 2)
    assert fp.get_meta_parameters().lifetime == 0.0
