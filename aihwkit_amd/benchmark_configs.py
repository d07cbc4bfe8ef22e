"""Parameter sets and synthetic data of the benchmark configurations (tile shapes, device and IO settings, seeded
inputs), shared by bench.py and the parity tests."""
import numpy as np
import torch

from aihwkit_amd.rpu_base import devices as dv


def io_params(**kw):
    io = dv.AnalogTileInputOutputParameter()
    for k, v in kw.items():
        setattr(io, k, v)
    return io


def noise_free_io(**kw):
    base = dict(out_noise=0.0, inp_noise=0.0)
    base.update(kw)
    return io_params(**base)


def make_meta(f_io=None, b_io=None, **up):
    meta = dv.AnalogTileParameter()
    if f_io is not None:
        meta.forward_io = f_io
    if b_io is not None:
        meta.backward_io = b_io
    for k, v in up.items():
        setattr(meta.update, k, v)
    return meta


def constant_step(**kw):
    d = dv.ConstantStepResistiveDeviceParameter()
    for k, v in kw.items():
        setattr(d, k, v)
    return d


def soft_bounds(**kw):
    d = dv.SoftBoundsResistiveDeviceParameter()
    for k, v in kw.items():
        setattr(d, k, v)
    return d


def config1(noise=True):
    """512 x 512 ConstantStep without variation (benchmark configuration 1)."""
    on = 0.06 if noise else 0.0
    f_io = io_params(inp_res=1 / 127.0, out_res=1 / 511.0, out_noise=on,
                     noise_management=dv.NoiseManagementType.AbsMax,
                     bound_management=dv.BoundManagementType.Iterative)
    b_io = io_params(inp_res=1 / 127.0, out_res=1 / 511.0, out_noise=on,
                     noise_management=dv.NoiseManagementType.AbsMax)
    meta = make_meta(f_io, b_io, desired_bl=31)
    dev = constant_step(dw_min=0.001, dw_min_dtod=0.0, dw_min_std=0.0, up_down_dtod=0.0, w_max_dtod=0.0,
                        w_min_dtod=0.0, construction_seed=123, enforce_consistency=True)
    return meta, dev


def config2(noise=True, ctoc=True):
    """1024 x 1024 SoftBounds with device-to-device and cycle-to-cycle variation (configuration 2)."""
    on = 0.06 if noise else 0.0
    f_io = io_params(out_noise=on, noise_management=dv.NoiseManagementType.AbsMax,
                     bound_management=dv.BoundManagementType.Iterative)
    b_io = io_params(out_noise=on, noise_management=dv.NoiseManagementType.AbsMax)
    meta = make_meta(f_io, b_io, desired_bl=31, update_management=True, update_bl_management=True)
    dev = soft_bounds(dw_min=0.001, dw_min_dtod=0.3, dw_min_std=0.3 if ctoc else 0.0, up_down=0.0,
                      up_down_dtod=0.01, w_max=0.6, w_min=-0.6, w_max_dtod=0.3, w_min_dtod=0.3,
                      construction_seed=123, enforce_consistency=True)
    return meta, dev


def config3(noise=True):
    """Tiki-Taka transfer compound of two SoftBounds devices (A fast, C slow): one column transferred every two
    mini-batches (configuration 3; settings of examples/08_simple_layer_with_tiki_taka.py:29-45 of the reference)."""
    on = 0.06 if noise else 0.0
    f_io = io_params(out_noise=on, noise_management=dv.NoiseManagementType.AbsMax,
                     bound_management=dv.BoundManagementType.Iterative)
    b_io = io_params(out_noise=on, noise_management=dv.NoiseManagementType.AbsMax)
    meta = make_meta(f_io, b_io, desired_bl=31, update_management=True, update_bl_management=True)
    fast = soft_bounds(w_min=-0.3, w_max=0.3, enforce_consistency=True)
    slow = soft_bounds(w_min=-0.6, w_max=0.6, enforce_consistency=True)
    tr = transfer_param([fast, slow], construction_seed=123, units_in_mbatch=True, transfer_every=2.0,
                        n_reads_per_transfer=1, gamma=0.0, scale_transfer_lr=True, transfer_lr=1.0, fast_lr=0.1,
                        transfer_columns=True)
    tr.transfer_forward = io_params(out_noise=on)
    return meta, tr


CONFIG3_SHAPES = ((785, 256), (257, 128), (129, 10))  # (x_size with bias column, d_size) of the MLP 784-256-128-10


def config2_data(x_size=1024, d_size=1024, batch=256):
    w = np.random.default_rng(0).uniform(-0.6, 0.6, (d_size, x_size)).astype(np.float32)
    x = np.random.default_rng(1).uniform(-1, 1, (batch, x_size)).astype(np.float32)
    d = (0.05 * np.random.default_rng(2).standard_normal((batch, d_size))).astype(np.float32)
    return w, x, d


def config1_data(x_size=512, d_size=512, batch=100):
    w = np.random.default_rng(0).uniform(-0.6, 0.6, (d_size, x_size)).astype(np.float32)
    x = np.random.default_rng(1).uniform(-1, 1, (batch, x_size)).astype(np.float32)
    d = (0.1 * np.random.default_rng(2).standard_normal((batch, d_size))).astype(np.float32)
    return w, x, d


def transfer_param(devices, **kw):
    """TransferResistiveDeviceParameter over the given device parameters."""
    tr = dv.TransferResistiveDeviceParameter()
    for d in devices:
        assert tr.append_parameter(d)
    for k, v in kw.items():
        setattr(tr, k, v)
    return tr




def conv_index_matrix(image_shape, kernel, with_bias=True):
    """Index matrix of an unpadded stride-1 2-d convolution: entry [k, p] names the image element (offset by 2) that
    patch p reads at kernel position k; 1 marks the bias row.  Returns (int32 indices [x_size * patches], patches)."""
    import torch.nn.functional as F

    size = int(torch.tensor(image_shape).prod())
    numbered = torch.arange(2, size + 2, dtype=torch.float32).reshape(1, *image_shape)
    unfolded = F.unfold(numbered, kernel_size=kernel)[0]                       # [C k k, patches]
    if with_bias:
        unfolded = torch.cat([unfolded, torch.ones(1, unfolded.shape[1])], dim=0)
    return unfolded.to(torch.int32).contiguous().reshape(-1), unfolded.shape[1]
