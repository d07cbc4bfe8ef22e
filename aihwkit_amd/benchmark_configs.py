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


# ---- configuration 5: the GPT-2-small linear layers as PCM inference tiles ---------------------------------------

# split into tiles of at most 512 x 512 the way the reference's tile array does
# (src/aihwkit/simulator/tiles/array.py:82-97): (in, out, input splits, output splits)
CONFIG5_LAYERS = (
    (768, 2304, (384, 384), (461, 461, 461, 461, 460)),
    (768, 768, (384, 384), (384, 384)),
    (768, 3072, (384, 384), (512,) * 6),
    (3072, 768, (512,) * 6, (384, 384)),
)


def config5_io(out_noise=0.04):
    return io_params(inp_res=1 / 254.0, out_res=1 / 254.0, out_noise=out_noise,
                     noise_management=dv.NoiseManagementType.AbsMax,
                     bound_management=dv.BoundManagementType.Iterative)


def config5_layers(tokens=1024, io=None, noise_model=None, t_inference=86400.0, seed=0):
    """The 38 tiles, on the GPU: weights N(0, 0.02), programmed with ``noise_model`` (default: the PCM model) and
    drifted to ``t_inference`` seconds.  Returns per layer a list of (x_part [tokens, n_in], row of tiles), one entry
    per input split; the inputs are N(0, 1)."""
    from aihwkit_amd.inference import InferenceTile
    rng = np.random.default_rng(seed)
    io = io or config5_io()
    layers, n_tiles = [], 0
    for in_size, out_size, in_split, out_split in CONFIG5_LAYERS:
        x = torch.from_numpy(rng.standard_normal((tokens, in_size)).astype(np.float32)).cuda()
        grid, i0 = [], 0
        for n_in in in_split:
            row = []
            for n_out in out_split:
                tile = InferenceTile(n_out, n_in, forward_io=io, noise_model=noise_model)
                tile.set_weights(torch.from_numpy((0.02 * rng.standard_normal((n_out, n_in))).astype(np.float32)))
                tile.cuda()
                tile.tile.set_seed(1000 + n_tiles)
                tile.drift_weights(t_inference)
                row.append(tile)
                n_tiles += 1
            grid.append((x[:, i0:i0 + n_in].contiguous(), row))
            i0 += n_in
        layers.append(grid)
    return layers


def config5_groups(layers, tokens=1024):
    """One tile group per layer: all tiles of the layer in a few launches.  The tiles read column slices of the layer
    input and write column slices of one partial-output matrix per input split in place; the drift-compensation
    factor of a tile rides on its ADC stage.  Returns per layer (group, tiles, inputs, outputs, partial [splits,
    tokens, out_size])."""
    from aihwkit_amd.rpu_base.tiles import TileGroup
    groups = []
    for (in_size, out_size, in_split, out_split), grid in zip(CONFIG5_LAYERS, layers):
        x_layer = torch.cat([x_part for x_part, _ in grid], dim=1)                       # [tokens, in_size]
        partial = torch.empty(len(in_split), tokens, out_size, device="cuda")
        flat_tiles, flat_x, flat_y, i0 = [], [], [], 0
        for i, (n_in, (_, row)) in enumerate(zip(in_split, grid)):
            o0 = 0
            for tile, n_out in zip(row, out_split):
                tile.compensate_in_tile(True)
                flat_tiles.append(tile)
                flat_x.append(x_layer[:, i0:i0 + n_in])
                flat_y.append(partial[i][:, o0:o0 + n_out])
                o0 += n_out
            i0 += n_in
        groups.append((TileGroup([t.tile for t in flat_tiles]), flat_tiles, flat_x, flat_y, partial))
    return groups


def config5_step(groups):
    """Forward pass of all tiles; the partial outputs of the input splits are summed digitally."""
    outs = []
    for group, _, flat_x, flat_y, partial in groups:
        group.forward(flat_x, is_test=True, non_blocking=True, outs=flat_y)
        outs.append(partial.sum(dim=0) if partial.shape[0] > 1 else partial[0])
    return outs
