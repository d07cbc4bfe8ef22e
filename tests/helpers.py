"""Shared builders for the parity tests: parameter sets of the benchmark configurations and data."""
from aihwkit_amd.benchmark_configs import (CONFIG3_SHAPES, config1, config1_data, config2, config2_data, config3,  # noqa: F401
                                           constant_step, conv_index_matrix, io_params, make_meta, noise_free_io,
                                           soft_bounds, transfer_param)


def build_pair(meta, dev, x_size, d_size, gpu=True):
    """Host tile of the library, the oracle tile with the same configuration, and (optionally) the GPU tile."""
    from aihwkit_amd.rpu_base import tiles
    from oracle_lib import OracleTile

    cfg = meta._config(dev)
    host = meta.create_array(x_size, d_size, dev)
    orc = OracleTile(x_size, d_size, cfg)
    gpu_tile = tiles.CudaAnalogTile(host) if gpu else None
    return host, orc, gpu_tile


def build_transfer_pair(meta, tr, x_size, d_size, gpu=True):
    """Host transfer tile of the library, the transfer oracle with the same device arrays, optionally the GPU tile."""
    from aihwkit_amd.rpu_base import tiles
    from transfer_oracle import TransferOracle

    host = meta.create_array(x_size, d_size, tr)
    orc = TransferOracle(x_size, d_size, meta._config(tr._vec_par[0]), tr._to_transfer_c())
    names = host.get_hidden_parameter_names()
    hidden = host.get_hidden_parameters().numpy()
    start = 0
    for k in range(len(tr._vec_par)):
        stop = names.index(f"hidden_weights_{k}")
        orc.set_device_hidden(k, hidden[start:stop].copy())
        start = stop + 1
    gpu_tile = tiles.CudaAnalogTile(host) if gpu else None
    return host, orc, gpu_tile


def device_weights(tile, k):
    """Weights of device k of a transfer tile (the hidden_weights_k entry of its hidden parameters)."""
    names = tile.get_hidden_parameter_names()
    return tile.get_hidden_parameters()[names.index(f"hidden_weights_{k}")].numpy()


def transfer_draws(seed, update_idx, frm):
    """The two uniforms a tile with this seed draws on the host for the transfer of device `frm` after update vector
    `update_idx`: Philox4x32-10, counter (device, counter low, counter high, 17), key = seed; 24-bit uniforms."""
    import ctypes as C

    import numpy as np

    from aihwkit_amd import _cabi
    out = (C.c_uint32 * 4)()
    _cabi.check(_cabi.lib().rpu_philox4x32_10((C.c_uint32 * 4)(frm, update_idx & 0xFFFFFFFF, update_idx >> 32, 17),
                                              (C.c_uint32 * 2)(seed & 0xFFFFFFFF, seed >> 32), out))
    return [np.float32((v >> 8) * (1.0 / 16777216.0)) for v in out]
