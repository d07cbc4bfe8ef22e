"""GPU parity of the inference weight pipeline (PCM programming noise, drift, read noise, global drift
compensation) against the numpy PCM oracle: exact where the model is deterministic, by moments where it draws."""
import numpy as np
import pytest
import torch

from aihwkit_amd.inference import InferenceTile, PCMLikeNoiseModel
from aihwkit_amd.rpu_base import devices as dv
from helpers import io_params, make_meta, noise_free_io
from oracle_lib import OracleTile
from pcm_oracle import PcmOracle

pytestmark = pytest.mark.gpu

DAY = 86400.0


def make_tile(out_size, in_size, w, **model):
    tile = InferenceTile(out_size, in_size, forward_io=noise_free_io(inp_res=1 / 254.0, out_res=1 / 254.0),
                         noise_model=PCMLikeNoiseModel(**model))
    tile.set_weights(torch.from_numpy(w))
    return tile.cuda()


def test_deterministic_parts_match_the_oracle(gpu_device):
    rng = np.random.default_rng(0)
    w = rng.normal(0, 0.3, (96, 130)).astype(np.float32)
    tile = make_tile(96, 130, w, prog_noise_scale=0.0, read_noise_scale=0.0, g_min=1.0)
    tile.tile.set_seed(5)
    tile.program_weights()
    prog, nu_p, nu_m = (t.numpy() for t in tile.drift_state())
    assert np.abs(prog - w).max() <= 1e-6 and np.abs(tile.get_weights().numpy() - w).max() <= 1e-6
    orc = PcmOracle(prog_noise_scale=0.0, read_noise_scale=0.0, g_min=1.0)
    for t_inf in (0.0, 3600.0, DAY, 365 * DAY):
        tile.drift_weights(t_inf)
        want = orc.apply_drift_noise(prog, [nu_p, nu_m], t_inf)
        assert np.abs(tile.get_weights().numpy() - want).max() <= 1e-5, t_inf
    # drifting starts from the programmed weights every time, not from the drifted ones
    tile.drift_weights(0.0)
    assert np.abs(tile.get_weights().numpy() - prog).max() <= 1e-6
    # from_reference: programming again starts from the stored reference, not from the current weights
    tile.drift_weights(DAY)
    tile.program_weights(from_reference=True)
    assert np.abs(tile.get_weights().numpy() - w).max() <= 1e-6
    tile.set_weights(torch.from_numpy(2 * w))
    tile.program_weights(from_reference=False)
    assert np.abs(tile.get_weights().numpy() - 2 * w).max() <= 2e-6


def binned_moments(g_rel, values, edges):
    out = []
    for lo, hi in zip(edges[:-1], edges[1:]):
        sel = (g_rel >= lo) & (g_rel < hi)
        out.append((values[sel].mean(), values[sel].std(), int(sel.sum())))
    return out


def test_programming_noise_and_drift_coefficients_by_conductance_bin(gpu_device):
    rng = np.random.default_rng(1)
    w = rng.uniform(-1, 1, (512, 512)).astype(np.float32)
    w.flat[0] = 1.0
    tile = make_tile(512, 512, w)
    tile.tile.set_seed(7)
    tile.program_weights()
    prog, nu_p, nu_m = (t.numpy() for t in tile.drift_state())
    orc = PcmOracle(seed=11)
    want_prog, (want_nu_p, want_nu_m) = orc.apply_programming_noise(w)
    edges = np.linspace(0.0, 1.0, 9)
    g_rel = np.abs(w)
    for got, want, what in [(prog - w, want_prog - w, "programming error"), (np.where(w > 0, nu_p, nu_m),
                                                                             np.where(w > 0, want_nu_p, want_nu_m), "nu")]:
        for (m_g, s_g, n), (m_w, s_w, _) in zip(binned_moments(g_rel, got, edges), binned_moments(g_rel, want, edges)):
            assert abs(m_g - m_w) < 4.5 * np.hypot(s_g, s_w) / np.sqrt(n), what
            assert abs(s_g - s_w) < 4.5 * s_w / np.sqrt(2 * n) + 1e-9, what
    # the device that is not used sits at g_min = 0: half-normal programming noise, drift coefficient at the upper clips
    idle = np.where(w > 0, nu_m, nu_p)
    assert idle.mean() == pytest.approx(0.1, rel=0.02) and idle.std() == pytest.approx(0.045, rel=0.05)
    # the two conductances of a cross-point draw independently
    strong = w > 0.5
    assert abs(np.corrcoef(nu_p[strong], nu_m[strong])[0, 1]) < 0.03
    # a second programming run draws new noise, a re-seeded one repeats
    tile.program_weights()
    again = tile.drift_state()[0].numpy()
    assert np.abs(again - prog).max() > 1e-3
    tile.tile.set_seed(7)
    tile.program_weights()
    assert np.array_equal(tile.drift_state()[0].numpy(), prog)


def test_drift_with_read_noise_by_conductance_bin(gpu_device):
    rng = np.random.default_rng(2)
    w = rng.uniform(-1, 1, (512, 512)).astype(np.float32)
    w.flat[0] = -1.0
    tile = make_tile(512, 512, w, prog_noise_scale=0.0)
    tile.tile.set_seed(9)
    tile.program_weights()
    prog, nu_p, nu_m = (t.numpy() for t in tile.drift_state())
    tile.drift_weights(DAY)
    got = tile.get_weights().numpy()
    want = PcmOracle(prog_noise_scale=0.0, seed=21).apply_drift_noise(prog, [nu_p, nu_m], DAY)
    clean = PcmOracle(prog_noise_scale=0.0, read_noise_scale=0.0).apply_drift_noise(prog, [nu_p, nu_m], DAY)
    edges = np.linspace(0.0, 1.0, 9)
    for (m_g, s_g, n), (m_w, s_w, _) in zip(binned_moments(np.abs(w), got - clean, edges),
                                            binned_moments(np.abs(w), want - clean, edges)):
        assert abs(m_g - m_w) < 4.5 * np.hypot(s_g, s_w) / np.sqrt(n)
        assert abs(s_g - s_w) < 4.5 * s_w / np.sqrt(2 * n)


def test_global_drift_compensation_restores_the_output_level(gpu_device):
    rng = np.random.default_rng(3)
    w = rng.normal(0, 0.25, (256, 384)).astype(np.float32)
    tile = make_tile(256, 384, w)
    tile.tile.set_seed(3)
    tile.program_weights()
    assert tile.alpha == 1.0 and tile.drift_baseline > 0
    # the read-out is the mean |output| of the unit vectors = mean |programmed weight| up to the ADC
    assert tile.drift_baseline == pytest.approx(np.abs(tile.get_weights().numpy()).mean(), rel=0.05)
    x = torch.from_numpy(rng.normal(0, 1, (64, 384)).astype(np.float32)).cuda()
    fresh = tile.forward(x, is_test=True).cpu().numpy()
    tile.drift_weights(30 * DAY)
    assert tile.alpha == pytest.approx((30 * DAY / 20.0) ** 0.06, rel=0.15)      # typical nu ~ 0.06
    raw = tile.forward(x, is_test=False).cpu().numpy()
    compensated = tile.forward(x, is_test=True).cpu().numpy()
    assert np.abs(raw).mean() < 0.7 * np.abs(fresh).mean()
    assert np.abs(compensated).mean() == pytest.approx(np.abs(fresh).mean(), rel=0.05)
    assert np.corrcoef(compensated.ravel(), fresh.ravel())[0, 1] > 0.97


def test_inference_forward_after_drift_matches_the_oracle_tile(gpu_device):
    """Transformer-width tile (512 x 512, 1024 tokens, 8-bit converters) with drifted weights: the analog
    forward pass on those weights against the CPU oracle tile holding the same weights."""
    rng = np.random.default_rng(4)
    w = rng.normal(0, 0.02, (512, 512)).astype(np.float32)
    io = noise_free_io(inp_res=1 / 254.0, out_res=1 / 254.0, noise_management=dv.NoiseManagementType.AbsMax)
    tile = InferenceTile(512, 512, forward_io=io)
    tile.set_weights(torch.from_numpy(w))
    tile.cuda()
    tile.tile.set_seed(1)
    tile.drift_weights(DAY)                      # programs first
    drifted = tile.get_weights().numpy()
    assert 0.4 < np.abs(drifted).mean() / np.abs(w).mean() < 0.9
    meta = make_meta(io, noise_free_io())
    meta.backward_io.is_perfect = True
    meta.update.pulse_type = dv.PulseType.NONE
    orc = OracleTile(512, 512, meta._config(dv.IdealResistiveDeviceParameter()))
    orc.set_weights(drifted)
    x = rng.normal(0, 1, (1024, 512)).astype(np.float32)
    got = tile.forward(torch.from_numpy(x).cuda(), is_test=False).cpu().numpy()
    want = orc.forward(x)
    step = np.abs(x).max(1, keepdims=True) * 24.0 / 254.0        # one ADC code after noise management
    off = np.abs(got - want) > 1e-5
    assert off.mean() < 0.005 and np.all(np.abs(got - want)[off] <= 1.001 * np.broadcast_to(step, got.shape)[off])


def test_pipeline_needs_an_ideal_device_gpu_tile(gpu_device):
    from helpers import build_pair, constant_step
    _, _, gpu = build_pair(make_meta(), constant_step(), 8, 8)
    from aihwkit_amd._cabi import PcmNoiseParams, lib
    import ctypes as C
    p = PcmNoiseParams()
    assert lib().rpu_pcm_noise_params_default(C.byref(p)) == 0 and p.g_max == 25.0
    assert lib().rpu_tile_program_weights(gpu._h, C.byref(p), 1, None) != 0
    assert b"ideal device" in lib().rpu_last_error()


def test_grouped_forward_equals_the_tiles_own_forward(gpu_device):
    """Tiles of different shapes and kernel variants, noise on: a group call must give every tile bit for bit
    what its own forward call gives for the same seed and call counter."""
    import copy

    from aihwkit_amd.rpu_base import tiles as tl
    from helpers import build_pair, constant_step

    rng = np.random.default_rng(6)
    shapes = [(384, 461), (512, 384), (384, 460), (100, 70), (128, 64), (512, 512)]   # (x_size, d_size)
    batch = 96
    f_io = io_params(inp_res=1 / 254.0, out_res=1 / 254.0, out_noise=0.04, noise_management=dv.NoiseManagementType.AbsMax,
                     bound_management=dv.BoundManagementType.Iterative)
    singles, grouped, xs = [], [], []
    for k, (x_size, d_size) in enumerate(shapes):
        io = f_io if k != 4 else noise_free_io(is_perfect=True)       # one tile with a perfect forward pass
        _, _, gpu = build_pair(make_meta(io, noise_free_io()), constant_step(construction_seed=k + 1), x_size, d_size)
        scale = 0.5 if k == 1 else 0.05                                # one tile saturates: several rounds
        gpu.set_weights(torch.from_numpy(rng.normal(0, scale, (d_size, x_size)).astype(np.float32)))
        gpu.set_seed(40 + k)
        singles.append(gpu)
        grouped.append(copy.deepcopy(gpu))
        grouped[-1].set_seed(40 + k)
        xs.append(torch.from_numpy(rng.normal(0, 1, (batch, x_size)).astype(np.float32)).cuda())
    group = tl.TileGroup(grouped)
    for _ in range(3):                                                 # the call counters advance together
        want = [t.forward(x, False, False, False, False, False) for t, x in zip(singles, xs)]
        got = group.forward(xs)
        for k, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a, b), k
    assert singles[1].get_bm_rounds(batch).max() > 1
    assert torch.equal(grouped[1].get_bm_rounds(batch), singles[1].get_bm_rounds(batch))
    with pytest.raises(RuntimeError):
        tl.TileGroup([grouped[0], grouped[0]])
    with pytest.raises(RuntimeError):
        group.forward(xs[:-1])


def test_grouped_forward_at_a_token_batch_is_exact_in_exact_arithmetic(gpu_device):
    """At a batch of 1024 the group runs round 0 on 128 x 128 workgroup tiles (another summation order than a tile's
    own forward).  With a power-of-two DAC step and weights on a 1/64 grid every partial sum is exact, so group,
    single-tile call and oracle must still agree to the last bit; one narrow tile stays on the 32 x 32 kernel."""
    from aihwkit_amd.rpu_base import tiles as tl
    from helpers import build_pair, constant_step

    rng = np.random.default_rng(8)
    batch = 1024
    shapes = [(70, 512), (96, 512), (130, 512), (64, 500), (33, 512), (70, 512), (96, 512), (130, 512), (64, 512),
              (50, 40)]
    f_io = noise_free_io(inp_res=1 / 128.0, out_res=1 / 512.0, noise_management=dv.NoiseManagementType.AbsMax,
                         bound_management=dv.BoundManagementType.Iterative)
    grouped, oracles, xs = [], [], []
    for k, (x_size, d_size) in enumerate(shapes):
        dev = constant_step(w_max_dtod=0.0, w_min_dtod=0.0, w_max=1.0, w_min=-1.0, construction_seed=k + 1)
        host, orc, _ = build_pair(make_meta(f_io, noise_free_io()), dev, x_size, d_size, gpu=False)
        w = (rng.integers(-60, 61, (d_size, x_size)) / 64.0).astype(np.float32)
        host.set_weights(torch.from_numpy(w))
        orc.set_weights(w)
        grouped.append(tl.CudaAnalogTile(host))
        oracles.append(orc)
        xs.append(rng.uniform(-1, 1, (batch, x_size)).astype(np.float32))
    group = tl.TileGroup(grouped)
    got = group.forward([torch.from_numpy(x).cuda() for x in xs])
    for k, (y, orc, x) in enumerate(zip(got, oracles, xs)):
        assert np.array_equal(y.cpu().numpy(), orc.forward(x)), k
        assert np.array_equal(grouped[k].get_bm_rounds(batch).numpy(), orc.bm_rounds(batch)), k
    assert oracles[2].bm_rounds(batch).max() > 1                       # the later rounds were exercised


def test_group_reads_and_writes_column_slices_and_compensation_in_the_tile(gpu_device):
    """Strided group call: inputs as column slices of the layer input, outputs as column slices of one matrix, must
    give bit for bit what the dense call gives; the drift-compensation factor on the ADC stage equals the multiply."""
    from aihwkit_amd.rpu_base import tiles as tl

    rng = np.random.default_rng(9)
    batch, in_sizes, out_sizes = 40, (24, 36), (17, 30, 9)
    f_io = io_params(inp_res=1 / 254.0, out_res=1 / 254.0, out_noise=0.04, noise_management=dv.NoiseManagementType.AbsMax,
                     bound_management=dv.BoundManagementType.Iterative)
    inf_tiles = []
    for n_in in in_sizes:
        for n_out in out_sizes:
            t = InferenceTile(n_out, n_in, forward_io=f_io)
            t.set_weights(torch.from_numpy(rng.normal(0, 0.1, (n_out, n_in)).astype(np.float32)))
            t.cuda()
            t.tile.set_seed(100 + len(inf_tiles))
            t.drift_weights(1000.0)
            inf_tiles.append(t)
    assert all(abs(t.alpha - 1.0) > 1e-3 for t in inf_tiles)
    x = torch.from_numpy(rng.normal(0, 1, (batch, sum(in_sizes))).astype(np.float32)).cuda()
    x_slices, i0 = [], 0
    for n_in in in_sizes:
        x_slices += [x[:, i0:i0 + n_in]] * len(out_sizes)
        i0 += n_in
    group = tl.TileGroup([t.tile for t in inf_tiles])
    for t in inf_tiles:
        t.tile.set_seed(5)
    dense = group.forward([s.contiguous() for s in x_slices], is_test=True)
    partial = torch.full((len(in_sizes), batch, sum(out_sizes)), 7.0, device="cuda")
    outs = []
    for i in range(len(in_sizes)):
        o0 = 0
        for n_out in out_sizes:
            outs.append(partial[i][:, o0:o0 + n_out])
            o0 += n_out
    for t in inf_tiles:
        t.tile.set_seed(5)
    got = group.forward(x_slices, is_test=True, outs=outs)
    for k, (a, b) in enumerate(zip(got, dense)):
        assert torch.equal(a, b), k
    assert torch.equal(partial[1][:, :out_sizes[0]], dense[len(out_sizes)])
    # the compensation factor in the tile
    for t in inf_tiles:
        t.tile.set_seed(5)
        t.compensate_in_tile(True)
    folded = group.forward(x_slices, is_test=True)
    for t, a, b in zip(inf_tiles, folded, dense):
        assert torch.allclose(a, b * t.alpha, rtol=1e-6, atol=1e-7)
    # a later drift step measures the uncompensated tile and renews the factor in the tile
    t = inf_tiles[0]
    before = t.alpha
    t.drift_weights(1.0e6)
    assert t.alpha > before * 1.01
    t.tile.set_seed(5)
    y_tile = t.forward(x_slices[0].contiguous(), is_test=True)
    t.compensate_in_tile(False)
    t.tile.set_seed(5)
    y_mul = t.forward(x_slices[0].contiguous(), is_test=True)
    assert torch.allclose(y_tile, y_mul, rtol=1e-6, atol=1e-7)
    with pytest.raises(RuntimeError):
        group.forward(x_slices, outs=outs[:-1])
    with pytest.raises(RuntimeError):
        group.forward([s.t() for s in x_slices])


@pytest.mark.parametrize("c_in,c_out", [(1, 16), (16, 32), (4, 48)])     # the two fused kernels and the unfolded path
def test_compensation_in_the_tile_for_a_convolution(gpu_device, c_in, c_out):
    """The drift-compensation factor on the ADC stage of the indexed forward equals the multiply of its output."""
    from aihwkit_amd.benchmark_configs import conv_index_matrix

    rng = np.random.default_rng(c_out)
    f_io = io_params(inp_res=1 / 254.0, out_res=1 / 254.0, out_noise=0.04, noise_management=dv.NoiseManagementType.AbsMax,
                     bound_management=dv.BoundManagementType.Iterative)
    indices, patches = conv_index_matrix((c_in, 12, 12), (5, 5))
    in_size = c_in * 25 + 1
    t = InferenceTile(c_out, in_size, forward_io=f_io)
    t.set_weights(torch.from_numpy((rng.uniform(-1, 1, (c_out, in_size)) / np.sqrt(in_size)).astype(np.float32)))
    t.cuda()
    t.set_matrix_indices(indices)
    t.drift_weights(86400.0)
    assert abs(t.alpha - 1.0) > 1e-3
    x = torch.from_numpy(rng.uniform(0, 1, (6, c_in, 12, 12)).astype(np.float32)).cuda()
    t.tile.set_seed(9)
    y_mul = t.forward_indexed(x, torch.empty(6, c_out, 8, 8, device="cuda"), is_test=True).clone()
    t.compensate_in_tile(True)
    t.tile.set_seed(9)
    y_tile = t.forward_indexed(x, torch.empty(6, c_out, 8, 8, device="cuda"), is_test=True)
    assert patches == 64 and y_mul.abs().max() > 0.1
    assert torch.allclose(y_tile, y_mul, rtol=1e-6, atol=1e-7)


def test_grouped_backward_equals_the_tiles_own_backward(gpu_device):
    """Noisy backward pass (abs-max noise management) of tiles of different shapes: the group call gives every tile bit
    for bit what its own backward call gives for the same seed and call counter; strided gradients are filled in place."""
    import copy

    from aihwkit_amd.rpu_base import tiles as tl
    from helpers import build_pair, constant_step

    rng = np.random.default_rng(12)
    shapes = [(384, 461), (512, 384), (100, 70), (129, 10)]            # (x_size, d_size)
    batch = 80
    b_io = io_params(inp_res=1 / 254.0, out_res=1 / 254.0, out_noise=0.04, noise_management=dv.NoiseManagementType.AbsMax)
    singles, grouped, ds = [], [], []
    for k, (x_size, d_size) in enumerate(shapes):
        _, _, gpu = build_pair(make_meta(noise_free_io(), b_io), constant_step(construction_seed=k + 1), x_size, d_size)
        gpu.set_weights(torch.from_numpy(rng.normal(0, 0.1, (d_size, x_size)).astype(np.float32)))
        gpu.set_seed(60 + k)
        singles.append(gpu)
        grouped.append(copy.deepcopy(gpu))
        grouped[-1].set_seed(60 + k)
        ds.append(torch.from_numpy(rng.normal(0, 0.3, (batch, d_size)).astype(np.float32)).cuda())
    group = tl.TileGroup(grouped)
    all_x = torch.zeros(batch, sum(x for x, _ in shapes), device="cuda")
    outs, i0 = [], 0
    for x_size, _ in shapes:
        outs.append(all_x[:, i0:i0 + x_size])
        i0 += x_size
    for rep in range(2):
        want = [t.backward(d, False, False, False, False) for t, d in zip(singles, ds)]
        got = group.backward(ds, outs=outs if rep else None)
        for k, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a, b), (rep, k)
    assert torch.equal(all_x[:, :shapes[0][0]], want[0])
    assert want[0].abs().max() > 0.1
