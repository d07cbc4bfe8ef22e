"""GPU parity of the analog non-idealities that act before the ADC (IR drop, output-referred weight noise) against
the CPU restatement, through the Python mirror over the C ABI."""
import numpy as np
import pytest
import torch

from aihwkit_amd.rpu_base import devices as dv
from aihwkit_amd.rpu_base import tiles
from helpers import build_pair, constant_step, io_params, make_meta

pytestmark = pytest.mark.gpu
F = np.float32


def pair(x_size, d_size, seed=0, **io):
    base = dict(out_noise=0.0, inp_noise=0.0, out_res=-1.0)
    base.update(io)
    meta = make_meta(io_params(**base), io_params(**base))
    dev = constant_step(w_max=1.0, w_min=-1.0, w_max_dtod=0.0, w_min_dtod=0.0, construction_seed=1)
    host, orc, gpu = build_pair(meta, dev, x_size, d_size)
    w = np.random.default_rng(seed).uniform(-0.6, 0.6, (d_size, x_size)).astype(F)
    host.set_weights(torch.from_numpy(w))
    orc.set_weights(w)
    gpu = tiles.CudaAnalogTile(host)
    return orc, gpu, w


@pytest.mark.parametrize("shape", [(37, 23, 50), (300, 200, 96), (129, 10, 33)])
def test_ir_drop_with_quantized_inputs_and_bound_management(gpu_device, shape):
    x_size, d_size, batch = shape
    rng = np.random.default_rng(1)
    w = np.random.default_rng(0).uniform(-0.6, 0.6, (d_size, x_size)).astype(F)   # the weights `pair` sets
    x = rng.uniform(-1, 1, (batch, x_size)).astype(F)
    x[3] = 0.0                                                    # a zero sample short-cuts to zero
    x[5] *= 0.01
    x[7] = np.sign(w[0])                                          # one output far beyond the bound: many rounds
    d = rng.normal(0, 0.5, (batch, d_size)).astype(F)
    mean_current = 0.3 * 0.5 * x_size                             # sum_j |w_ij| |x_j| of a typical output
    # ADC bound at the median over the samples of the largest output: about half of them need a second round
    scaled = x / np.maximum(np.abs(x).max(axis=1, keepdims=True), 1e-9)
    out_bound = float(np.median(np.abs(scaled @ w.T).max(axis=1)))
    for ir_drop, a_typ in ((1.0, 0.5), (2.5, 0.2)):
        io = dict(ir_drop=ir_drop, ir_drop_g_ratio=x_size * mean_current / a_typ, out_bound=out_bound,
                  noise_management=dv.NoiseManagementType.AbsMax, bound_management=dv.BoundManagementType.Iterative)
        orc, gpu, _w = pair(x_size, d_size, **io)
        plain_orc, _plain_gpu, _w = pair(x_size, d_size, **dict(io, ir_drop=0.0))
        want = orc.forward(x)
        got = gpu.forward(torch.from_numpy(x).cuda()).cpu().numpy()
        rounds = orc.bm_rounds(batch)
        # several rounds: the terms follow the rescaled rows of the samples that are still listed
        assert rounds.max() >= 3 and (rounds == 1).sum() >= 3 and (rounds == 2).sum() >= 3
        assert np.array_equal(gpu.get_bm_rounds(batch).numpy(), rounds)
        # tolerance 1e-5 of the output range: three contractions summed in another order than the oracle's loops
        scale = np.abs(want).max()
        assert np.abs(got - want).max() <= 1e-5 * scale
        assert np.abs(want - plain_orc.forward(x)).max() > 1e-2 * scale   # the drop itself is far above the tolerance
        assert not got[3].any()
        want_b = orc.backward(d)
        got_b = gpu.backward(torch.from_numpy(d).cuda()).cpu().numpy()
        assert np.abs(got_b - want_b).max() <= 1e-5 * np.abs(want_b).max()
        assert np.abs(want_b - plain_orc.backward(d)).max() > 1e-3 * np.abs(want_b).max()
        # transposed layouts take the same path
        got_t = gpu.forward(torch.from_numpy(np.ascontiguousarray(x.T)).cuda(), False, True, True).cpu().numpy()
        assert np.abs(got_t.T - want).max() <= 1e-5 * scale


def test_ir_drop_with_a_bias_column_and_adc_quantization(gpu_device):
    rng = np.random.default_rng(2)
    x = rng.uniform(-1, 1, (40, 64)).astype(F)
    io = dict(ir_drop=1.0, ir_drop_g_ratio=65 * 10.0 / 0.4, out_res=1.0 / 510, out_bound=12.0,
              noise_management=dv.NoiseManagementType.AbsMax, bound_management=dv.BoundManagementType.Iterative)
    orc, gpu, _w = pair(65, 31, **io)
    want = orc.forward(x, bias=True)
    got = gpu.forward(torch.from_numpy(x).cuda(), True).cpu().numpy()
    # an output may sit on the other side of an ADC rounding edge: every mismatch is one step and they are rare
    step = 24.0 / 510
    diff = np.abs(got - want)
    off = diff > 1e-5
    assert off.mean() < 5e-3 and np.allclose(diff[off], step, rtol=1e-3)


def moments_ok(z):
    n = z.size
    return abs(z.mean()) < 4 / np.sqrt(n) and abs(z.std() - 1) < 4 / np.sqrt(2 * n)


def test_weight_noise_variance_laws(gpu_device):
    rng = np.random.default_rng(3)
    x_size, d_size, batch = 96, 160, 64
    x = rng.uniform(-1, 1, (batch, x_size)).astype(F)
    d = rng.uniform(-1, 1, (batch, d_size)).astype(F)
    base = dict(inp_res=-1.0, out_bound=1e6, noise_management=dv.NoiseManagementType.NONE,
                bound_management=dv.BoundManagementType.NONE)
    x64, d64 = x.astype(np.float64), d.astype(np.float64)
    # additive constant: sigma = w_noise |x|_2 for every output
    _orc, gpu, w = pair(x_size, d_size, w_noise=0.05, w_noise_type=dv.WeightNoiseType.AdditiveConstant, **base)
    w64 = w.astype(np.float64)
    y = gpu.forward(torch.from_numpy(x).cuda()).cpu().numpy().astype(np.float64)
    z = (y - x64 @ w64.T) / (0.05 * np.linalg.norm(x64, axis=1))[:, None]
    assert moments_ok(z)
    y2 = gpu.forward(torch.from_numpy(x).cuda()).cpu().numpy().astype(np.float64)   # a new call draws anew
    z2 = (y2 - x64 @ w64.T) / (0.05 * np.linalg.norm(x64, axis=1))[:, None]
    assert moments_ok(z2) and abs(np.corrcoef(z.ravel(), z2.ravel())[0, 1]) < 4 / np.sqrt(z.size)
    assert abs(np.corrcoef(z[:, :-1].ravel(), z[:, 1:].ravel())[0, 1]) < 4 / np.sqrt(z.size)
    gx = gpu.backward(torch.from_numpy(d).cuda()).cpu().numpy().astype(np.float64)
    assert moments_ok((gx - d64 @ w64) / (0.05 * np.linalg.norm(d64, axis=1))[:, None])
    # together with the output noise the variances add
    _orc, gpu, w = pair(x_size, d_size, w_noise=0.05, w_noise_type=dv.WeightNoiseType.AdditiveConstant, out_noise=0.2,
                        **base)
    y = gpu.forward(torch.from_numpy(x).cuda()).cpu().numpy().astype(np.float64)
    sigma = np.sqrt((0.05 * np.linalg.norm(x64, axis=1)) ** 2 + 0.2 ** 2)
    assert moments_ok((y - x64 @ w.astype(np.float64).T) / sigma[:, None])
    # PCM read noise: sigma_i^2 = w_noise^2 sum_j |w_ij| x_j^2, transposed for the backward pass
    _orc, gpu, w = pair(x_size, d_size, w_noise=0.1, w_noise_type=dv.WeightNoiseType.PCMRead, **base)
    w64 = w.astype(np.float64)
    y = gpu.forward(torch.from_numpy(x).cuda()).cpu().numpy().astype(np.float64)
    z = (y - x64 @ w64.T) / (0.1 * np.sqrt((x64 ** 2) @ np.abs(w64.T)))
    assert moments_ok(z)
    quiet = np.argsort(np.abs(w64).sum(axis=1))[:20]             # per-output scale, not one scale per sample
    assert moments_ok(z[:, quiet])
    gx = gpu.backward(torch.from_numpy(d).cuda()).cpu().numpy().astype(np.float64)
    assert moments_ok((gx - d64 @ w64) / (0.1 * np.sqrt((d64 ** 2) @ np.abs(w64))))


def test_weight_noise_under_bound_management_and_other_paths(gpu_device):
    rng = np.random.default_rng(4)
    x_size, d_size, batch = 64, 48, 256
    x = rng.uniform(-1, 1, (batch, x_size)).astype(F)
    io = dict(w_noise=0.02, w_noise_type=dv.WeightNoiseType.PCMRead, ir_drop=1.0, ir_drop_g_ratio=64 * 10.0 / 0.3,
              out_bound=0.9, noise_management=dv.NoiseManagementType.AbsMax,
              bound_management=dv.BoundManagementType.Iterative)
    orc, gpu, _w = pair(x_size, d_size, **io)
    quiet_orc, quiet_gpu, _w = pair(x_size, d_size, **dict(io, w_noise=0.0))
    want = quiet_orc.forward(x)
    got = gpu.forward(torch.from_numpy(x).cuda()).cpu().numpy()
    rounds = gpu.get_bm_rounds(batch).numpy()
    assert rounds.max() >= 2 and np.abs(rounds - quiet_orc.bm_rounds(batch)).max() <= 1
    same = rounds == quiet_orc.bm_rounds(batch)
    resid = (got - want)[same]
    # the noise rides on the drifted sums of whichever round was the last one: small against the signal, not zero
    assert 0.01 < resid.std() < 0.15 and abs(resid.mean()) < 4 * resid.std() / np.sqrt(resid.size)
    # a group takes these tiles and runs them one after the other, each with the launches of its own call (bound to a
    # shared tensor they mirror it, and the group refuses them at once)
    if tiles.CudaAnalogTile.bind_shared_weights:
        with pytest.raises(RuntimeError, match="cannot be in a group"):
            tiles.TileGroup([gpu, quiet_gpu])
        return
    _orc, twin, _w = pair(x_size, d_size, **io)
    gpu.set_seed(77)
    twin.set_seed(77)                                                          # same seed, same call numbers: same draws
    d = rng.normal(0, 0.5, (batch, d_size)).astype(F)
    group = tiles.TileGroup([gpu, quiet_gpu])
    wide = torch.zeros(batch, x_size + 24).cuda()                              # inputs and outputs as column slices
    wide[:, 8:8 + x_size] = torch.from_numpy(x).cuda()
    outs = [torch.zeros(batch, d_size + 8).cuda()[:, 3:3 + d_size], torch.empty(batch, d_size).cuda()]
    ys = group.forward([wide[:, 8:8 + x_size], torch.from_numpy(x).cuda()], outs=outs)
    assert torch.equal(ys[0], twin.forward(torch.from_numpy(x).cuda()))
    assert torch.equal(ys[1], quiet_gpu.forward(torch.from_numpy(x).cuda()))
    assert torch.equal(outs[0], ys[0])                                          # written through the column slice
    gs = group.backward([torch.from_numpy(d).cuda(), torch.from_numpy(d).cuda()])
    assert torch.equal(gs[0], twin.backward(torch.from_numpy(d).cuda()))
    assert torch.equal(gs[1], quiet_gpu.backward(torch.from_numpy(d).cuda()))


@pytest.mark.parametrize("bm", [dv.BoundManagementType.NONE, dv.BoundManagementType.Iterative,
                                dv.BoundManagementType.IterativeWorstCase])
def test_running_average_noise_management_is_bit_exact_and_shared(gpu_device, bm):
    """AverageAbsMax in the exact-arithmetic setting: the scale of a sample depends on every sample before it, in this
    call and in earlier forward and backward calls; outputs, rounds and the continuation must equal the oracle's."""
    rng = np.random.default_rng(11)
    x_size, d_size = 100, 70
    io = dict(inp_res=1 / 128.0, out_res=1 / 512.0, out_noise=0.0, inp_noise=0.0, out_bound=4.0, nm_decay=0.25,
              noise_management=dv.NoiseManagementType.AverageAbsMax)
    meta = make_meta(io_params(bound_management=bm, **io), io_params(**io))
    dev = constant_step(w_max=1.0, w_min=-1.0, w_max_dtod=0.0, w_min_dtod=0.0, construction_seed=1)
    host, orc, _ = build_pair(meta, dev, x_size, d_size, gpu=False)
    w = (rng.integers(-38, 39, (d_size, x_size)) / 64.0).astype(F)
    host.set_weights(torch.from_numpy(w))
    orc.set_weights(w)
    gpu = tiles.CudaAnalogTile(host)
    for batch in (1, 37, 300):
        x = ((rng.integers(-64, 65, (batch, x_size)) / 64.0) * rng.uniform(0.05, 1.0, (batch, 1))).astype(F)
        x = (np.round(x * 64) / 64).astype(F)
        if batch > 2:
            x[1] = 0.0
        assert np.array_equal(gpu.forward(torch.from_numpy(x).cuda()).cpu().numpy(), orc.forward(x)), batch
        if bm != dv.BoundManagementType.NONE:
            assert np.array_equal(gpu.get_bm_rounds(batch).numpy(), orc.bm_rounds(batch))
        d = (rng.integers(-64, 65, (batch, d_size)) / 64.0).astype(F)
        assert np.array_equal(gpu.backward(torch.from_numpy(d).cuda()).cpu().numpy(), orc.backward(d)), batch
    # the running value is part of the extra state: a copy that loads it continues identically
    state = gpu.dump_extra()
    assert "rpu.nm_running_average.bits" in state
    other = tiles.CudaAnalogTile(host)
    other.load_extra(state, True)
    x = (rng.integers(-64, 65, (9, x_size)) / 256.0).astype(F)
    want = orc.forward(x)
    assert np.array_equal(other.forward(torch.from_numpy(x).cuda()).cpu().numpy(), want)
    assert np.array_equal(gpu.forward(torch.from_numpy(x).cuda()).cpu().numpy(), want)
    fresh = tiles.CudaAnalogTile(host)                            # without the state the average starts anew
    assert not np.array_equal(fresh.forward(torch.from_numpy(x).cuda()).cpu().numpy(), want)
    import copy
    twin = copy.deepcopy(gpu)                                     # a copy carries the value
    x2 = (rng.integers(-64, 65, (5, x_size)) / 128.0).astype(F)
    assert np.array_equal(twin.forward(torch.from_numpy(x2).cuda()).cpu().numpy(), orc.forward(x2))
    # a group runs such tiles one after the other: the recurrence goes on from each tile's own running value
    if not tiles.CudaAnalogTile.bind_shared_weights:
        x3 = (rng.integers(-64, 65, (7, x_size)) / 128.0).astype(F)
        gpu.forward(torch.from_numpy(x2).cuda())                   # now both tiles have seen x2 last
        ys = tiles.TileGroup([gpu, twin]).forward([torch.from_numpy(x3).cuda(), torch.from_numpy(x3).cuda()])
        want3 = orc.forward(x3)
        assert np.array_equal(ys[0].cpu().numpy(), want3) and np.array_equal(ys[1].cpu().numpy(), want3)


@pytest.mark.parametrize("noise_type", ["AdditiveConstant", "PCMRead"])
def test_weight_noise_under_bound_management_is_a_function_of_the_seed(gpu_device, noise_type):
    """Output-referred weight noise in the later rounds of bound management: a sample's row in such a round depends on
    the order in which workgroups finished the round before, its draws do not (they are keyed by the sample).  The same
    seed gives the same outputs and round counts, on the same tile and on another one."""
    rng = np.random.default_rng(6)
    x_size, d_size, batch = 64, 48, 256
    x = torch.from_numpy(rng.uniform(-1, 1, (batch, x_size)).astype(F)).cuda()
    io = dict(w_noise=0.02, w_noise_type=getattr(dv.WeightNoiseType, noise_type), out_bound=0.9,
              noise_management=dv.NoiseManagementType.AbsMax, bound_management=dv.BoundManagementType.Iterative)
    got = []
    for _tile in range(2):
        _orc, gpu, _w = pair(x_size, d_size, **io)
        for _call in range(2):
            gpu.set_seed(77)
            got.append((gpu.forward(x).clone(), gpu.get_bm_rounds(batch).clone()))
    assert got[0][1].max() >= 3 and got[0][1].min() < got[0][1].max()      # rows change hands between the rounds
    for y, rounds in got[1:]:
        assert torch.equal(rounds, got[0][1]) and torch.equal(y, got[0][0])
