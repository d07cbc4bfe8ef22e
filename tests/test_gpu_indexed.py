"""GPU parity of the indexed (convolution) interface against the indexed oracle, and against torch's convolution
for a perfect tile."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from aihwkit_amd.rpu_base import devices as dv
from aihwkit_amd.rpu_base import tiles
from helpers import build_pair, constant_step, make_meta, noise_free_io, soft_bounds
from indexed_oracle import IndexedOracle
from test_oracle_indexed_pins import conv_indices

pytestmark = pytest.mark.gpu


def cuda(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def test_perfect_tile_is_a_convolution(gpu_device):
    rng = np.random.default_rng(0)
    c_in, c_out, height, width, n, kernel = 16, 32, 12, 12, 8, (5, 5)      # the second LeNet convolution
    indices, patches = conv_indices((c_in, height, width), kernel, (1, 1), (0, 0), (1, 1), True)
    x_size = c_in * 25 + 1
    meta = dv.FloatingPointTileParameter()
    host = meta.create_array(x_size, c_out)
    w = rng.normal(0, 0.1, (c_out, x_size)).astype(np.float32)
    host.set_weights(torch.from_numpy(w))
    gpu = tiles.CudaFloatingPointTile(host)
    assert not gpu.has_matrix_indices()
    with pytest.raises(RuntimeError):
        gpu.forward_indexed(torch.zeros(n, c_in, height, width).cuda(), torch.zeros(n, c_out, 8, 8).cuda())
    gpu.set_matrix_indices(indices)
    assert gpu.has_matrix_indices()
    x = rng.normal(0, 1, (n, c_in, height, width)).astype(np.float32)
    y = gpu.forward_indexed(cuda(x), torch.empty(n, c_out, 8, 8).cuda()).cpu()
    weight = torch.from_numpy(w[:, :-1].reshape(c_out, c_in, 5, 5).copy())
    want = F.conv2d(torch.from_numpy(x), weight, torch.from_numpy(w[:, -1].copy()))
    assert torch.allclose(y, want, atol=1e-4)
    grad = rng.normal(0, 1, (n, c_out, 8, 8)).astype(np.float32)
    dx = gpu.backward_indexed(cuda(grad), torch.empty(n, c_in, height, width).cuda()).cpu()
    want_dx = F.conv_transpose2d(torch.from_numpy(grad), weight)
    assert torch.allclose(dx, want_dx, atol=1e-4)
    gpu.set_learning_rate(0.01)
    gpu.update_indexed(cuda(x), cuda(grad))
    xt = torch.from_numpy(x).requires_grad_(False)
    wg = weight.clone().requires_grad_(True)
    bg = torch.from_numpy(w[:, -1].copy()).requires_grad_(True)
    (F.conv2d(xt, wg, bg) * torch.from_numpy(grad)).sum().backward()
    want_w = w.copy()
    want_w[:, :-1] -= 0.01 * wg.grad.numpy().reshape(c_out, -1)
    want_w[:, -1] -= 0.01 * bg.grad.numpy()
    assert np.abs(gpu.get_weights().numpy() - want_w).max() <= 2e-4


@pytest.mark.parametrize("kernel,stride,padding", [((3, 3), (1, 1), (1, 1)), ((5, 5), (2, 2), (0, 0))])
def test_analog_tile_matches_the_indexed_oracle(gpu_device, kernel, stride, padding):
    rng = np.random.default_rng(1)
    c_in, c_out, height, width, n = 3, 20, 11, 10, 5
    indices, patches = conv_indices((c_in, height, width), kernel, stride, padding, (1, 1), True)
    x_size = c_in * kernel[0] * kernel[1] + 1
    f_io = noise_free_io(noise_management=dv.NoiseManagementType.AbsMax, bound_management=dv.BoundManagementType.Iterative)
    b_io = noise_free_io(noise_management=dv.NoiseManagementType.AbsMax)
    meta = make_meta(f_io, b_io, pulse_type=dv.PulseType.DeterministicImplicit, desired_bl=31)
    dev = constant_step(dw_min=0.002, dw_min_std=0.0, construction_seed=4)
    host, orc_tile, gpu = build_pair(meta, dev, x_size, c_out)
    w = rng.normal(0, 0.2, (c_out, x_size)).astype(np.float32)
    gpu.set_weights(torch.from_numpy(w))
    orc_tile.set_weights(w)
    gpu.set_matrix_indices(indices)
    twin = tiles.CudaAnalogTile(host)                       # a copy made before the indices were set has none
    assert not twin.has_matrix_indices()
    orc = IndexedOracle(orc_tile, indices.numpy(), patches)
    x = rng.normal(0, 1, (n, c_in, height, width)).astype(np.float32)
    out_hw = (int(np.sqrt(patches)), patches // int(np.sqrt(patches))) if int(np.sqrt(patches)) ** 2 == patches else (1, patches)
    y = gpu.forward_indexed(cuda(x), torch.empty(n, c_out, *out_hw).cuda()).cpu().numpy().reshape(n, c_out, patches)
    want = orc.forward(x)
    off = np.abs(y - want) > 1e-5
    assert off.mean() < 0.005 and np.abs(y - want).max() < 0.2      # an ADC code may flip at a rounding edge
    grad = (0.3 * rng.normal(0, 1, (n, c_out, patches))).astype(np.float32)
    dx = gpu.backward_indexed(cuda(grad.reshape(n, c_out, *out_hw)), torch.empty(n, c_in, height, width).cuda())
    want_dx = orc.backward(grad, c_in * height * width)
    diff = np.abs(dx.cpu().numpy().reshape(n, -1) - want_dx)
    assert (diff > 1e-4).mean() < 0.01 and diff.max() < 0.5
    gpu.set_learning_rate(0.05)
    orc_tile.set_learning_rate(0.05)
    gpu.update_indexed(cuda(x), cuda(grad.reshape(n, c_out, *out_hw)))
    orc.update(x, grad)
    assert np.abs(gpu.get_weights().numpy() - orc_tile.get_weights()).max() <= 1e-5
    assert np.abs(orc_tile.get_weights() - np.clip(w, orc_tile.get_hidden()[1], orc_tile.get_hidden()[0])).max() > 1e-3


@pytest.mark.parametrize("c_in", [2, 8])          # patch rows of 19 (one contraction step) and 73 elements (three)
def test_fused_convolution_forward_is_bit_exact_with_bound_management_rounds(gpu_device, c_in):
    """Exact arithmetic (power-of-two DAC step, weights on a 1/64 grid) with weights large enough to saturate the ADC:
    outputs and rounds per patch of the fused kernel must equal the oracle's to the last bit."""
    rng = np.random.default_rng(2)
    c_out, height, width, n = 20, 9, 8, 13
    indices, patches = conv_indices((c_in, height, width), (3, 3), (1, 1), (1, 1), (1, 1), True)
    x_size = c_in * 9 + 1
    f_io = noise_free_io(inp_res=1 / 128.0, out_res=1 / 512.0, out_bound=4.0, noise_management=dv.NoiseManagementType.AbsMax,
                         bound_management=dv.BoundManagementType.Iterative)
    meta = make_meta(f_io, noise_free_io())
    dev = constant_step(w_max_dtod=0.0, w_min_dtod=0.0, w_max=1.0, w_min=-1.0, construction_seed=3)
    host, orc_tile, _ = build_pair(meta, dev, x_size, c_out, gpu=False)
    w = (rng.integers(-60, 61, (c_out, x_size)) / 64.0).astype(np.float32)
    host.set_weights(torch.from_numpy(w))
    orc_tile.set_weights(w)
    gpu = tiles.CudaAnalogTile(host)
    gpu.set_matrix_indices(indices)
    x = rng.uniform(-1, 1, (n, c_in, height, width)).astype(np.float32)
    x[0] = 0.0                                                          # patches of zeros: the zero short-cut
    y = gpu.forward_indexed(cuda(x), torch.empty(n, c_out, height, width).cuda()).cpu().numpy().reshape(n, c_out, patches)
    want = IndexedOracle(orc_tile, indices.numpy(), patches).forward(x)
    assert np.array_equal(y, want)
    rounds = orc_tile.bm_rounds(n * patches)
    assert rounds.max() > 1 and rounds.min() >= 1
    assert np.array_equal(gpu.get_bm_rounds(n * patches).numpy(), rounds)


@pytest.mark.parametrize("c_in,kernel", [(3, 3), (16, 5)])       # the per-wave kernel and the one that splits long rows
def test_zero_patches_beside_others_without_a_bias_column(gpu_device, c_in, kernel):
    """Without a bias column a patch of zeros short-cuts to zero outputs (its noise-management scale is zero); the
    other patches of the same 32-patch tile must not notice."""
    rng = np.random.default_rng(8)
    c_out, height, width, n = 20, 9, 10, 3
    indices, patches = conv_indices((c_in, height, width), (kernel, kernel), (1, 1), (0, 0), (1, 1), False)
    x_size = c_in * kernel * kernel
    f_io = noise_free_io(inp_res=1 / 128.0, out_res=1 / 512.0, out_bound=4.0, noise_management=dv.NoiseManagementType.AbsMax,
                         bound_management=dv.BoundManagementType.Iterative)
    meta = make_meta(f_io, noise_free_io())
    dev = constant_step(w_max_dtod=0.0, w_min_dtod=0.0, w_max=1.0, w_min=-1.0, construction_seed=3)
    host, orc_tile, _ = build_pair(meta, dev, x_size, c_out, gpu=False)
    w = (rng.integers(-60, 61, (c_out, x_size)) / 64.0).astype(np.float32)
    host.set_weights(torch.from_numpy(w))
    orc_tile.set_weights(w)
    gpu = tiles.CudaAnalogTile(host)
    gpu.set_matrix_indices(indices)
    x = (rng.integers(-64, 65, (n, c_in, height, width)) / 64.0).astype(np.float32)
    x[0, :, :, : width // 2 + 1] = 0.0                              # zero and non-zero patches alternate along a row
    x[2] = 0.0
    y = gpu.forward_indexed(cuda(x), torch.empty(n, c_out, 1, patches).cuda()).cpu().numpy().reshape(n, c_out, patches)
    want = IndexedOracle(orc_tile, indices.numpy(), patches).forward(x)
    rounds = orc_tile.bm_rounds(n * patches)
    assert (rounds == 0).sum() >= patches and (rounds[:patches] == 0).any() and (rounds[:patches] > 0).any()
    assert np.array_equal(y, want)
    assert np.array_equal(gpu.get_bm_rounds(n * patches).numpy(), rounds)


@pytest.mark.parametrize("c_in,kernel", [(2, 3), (5, 3), (16, 5)])   # patch rows of 19, 46 and 401 elements: the three kernels
@pytest.mark.parametrize("stochastic", [False, True])
def test_fused_convolution_forward_draws_what_the_unfolded_pass_draws(gpu_device, c_in, kernel, stochastic):
    """The fused convolution kernels key their random draws by (patch row element, patch number) like the ordinary
    forward pass on the unfolded patch matrix: with output noise, and with DAC / ADC stochastic rounding and input noise
    (the kernel variants that compile those draws in), a tile gives on the images what a twin with the same seed gives on
    the explicitly unfolded matrix -- up to the summation order of the contraction, which can move a value across one ADC
    rounding edge."""
    from indexed_oracle import copy_indexed_input
    from helpers import io_params, soft_bounds
    rng = np.random.default_rng(31 + c_in)
    c_out, height, width, n = 24, 10, 9, 7
    indices, patches = conv_indices((c_in, height, width), (kernel, kernel), (1, 1), (1, 1), (1, 1), True)
    x_size = c_in * kernel * kernel + 1
    out_res, out_bound = 1 / 4096.0, 16.0
    io = io_params(inp_res=1 / 256.0, out_res=out_res, out_bound=out_bound, out_noise=0.05,
                   inp_noise=0.01 if stochastic else 0.0, inp_sto_round=stochastic, out_sto_round=stochastic,
                   noise_management=dv.NoiseManagementType.AbsMax, bound_management=dv.BoundManagementType.Iterative)
    meta = make_meta(io, noise_free_io())
    host, _orc, _ = build_pair(meta, soft_bounds(construction_seed=4), x_size, c_out, gpu=False)
    host.set_weights(torch.from_numpy(rng.uniform(-0.3, 0.3, (c_out, x_size)).astype(np.float32)))
    conv, plain = tiles.CudaAnalogTile(host), tiles.CudaAnalogTile(host)
    conv.set_matrix_indices(indices)
    x = rng.uniform(-1, 1, (n, c_in, height, width)).astype(np.float32)
    x[1] = 0.0
    unfolded = copy_indexed_input(x.reshape(n, -1), indices.numpy().reshape(-1).astype(np.int64), x_size, patches)  # [X, N P]
    for call in range(2):
        conv.set_seed(900 + call)
        plain.set_seed(900 + call)
        y = conv.forward_indexed(cuda(x), torch.empty(n, c_out, 1, patches).cuda()).cpu().numpy().reshape(n, c_out, patches)
        y_rows = plain.forward(cuda(unfolded.T)).cpu().numpy()                                  # [N P, D]
        want = y_rows.reshape(n, patches, c_out).transpose(0, 2, 1)
        assert np.array_equal(conv.get_bm_rounds(n * patches).numpy(), plain.get_bm_rounds(n * patches).numpy())
        diff = np.abs(y - want)
        # one ADC step (the range 2 out_bound in 1 / out_res steps) in output units: the abs-max scale of a patch is below
        # 1.2, and each further round doubles it
        rounds = plain.get_bm_rounds(n * patches).numpy().reshape(n, 1, patches)
        step = 2 * out_res * out_bound * 1.2 * np.exp2(np.maximum(rounds, 1) - 1)
        assert (diff <= step * 1.01).all()
        assert (diff > 1e-5).mean() < 0.002
        assert np.abs(want).max() > 0.5


def test_indexed_backward_adds_overlapping_patches_in_a_fixed_order(gpu_device):
    """Input gradients of overlapping patches are summed per image element in a fixed order (no atomics): repeated calls
    give the same bits, and a perfect tile on values of a binary grid, where no rounding happens, is exact."""
    rng = np.random.default_rng(4)
    c_in, c_out, height, width, n = 6, 40, 11, 10, 9
    indices, patches = conv_indices((c_in, height, width), (3, 3), (1, 1), (1, 1), (1, 1), True)
    x_size = c_in * 9 + 1
    host = dv.FloatingPointTileParameter().create_array(x_size, c_out)
    w = rng.normal(0, 0.1, (c_out, x_size)).astype(np.float32)
    host.set_weights(torch.from_numpy(w))
    gpu = tiles.CudaFloatingPointTile(host)
    gpu.set_matrix_indices(indices)
    grad = rng.normal(0, 1, (n, c_out, height, width)).astype(np.float32)
    runs = [gpu.backward_indexed(cuda(grad), torch.empty(n, c_in, height, width).cuda()).clone() for _ in range(3)]
    assert torch.equal(runs[0], runs[1]) and torch.equal(runs[0], runs[2])
    weight = torch.from_numpy(w[:, :-1].reshape(c_out, c_in, 3, 3).copy())
    assert torch.allclose(runs[0].cpu(), F.conv_transpose2d(torch.from_numpy(grad), weight, padding=1), atol=1e-4)
    # exact arithmetic: integers / 8 times integers / 8, sums far below 2^24 / 64
    w_grid = (rng.integers(-8, 9, (c_out, x_size)) / 8.0).astype(np.float32)
    g_grid = (rng.integers(-8, 9, (n, c_out, height, width)) / 8.0).astype(np.float32)
    gpu.set_weights(torch.from_numpy(w_grid))
    got = gpu.backward_indexed(cuda(g_grid), torch.empty(n, c_in, height, width).cuda()).cpu()
    want = F.conv_transpose2d(torch.from_numpy(g_grid).double(),
                              torch.from_numpy(w_grid[:, :-1].reshape(c_out, c_in, 3, 3).copy()).double(), padding=1)
    assert torch.equal(got.double(), want)


@pytest.mark.parametrize("c_in,side,n,c_out,bm,nm", [
    (16, 16, 8, 40, True, "AbsMax"),     # 2048 patches of 145 elements: patches gathered by the init kernels, 32 x 32 tiles
    (16, 16, 8, 40, True, "Max"),        # ... with the other noise managements of the gathering kernels
    (16, 16, 8, 40, True, "Constant"),
    (16, 16, 8, 136, True, "AbsMax"),    # rows quantized ahead: the patch matrix is written; large tiles in both directions
    (16, 16, 8, 136, False, "AbsMax"),   # a single round: gathered patches on the wide tile too, large tiles in both directions
    (3, 64, 5, 40, True, "AbsMax"),      # 20480 patches of 28 elements: gathered patches and large tiles with idle outputs
    (3, 64, 5, 40, True, "Max"),
    (3, 64, 5, 40, True, "Constant"),
    (8, 48, 8, 40, True, "AbsMax"),      # 18432 patches of 73 elements: the same with rows of two blocks of the gathering kernel
])
def test_wide_convolution_on_many_patches_equals_the_pass_over_the_unfolded_images(gpu_device, c_in, side, n, c_out, bm, nm):
    """Forward and backward of convolutions too wide for the fused kernel: same bits as the pass over the patch matrix
    that torch unfolds (the samples that saturate the ADC go through further rounds either way), and the fold of that
    pass's input gradients."""
    rng = np.random.default_rng(12)
    indices, patches = conv_indices((c_in, side, side), (3, 3), (1, 1), (1, 1), (1, 1), True)
    x_size = c_in * 9 + 1
    f_io = noise_free_io(inp_res=1 / 128.0, out_res=1 / 512.0, out_bound=2.0, noise_management=getattr(dv.NoiseManagementType, nm),
                         nm_thres=3.0 if nm == "Constant" else 0.0,
                         bound_management=dv.BoundManagementType.Iterative if bm else dv.BoundManagementType.NONE)
    b_io = noise_free_io(inp_res=1 / 128.0, out_res=1 / 512.0, noise_management=dv.NoiseManagementType.AbsMax)
    dev = constant_step(dw_min=0.002, dw_min_std=0.0, construction_seed=4, w_max_dtod=0.0, w_min_dtod=0.0, w_max=1.0, w_min=-1.0)
    _host, _orc, gpu = build_pair(make_meta(f_io, b_io), dev, x_size, c_out)
    gpu.set_weights(torch.from_numpy(rng.normal(0, 0.25, (c_out, x_size)).astype(np.float32)))
    gpu.set_matrix_indices(indices)
    x = torch.from_numpy(rng.normal(0, 1, (n, c_in, side, side)).astype(np.float32)).cuda()
    y = gpu.forward_indexed(x, torch.empty(n, c_out, side, side).cuda())
    if bm:
        rounds = gpu.get_bm_rounds(n * patches)
        assert rounds.max() > 1 and (rounds == 1).any()              # some patches saturate the ADC, others do not
    unfolded = torch.cat([F.unfold(x, 3, padding=1), torch.ones(n, 1, patches).cuda()], dim=1)      # [n, x_size, patches]
    x_mat = unfolded.permute(0, 2, 1).reshape(n * patches, x_size).contiguous()
    y_mat = gpu.forward(x_mat)
    assert torch.equal(y, y_mat.reshape(n, patches, c_out).permute(0, 2, 1).reshape(n, c_out, side, side))
    grad = torch.from_numpy((0.3 * rng.normal(0, 1, (n, c_out, side, side))).astype(np.float32)).cuda()
    dx = gpu.backward_indexed(grad, torch.empty(n, c_in, side, side).cuda())
    d_mat = grad.reshape(n, c_out, patches).permute(0, 2, 1).reshape(n * patches, c_out).contiguous()
    back = gpu.backward(d_mat).reshape(n, patches, x_size)[:, :, :-1].permute(0, 2, 1)                # bias column dropped
    want = F.fold(back.double(), (side, side), 3, padding=1)
    assert (dx.double() - want).abs().max() <= 1e-5 * want.abs().max()
    assert dx.abs().max() > 0.1


@pytest.mark.parametrize("mode", [2, -1, 3])
def test_gathered_forward_runs_every_round_whatever_the_launch_mode(gpu_device, mode):
    """A wide convolution whose patches are gathered by the init kernels (2048 patches, 40 outputs: few enough workgroups
    for the launch that merges the later rounds): two calls in a row, quiet inputs and then saturating ones, give the
    outputs and round counts of the separate launches (mode 0) in every launch mode."""
    rng = np.random.default_rng(21)
    c_in, side, n, c_out = 16, 16, 8, 40
    indices, patches = conv_indices((c_in, side, side), (3, 3), (1, 1), (1, 1), (1, 1), True)
    x_size = c_in * 9 + 1
    f_io = noise_free_io(inp_res=1 / 128.0, out_res=1 / 512.0, out_bound=1.0, noise_management=dv.NoiseManagementType.AbsMax,
                         bound_management=dv.BoundManagementType.Iterative)
    dev = constant_step(dw_min=0.002, dw_min_std=0.0, construction_seed=4, w_max_dtod=0.0, w_min_dtod=0.0, w_max=1.0, w_min=-1.0)
    w = torch.from_numpy(rng.normal(0, 0.25, (c_out, x_size)).astype(np.float32))
    quiet = torch.from_numpy(rng.normal(0, 1, (n, c_in, side, side)).astype(np.float32)).cuda()
    loud = quiet.clone()
    quiet_w = w * 0.02          # no patch saturates the ADC with these weights
    results = {}
    for m in (0, mode):
        _host, _orc, gpu = build_pair(make_meta(f_io, noise_free_io()), dev, x_size, c_out)
        gpu.set_matrix_indices(indices)
        gpu.set_fused_rounds(m)
        out = []
        for weights, x in ((quiet_w, quiet), (quiet_w, quiet), (w, loud), (w, loud)):
            gpu.set_weights(weights)
            y = gpu.forward_indexed(x, torch.empty(n, c_out, side, side).cuda())
            out.append((y.clone(), gpu.get_bm_rounds(n * patches).clone()))
        results[m] = out
    assert results[0][0][1].max() == 1                       # the quiet calls stop after one round
    assert results[0][2][1].max() >= 3                       # the loud ones need at least two further rounds
    for (y0, r0), (y1, r1) in zip(results[0], results[mode]):
        assert torch.equal(r0, r1)
        assert torch.equal(y0, y1)


@pytest.mark.parametrize("case", [
    # 110 patches per image, 28 elements per patch with zero padding and a bias entry, 20 outputs (one block of 16 and a
    # tail), ConstantStep with update-BL management: short bit lines
    dict(c_in=3, hw=(11, 10), kernel=(3, 3), stride=(1, 1), padding=(1, 1), n=5, c_out=20, device="constant", bl=31,
         pulse="StochasticCompressed"),
    # 196 patches of 73 elements, 40 outputs, SoftBounds with cycle-to-cycle noise
    dict(c_in=8, hw=(14, 14), kernel=(3, 3), stride=(1, 1), padding=(1, 1), n=3, c_out=40, device="soft", bl=31,
         pulse="StochasticCompressed"),
    # 9 patches per image (a block of 64 samples spans seven images), bit lines of 80 pulses: three rows of words per sample
    dict(c_in=2, hw=(9, 9), kernel=(5, 5), stride=(2, 2), padding=(0, 0), n=23, c_out=33, device="constant", bl=80,
         pulse="StochasticCompressed"),
    dict(c_in=3, hw=(11, 10), kernel=(3, 3), stride=(1, 1), padding=(1, 1), n=5, c_out=20, device="constant", bl=31,
         pulse="DeterministicImplicit"),
    # 4800 samples: the per-sample maxima come from the kernel with one thread per sample
    dict(c_in=3, hw=(40, 40), kernel=(3, 3), stride=(1, 1), padding=(1, 1), n=3, c_out=20, device="soft", bl=31,
         pulse="StochasticCompressed"),
])
def test_pulsed_update_reads_patches_and_gradients_in_place(gpu_device, case):
    """update_indexed of a pulsed tile reads the images through the index matrix and the gradient tensor where the caller
    keeps it; neither the patch matrix nor a patch-major copy of the gradients is made.  Same weights, bit for bit, as
    update() of a twin tile on the patch matrix that torch unfolds and the patch-major gradients."""
    rng = np.random.default_rng(31)
    c_in, (height, width), kernel, n, c_out = case["c_in"], case["hw"], case["kernel"], case["n"], case["c_out"]
    indices, patches = conv_indices((c_in, height, width), kernel, case["stride"], case["padding"], (1, 1), True)
    x_size = c_in * kernel[0] * kernel[1] + 1
    meta = make_meta(noise_free_io(), noise_free_io(), pulse_type=getattr(dv.PulseType, case["pulse"]), desired_bl=case["bl"],
                     update_bl_management=case["bl"] == 31, update_management=True)
    if case["device"] == "soft":
        dev = soft_bounds(dw_min=0.002, dw_min_std=0.3, construction_seed=9)
    else:
        dev = constant_step(dw_min=0.002, dw_min_std=0.0, construction_seed=4)
    w = torch.from_numpy(rng.normal(0, 0.2, (c_out, x_size)).astype(np.float32))
    x = torch.from_numpy(rng.normal(0, 1, (n, c_in, height, width)).astype(np.float32)).cuda()
    grad = torch.from_numpy((0.3 * rng.normal(0, 1, (n, c_out, patches))).astype(np.float32)).cuda()
    unfolded = torch.cat([F.unfold(x, kernel, padding=case["padding"], stride=case["stride"]), torch.ones(n, 1, patches).cuda()], dim=1)
    x_mat = unfolded.permute(0, 2, 1).reshape(n * patches, x_size).contiguous()
    d_mat = grad.permute(0, 2, 1).reshape(n * patches, c_out).contiguous()
    got = []
    for in_place in (True, False):
        _host, _orc, gpu = build_pair(meta, dev, x_size, c_out)
        gpu.set_weights(w)
        gpu.set_learning_rate(0.05)
        gpu.set_matrix_indices(indices)
        for _ in range(2):
            if in_place:
                gpu.update_indexed(x, grad)
            else:
                gpu.update(x_mat, d_mat, False)
        got.append(gpu.get_weights().clone())
    assert torch.equal(got[0], got[1])
    assert (got[0] - torch.from_numpy(np.clip(w.numpy(), -0.6, 0.6))).abs().max() > 1e-3
