import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "oracle"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP GPU (run on the MI355X box)")


@pytest.fixture(scope="session")
def gpu_device():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda", 0)


# GPU suites that run twice: on tiles that own their row-major weight matrix and on tiles bound to an [x_size, d_size]
# shared tensor, as the reference's Python binds every CUDA tile (the library then works on that layout in place)
BOTH_STORAGES = ("test_gpu_parity", "test_gpu_statistics", "test_gpu_benchmark_configs", "test_gpu_fused_rounds",
                 "test_gpu_group_update", "test_gpu_inference", "test_gpu_indexed", "test_gpu_long_batches",
                 "test_gpu_state", "test_gpu_hwa", "test_zz_no_alloc")


def pytest_generate_tests(metafunc):
    if "storage_mode" in metafunc.fixturenames:
        module = metafunc.module.__name__.split(".")[-1]
        modes = ["row_major", "xd_shared"] if module in BOTH_STORAGES else ["row_major"]
        # RPU_TEST_STORAGE=xd_shared runs every module on bound tiles only (the sweeps too: a longer, occasional run)
        if os.environ.get("RPU_TEST_STORAGE") in ("row_major", "xd_shared"):
            modes = [os.environ["RPU_TEST_STORAGE"]]
        metafunc.parametrize("storage_mode", modes, indirect=True)


@pytest.fixture(autouse=True)
def storage_mode(request):
    mode = getattr(request, "param", "row_major")
    if mode == "row_major":
        yield mode
        return
    from aihwkit_amd.rpu_base import tiles
    tiles.CudaAnalogTile.bind_shared_weights = True
    try:
        yield mode
    finally:
        tiles.CudaAnalogTile.bind_shared_weights = False
