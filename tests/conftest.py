import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a ROCm GPU (MI355X); run with -m gpu")
    config.addinivalue_line("markers", "routing(*modes): decode routing modes the test runs under "
                                       "(\"balanced\", \"library\")")


@pytest.fixture(scope="session")
def device():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


# Automatic decode calls (partition_size 0) are routed by size: small calls take the grid schedule,
# large ones the balanced schedule.  Test shapes are small, so the routing threshold decides which
# kernels a test reaches.  "balanced" sets it to 0 (every supported shape on the balanced schedule),
# "library" leaves the library's default (what a small deployment gets).  Modules whose tests run
# decode steps through sessions, graphs or the fused append run under both; a test can narrow that
# with @pytest.mark.routing("balanced") or ("library").
LIBRARY_DEFAULT_SMALL_DECODE_TOKENS = 32768
BOTH_ROUTINGS = {"test_gpu_adapter", "test_gpu_generation", "test_gpu_block_manager", "test_gpu_graph",
                 "test_gpu_fp16", "test_gpu_decode", "test_gpu_fp8_bound", "test_zz_no_alloc"}


def pytest_generate_tests(metafunc):
    if "decode_routing" not in metafunc.fixturenames:
        return
    marker = metafunc.definition.get_closest_marker("routing")
    if marker is not None:
        modes = list(marker.args)
    elif metafunc.module.__name__.rsplit(".", 1)[-1] in BOTH_ROUTINGS:
        modes = ["balanced", "library"]
    else:
        return                                   # one run, threshold 0 (the fixture's default)
    metafunc.parametrize("decode_routing", modes, indirect=True)


@pytest.fixture(autouse=True)
def decode_routing(request):
    mode = getattr(request, "param", "balanced")
    from aicomp_amd import _lib, ops
    try:
        prev = ops.set_small_decode_tokens(0 if mode == "balanced" else LIBRARY_DEFAULT_SMALL_DECODE_TOKENS)
    except _lib.LibraryMissing:                  # oracle-only tests do not need the library
        yield mode
        return
    yield mode
    ops.set_small_decode_tokens(prev)


@pytest.fixture(params=["fast", "torch_op", "ctypes"])
def host_route(request, monkeypatch):
    """The host routes of the drop-in operator's decode step into the HIP library: the CPython
    function over a per-layer handle (aicomp_amd._aicomp_fast), the registered PyTorch operator
    (torch.ops.mi355_kv.decode_step) and the ctypes binding."""
    from aicomp_amd import kv_cache as akv
    if request.param == "fast":
        assert akv._FAST is not None, "aicomp_amd/_aicomp_fast is not built"
    elif request.param == "torch_op":
        assert akv._TORCH_DECODE is not None, "libaicomp_kv_torch.so is not built"
    monkeypatch.setattr(akv, "_route", request.param)
    return request.param
