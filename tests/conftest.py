import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    # A GPU test on a machine without a GPU is an error of the invocation, not a pass:
    # skip loudly so `-m "not gpu"` is the CPU suite and `-m gpu` the device suite.
    try:
        import torch
        has_gpu = torch.cuda.is_available()
    except Exception:
        has_gpu = False
    if has_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def mie_lib():
    from maskedincrementeval_amd import _lib
    return _lib.lib()


@pytest.fixture(autouse=True)
def _f32_matmul_mode(request):
    """Tests parametrized over `f32mode` run with ops.f32_matmul set to it: "bf16x3" (fp32 deltas multiplied as three
    bf16 terms on the bf16 matrix-core instruction, the default) or "native" (the fp32 instruction)."""
    spec = getattr(request.node, "callspec", None)
    mode = spec.params.get("f32mode") if spec is not None else None
    if mode is None:
        yield
        return
    from maskedincrementeval_amd import ops
    old = ops.f32_matmul
    ops.f32_matmul = mode
    yield
    ops.f32_matmul = old
