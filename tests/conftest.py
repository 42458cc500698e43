import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "nnlib.jl_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _gpu_available():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _gpu_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this container")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as O
    O.lib()
    return O


@pytest.fixture(scope="session")
def nn():
    """The product package with the HIP library loaded; fails loudly when it is not built."""
    import nnlib_amd
    nnlib_amd._lib.load()
    if _gpu_available():
        nnlib_amd._lib.check(nnlib_amd._lib.load().mi_init(0))
    return nnlib_amd


@pytest.fixture(autouse=True)
def _stale_device_state(request):
    """Before every GPU test: NaN-filled device blocks of many sizes, written and freed.  The arrays the test then
    allocates start out as NaN instead of whatever the box happened to hold, and the SIMDs' register files hold NaN
    patterns from the fill kernel: a kernel that reads memory or a register it never wrote (one did, through a
    compiler's partial reload of a spilled operand) then fails every time instead of from run to run."""
    if "gpu" in request.keywords and _gpu_available():
        import torch
        blocks = [torch.full((n,), float("nan"), device="cuda") for n in (1 << 10, 1 << 14, 1 << 18, 1 << 22, 1 << 25) for _ in range(2)]
        torch.cuda.synchronize()
        del blocks
    yield


def bf16_round(a):
    """float32 -> nearest-even bfloat16, returned as float32 (pure numpy bit arithmetic)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    u = a.view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    out = r.astype(np.uint32).view(np.float32).reshape(a.shape)
    return np.where(np.isnan(a), a, out)


def round_to(a, dtype):
    """Values of ``a`` after a round trip through the named storage type, as float32."""
    a = np.asarray(a, dtype=np.float32)
    if dtype == "f32":
        return a
    if dtype == "f16":
        return a.astype(np.float16).astype(np.float32)
    return bf16_round(a)


def rel_err(x, ref):
    """max |x - ref| / max |ref|: the parity metric (error against output scale)."""
    x, ref = np.asarray(x, dtype=np.float64), np.asarray(ref, dtype=np.float64)
    return float(np.max(np.abs(x - ref)) / max(np.max(np.abs(ref)), 1e-30))
