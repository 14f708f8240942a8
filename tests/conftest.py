"""Test set-up: import paths, the `gpu` marker, helpers shared by the suites."""
import os
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "vllm-kunlun_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def bits(t: torch.Tensor) -> np.ndarray:
    """bf16 tensor -> uint16 bit patterns (numpy, on the host)."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def from_bits(b: np.ndarray) -> torch.Tensor:
    """uint16 bit patterns -> bf16 tensor."""
    return torch.from_numpy(np.ascontiguousarray(b).view(np.int16)).view(torch.bfloat16)


def rel_l2(a: torch.Tensor, b: torch.Tensor) -> float:
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))


def fetch_silu_table(f16: bool) -> np.ndarray:
    """The product's SiLU of all 65536 activation patterns of one type (kmoe_silu_table)."""
    from vllm_kunlun_amd import _lib as L
    table = torch.empty(65536, dtype=torch.float32, device="cuda")
    L.check(L.lib.kmoe_silu_table(L.ptr(table), L.KMOE_DT_F16 if f16 else L.KMOE_DT_BF16, L.stream()))
    torch.cuda.synchronize()
    return table.cpu().numpy()


@pytest.fixture(scope="session", autouse=True)
def device_silu():
    """On a GPU box the oracle follows the device's SiLU (oracle/c_oracle.py::install_device_silu); without a GPU it keeps its own
    closed form, which is what the CPU tests and the golden fixtures use."""
    if torch.cuda.is_available():
        from oracle import c_oracle as co
        co.install_device_silu(fetch_silu_table)
    yield
