"""Host-side rules of the argument plumbing, without a GPU: which memory counts as re-tiled weights
(the mark follows the storage through views, `.data`, `.t()` and Parameter wrappers, and dies with
it), which views of such memory an operator refuses, one workspace per (device, stream), and a plan's
refusal to launch on another stream than the one it was built on."""
import gc

import pytest
import torch

from vllm_kunlun_amd import _lib as L
from vllm_kunlun_amd import _plan


def test_tiled_mark_follows_the_storage_not_the_tensor_object():
    w = torch.zeros(3, 32, 128, dtype=torch.int8)
    assert not _plan.is_tiled(w) and _plan.weight_layout(w) == L.KMOE_W_ROWMAJOR
    _plan._mark_tiled(w, 32, 128)          # what tile_int8_weights_ does after re-arranging the bytes
    p = torch.nn.Parameter(w, requires_grad=False)
    for view in (w, w.data, w.detach(), p, p.data, w[1], w.view(1, 3, 32, 128), w[1:], w[0].t().t()):
        assert _plan.is_tiled(view)
        assert _plan.weight_layout(view) == L.KMOE_W_TILED
    assert not _plan.is_tiled(w.clone())   # a copy is other memory (and would hold tiled bytes unmarked: do not copy)
    # views that would read scrambled values are refused, not served as row-major
    for bad in (w[0].t(), w[:, :16], w[:, :, :64], w.view(3, 64, 64), w.view(torch.bfloat16)[..., :32]):
        assert _plan.is_tiled(bad)
        with pytest.raises(ValueError):
            _plan.weight_layout(bad)
    # bf16 weights are tiled on their bytes: k counts bytes
    wb = torch.zeros(2, 16, 32, dtype=torch.bfloat16)
    _plan._mark_tiled(wb, 16, 64)
    assert _plan.weight_layout(wb) == L.KMOE_W_TILED


def test_tiled_mark_dies_with_the_storage():
    w = torch.zeros(16, 64, dtype=torch.int8)
    _plan._mark_tiled(w, 16, 64)
    key = w.untyped_storage()._cdata
    view = w.t()
    del w
    gc.collect()
    assert key in _plan._TILED             # the view keeps the memory, and the mark, alive
    del view
    gc.collect()
    assert key not in _plan._TILED         # a later tensor at the same address does not inherit it


def test_one_workspace_per_device_and_stream():
    ws = _plan._Workspace()
    cpu = torch.device("cpu")
    a = ws.get(100, cpu, stream_id=1)
    assert ws.get(50, cpu, stream_id=1) is a              # grows only
    b = ws.get(100, cpu, stream_id=2)
    assert b.data_ptr() != a.data_ptr()                    # another stream never shares scratch
    big = ws.get(1000, cpu, stream_id=1)
    assert big.numel() >= 1000 and ws.get(10, cpu, stream_id=1) is big


def test_plan_refuses_another_stream(monkeypatch):
    plan = _plan.MoEPlan(args=None, layout=None, workspace=torch.zeros(8, dtype=torch.uint8), keepalive=[],
                         stream_id=0x10)
    monkeypatch.setattr(_plan, "_current_stream_id", lambda device: 0x20)
    with pytest.raises(RuntimeError, match="built on stream 0x10"):
        plan()
