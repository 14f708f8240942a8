"""kmoe_moe_forward_static, the entry point that takes no workspace and allocates nothing
(its intermediates live in a 64 MiB buffer inside the library's device image), against
kmoe_moe_forward on the same arguments: bit-identical outputs, on two calls in a row, the
second on a smaller batch (the buffer then still holds the first call's intermediates), and
also against the C oracle. Called through the C ABI (ctypes), not through the plugin."""
import ctypes as C
import gc

import numpy as np
import pytest
import torch

from conftest import bits

pytestmark = pytest.mark.gpu


def _plan_for(sl, out):
    from vllm_kunlun_amd import _lib as L
    from vllm_kunlun_amd._plan import make_moe_plan
    s, lay = sl.shape, sl.layer
    return make_moe_plan(L.KMOE_FMT_INT8, sl.x.contiguous(), sl.logits.contiguous(), out, s.K, lay.w13_weight,
                         lay.w2_weight, lay.w13_weight_scale, lay.w2_weight_scale, s.scoring, True, s.n_group,
                         s.topk_group, s.routed_scale, sl.bias, sl.shared, 1.0)


def _device_free_bytes():
    """Free device memory as the driver sees it (hipMemGetInfo): it drops for ANY allocation on the
    GPU, also one made inside libkmoe.so, which torch's allocator statistics cannot see."""
    return torch.cuda.mem_get_info()[0]


def _both_ways(sl):
    """(output of kmoe_moe_forward, output of kmoe_moe_forward_static) for one synthetic layer.
    Around the static call nothing may be allocated: the driver's free-byte count must not drop
    and torch's allocator must not have been asked for a block. Python's cyclic collector is
    switched off for the window (garbage of earlier tests freed inside it would move the figures)."""
    from vllm_kunlun_amd import _lib as L
    want = torch.empty_like(sl.x)
    plan = _plan_for(sl, want)
    assert plan.layout.total_bytes <= L.STATIC_WORKSPACE_BYTES
    plan()
    got = torch.full_like(sl.x, float("nan"))
    plan.args.out = got.data_ptr()
    stream = L.stream()
    # warm-up: the first call on a GPU resolves the buffer's device address (not part of the claim)
    L.check(L.lib.kmoe_moe_forward_static(C.byref(plan.args), stream))
    torch.cuda.synchronize()
    got.fill_(float("nan"))
    torch.cuda.synchronize()
    gc.collect()
    gc.disable()
    try:
        free_before = _device_free_bytes()
        blocks_before = torch.cuda.memory_stats()["allocation.all.allocated"]
        segments_before = torch.cuda.memory_stats()["segment.all.allocated"]
        rc = L.lib.kmoe_moe_forward_static(C.byref(plan.args), stream)
        torch.cuda.synchronize()
        free_after = _device_free_bytes()
        blocks_after = torch.cuda.memory_stats()["allocation.all.allocated"]
        segments_after = torch.cuda.memory_stats()["segment.all.allocated"]
    finally:
        gc.enable()
    L.check(rc)
    assert free_after >= free_before, f"device memory shrank by {free_before - free_after} B across the static call"
    assert blocks_after == blocks_before and segments_after == segments_before, "torch allocated during the static call"
    return want, got


def test_static_workspace_forward_matches_the_workspace_entry_point_twice():
    from oracle import c_oracle as co
    from vllm_kunlun_amd import synth
    # a decode batch on the weight-streaming path with a folded shared expert, then a smaller
    # batch of another shape on the tile kernel
    first = synth.scaled(synth.SHAPES["dsv3-decode"], M=96, H=1024, E=32, K=4, I=256, n_group=4, topk_group=2,
                         I_shared=256)
    second = synth.scaled(synth.SHAPES["qwen3-decode"], M=40, H=512, E=8, K=4, I=128)
    for shape, seed in ((first, 3), (second, 4)):
        sl = synth.make_w8a8_layer(shape, "cuda", seed=seed)
        want, got = _both_ways(sl)
        assert np.array_equal(bits(got), bits(want)), f"{shape.name} M={shape.M}: static-workspace output differs"
        w13, w13_max, w2, w2_max, shared = sl.host_weights()
        ref = co.forward_w8a8(bits(sl.x), sl.logits.cpu().numpy(), w13.numpy(), w13_max.numpy(), w2.numpy(),
                              w2_max.numpy(), shape.K, shape.scoring, True, shape.n_group, shape.topk_group,
                              shape.routed_scale, None if sl.bias is None else sl.bias.cpu().numpy(),
                              None if shared is None else tuple(t.numpy() for t in shared))
        assert np.array_equal(bits(got), ref), f"{shape.name} M={shape.M}: differs from the oracle"
