"""Seeded random layer shapes through apply_monolithic against the C oracle, bit for bit (W8A8 path, bfloat16 and
float16 activations). The curated cases elsewhere sit on the known switch points of the launchers (rows per expert
10 / 48 / 96 / 256, tileable or not, shared expert folded or not); these draw the dimensions at random so that
combinations nobody thought of get a turn: any hidden and intermediate size that is a multiple of 16, 2 to 96
experts, top-1 to top-8, softmax or sigmoid routing with a random valid grouping, no shared expert, one of the
routed width or one of another width, 1 to 900 tokens, sometimes with a few hot experts."""
import random

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import c_oracle as co  # noqa: E402


def _bits16(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _draw(seed):
    rng = random.Random(seed)
    E = rng.choice([2, 3, 4, 6, 8, 12, 16, 24, 32, 48, 64, 96])
    K = rng.randint(1, min(E, 8))
    M = int(round(2 ** rng.uniform(0, 9.8)))                       # 1 .. 891, more small than large
    H = 16 * rng.randint(4, 48) if rng.random() < 0.3 else 64 * rng.randint(2, 16)
    I = 16 * rng.randint(2, 24) if rng.random() < 0.3 else 64 * rng.randint(1, 8)
    over = dict(M=M, H=H, E=E, K=K, I=I)
    sigmoid = rng.random() < 0.5
    if sigmoid:
        groups = [g for g in (1, 2, 3, 4, 8) if E % g == 0 and E // g >= 2]
        g = rng.choice(groups)
        tg = rng.randint(1, g)
        while K > tg * (E // g):
            tg += 1
        over.update(n_group=g, topk_group=tg, routed_scale=rng.choice([1.0, 2.5, 16.0]))
        shared = rng.choice(["none", "same", "other"])
        over["I_shared"] = {"none": 0, "same": I, "other": 16 * rng.randint(2, 40)}[shared]
    if rng.random() < 0.25 and E >= 4:
        over.update(hot_experts=rng.choice([1, 2]), hot_bias=rng.choice([1.0, 3.0]))
    return ("dsv3-decode" if sigmoid else "qwen3-decode"), over, rng.random() < 0.4


@pytest.mark.parametrize("seed", range(200))
def test_random_layer_shape(seed):
    from vllm_kunlun_amd import synth
    base, over, half = _draw(seed)
    shape = synth.scaled(synth.SHAPES[base], **over)
    sl = synth.make_layer(shape, "cuda", seed=seed, dtype=torch.float16 if half else torch.bfloat16)
    out = sl.layer.quant_method.apply_monolithic(sl.layer, sl.x, sl.logits, **sl.apply_kwargs())
    torch.cuda.synchronize()
    w13, w13_max, w2, w2_max, shared = sl.host_weights()
    sh = None if shared is None else tuple(t.numpy() for t in shared)
    ref = co.forward_w8a8(_bits16(sl.x), sl.logits.cpu().numpy(), w13.numpy(), w13_max.numpy(), w2.numpy(),
                          w2_max.numpy(), shape.K, shape.scoring, True, shape.n_group, shape.topk_group,
                          shape.routed_scale, None if sl.bias is None else sl.bias.cpu().numpy(), sh, f16=half)
    assert out.dtype == sl.x.dtype and np.array_equal(_bits16(out), ref), f"{base} {over} half={half}"


def _rel_l2(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))


@pytest.mark.parametrize("seed", range(48))
def test_random_unquantized_layer_shape(seed):
    """The same draw for the unquantized layer (bfloat16 or float16 weights): MFMA sums in its own order, so the
    output is held to rel-L2 <= 1e-2 (bfloat16) / 1e-3 (float16) against the oracle; no shared expert on this path."""
    from vllm_kunlun_amd import synth
    base, over, half = _draw(1000 + seed)
    over = {k: v for k, v in over.items() if k not in ("I_shared", "routed_scale")}
    over.update(quant="none", I_shared=0)
    shape = synth.scaled(synth.SHAPES[base], **over)
    sl = synth.make_layer(shape, "cuda", seed=seed, dtype=torch.float16 if half else torch.bfloat16)
    out = sl.layer(sl.x, sl.logits)
    torch.cuda.synchronize()
    w13, _, w2, _, _ = sl.host_weights()
    ref = co.forward_bf16(_bits16(sl.x), sl.logits.cpu().numpy(), _bits16(w13), _bits16(w2), shape.K, shape.scoring, True,
                          shape.n_group, shape.topk_group, 1.0, None if sl.bias is None else sl.bias.cpu().numpy(),
                          f16=half)
    ref_t = torch.from_numpy(ref.view(np.int16)).view(torch.float16 if half else torch.bfloat16)
    assert _rel_l2(out, ref_t) <= (1e-3 if half else 1e-2), f"{base} {over} half={half}"


@pytest.mark.parametrize("seed", range(32))
def test_random_fp8_layer_shape(seed):
    """fp8 block-scaled layer (hidden and intermediate sizes in multiples of 128; bfloat16 or float16 activations):
    rel-L2 <= 3e-2 against the oracle."""
    from vllm_kunlun_amd import synth
    base, over, half = _draw(2000 + seed)
    rng = random.Random(seed)
    over.update(H=128 * rng.randint(1, 6), I=128 * rng.randint(1, 4), quant="fp8")
    if over.get("I_shared"):
        over["I_shared"] = over["I"] if rng.random() < 0.5 else 128 * rng.randint(1, 4)
    shape = synth.scaled(synth.SHAPES[base], **over)
    sl = synth.make_layer(shape, "cuda", seed=seed, dtype=torch.float16 if half else torch.bfloat16)
    out = sl.layer.quant_method.apply_monolithic(sl.layer, sl.x, sl.logits, **sl.apply_kwargs())
    torch.cuda.synchronize()
    w13, w13_s, w2, w2_s, sh = sl.host_weights()
    u8 = lambda t: t.view(torch.uint8).numpy()  # noqa: E731
    shared = None if sh is None else (u8(sh[0]), sh[1].numpy(), u8(sh[2]), sh[3].numpy())
    ref = co.forward_fp8(_bits16(sl.x), sl.logits.cpu().numpy(), u8(w13), w13_s.numpy(), u8(w2), w2_s.numpy(), shape.K,
                         shape.scoring, True, shape.n_group, shape.topk_group, shape.routed_scale,
                         None if sl.bias is None else sl.bias.cpu().numpy(), shared, f16=half)
    ref_t = torch.from_numpy(ref.view(np.int16)).view(torch.float16 if half else torch.bfloat16)
    assert out.dtype == sl.x.dtype and _rel_l2(out, ref_t) <= 3e-2, f"{base} {over} half={half}"


@pytest.mark.parametrize("seed", range(32))
def test_random_w4_layer_shape(seed):
    """Packed 4-bit weights kept alone (hidden and intermediate sizes in multiples of 128, groups of 32, 64, 128 or a
    whole row; bfloat16 or float16): small batches on the streaming kernel, 25 rows per expert and more on the
    128-row tile kernel; against the oracle's unquantized layer on the weights its unpacking gives."""
    from vllm_kunlun_amd import synth
    base, over, half = _draw(3000 + seed)
    rng = random.Random(seed)
    over = {k: v for k, v in over.items() if k not in ("I_shared", "routed_scale")}
    H = 128 * rng.randint(1, 6)
    over.update(H=H, I=H if rng.random() < 0.3 else 128 * rng.randint(1, 4), quant="w4", I_shared=0)
    if rng.random() < 0.4:
        over["M"] = rng.randint(200, 2500)  # enough rows per expert for the tile kernel with most draws of E and K
    gs = rng.choice([32, 64, 128, None])
    over["group_size"] = gs if gs else (over["H"] if over["H"] == over["I"] else 128)
    shape = synth.scaled(synth.SHAPES[base], **over)
    sl = synth.make_layer(shape, "cuda", seed=seed, dtype=torch.float16 if half else torch.bfloat16)
    out = sl.layer(sl.x, sl.logits)
    torch.cuda.synchronize()
    p13, s13, p2, s2, _ = sl.host_weights()
    w13 = co.dequant_w4_bf16(p13.numpy(), _bits16(s13), shape.group_size, f16=half)
    w2 = co.dequant_w4_bf16(p2.numpy(), _bits16(s2), shape.group_size, f16=half)
    ref = co.forward_bf16(_bits16(sl.x), sl.logits.cpu().numpy(), w13, w2, shape.K, shape.scoring, True, shape.n_group,
                          shape.topk_group, 1.0, None if sl.bias is None else sl.bias.cpu().numpy(), f16=half)
    ref_t = torch.from_numpy(ref.view(np.int16)).view(torch.float16 if half else torch.bfloat16)
    assert _rel_l2(out, ref_t) <= (1e-3 if half else 1e-2), f"{base} {over} half={half}"
