"""The benchmark configurations at their FULL sizes. The oracle cannot run thousands of tokens
through 256 experts in test time, so the large batches are held to what does not depend on
size: every token's result is independent of the batch it travels in. That gives, bit for bit,
  * permutation equivariance: shuffling the tokens shuffles the outputs;
  * batch-size independence: a token gets the same bits in a decode batch (weight-streaming
    kernels, chunk-major codes, fused prologue) as in a prefill batch (persistent tile kernel), and in
    the batches in between, on either side of every switch of kernel and tile height;
  * a spot check: a handful of tokens of the big batch through the C oracle.
The decode batches are compared with the C oracle in full."""
import numpy as np
import pytest
import torch


pytestmark = pytest.mark.gpu

from oracle import c_oracle as co  # noqa: E402

REL_L2_FP8 = 3e-2  # tolerance of the fp8 layer's bf16 output against the oracle


def _host(t):
    return None if t is None else t.detach().cpu()


def bits(t):
    """16-bit patterns of a bfloat16 or float16 tensor."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _oracle(sl, host, x, logits):
    w13, w13_max, w2, w2_max, shared = host
    s = sl.shape
    sh = None if shared is None else tuple(t.numpy() for t in shared)
    return co.forward_w8a8(bits(x), _host(logits).float().numpy(), w13.numpy(), w13_max.numpy(), w2.numpy(),
                           w2_max.numpy(), s.K, s.scoring, True, s.n_group, s.topk_group, s.routed_scale,
                           None if sl.bias is None else _host(sl.bias).numpy(), sh, f16=x.dtype == torch.float16)


def _run(sl, x, logits):
    out = sl.layer.quant_method.apply_monolithic(sl.layer, x, logits, **sl.apply_kwargs())
    torch.cuda.synchronize()
    return out


@pytest.fixture(scope="module")
def qwen3():
    from vllm_kunlun_amd import synth
    sl = synth.make_w8a8_layer(synth.SHAPES["qwen3-prefill"], "cuda", seed=0)  # 8192 tokens; decode = its first 64
    return sl, sl.host_weights()


@pytest.fixture(scope="module")
def dsv3():
    from vllm_kunlun_amd import synth
    sl = synth.make_w8a8_layer(synth.SHAPES["dsv3-prefill"], "cuda", seed=0)   # 4096 tokens; decode = its first 128
    return sl, sl.host_weights()


def _properties(sl, host, n_decode, n_spot, seed, mids=(), half=False):
    g = torch.Generator(device="cuda").manual_seed(seed)
    x, logits = (sl.x.half() if half else sl.x), sl.logits
    M = x.shape[0]
    full = _run(sl, x, logits)
    assert bool(torch.isfinite(full.float()).all())
    # permutation equivariance
    perm = torch.randperm(M, generator=g, device="cuda")
    shuffled = _run(sl, x[perm].contiguous(), logits[perm].contiguous())
    assert torch.equal(shuffled, full[perm]), "a token's output depends on its position in the batch"
    # the decode batch of the configuration, alone: same bits as inside the prefill batch, and the oracle's bits
    dec = _run(sl, x[:n_decode].contiguous(), logits[:n_decode].contiguous())
    assert torch.equal(dec, full[:n_decode]), "decode and prefill kernels disagree"
    ref = _oracle(sl, host, x[:n_decode], logits[:n_decode])
    assert np.array_equal(bits(dec), ref), "decode batch vs C oracle"
    # batches in between: the streaming kernels' last sizes, the tile kernel on 64-row tiles, on 96-row tiles and
    # on 128-row tiles that are mostly padding
    for m in mids:
        mid = _run(sl, x[:m].contiguous(), logits[:m].contiguous())
        assert torch.equal(mid, full[:m]), f"a batch of {m} tokens disagrees with the full batch"
    # spot check of the big batch: random tokens through the oracle
    idx = torch.randperm(M, generator=g, device="cuda")[:n_spot]
    ref_spot = _oracle(sl, host, x[idx], logits[idx])
    assert np.array_equal(bits(full[idx]), ref_spot), "prefill batch vs C oracle on a sample of its tokens"


def test_qwen3_full_size(qwen3):
    """Qwen3-30B-A3B shape: 128 experts, top-8, hidden 2048, intermediate 768; 8192 and 64 tokens."""
    sl, host = qwen3
    _properties(sl, host, n_decode=64, n_spot=48, seed=1, mids=(160, 176, 512, 768, 800, 1100, 1200, 1500))


def test_qwen3_full_size_float16(qwen3):
    """The same layer with float16 activations (the dtype of the reference's deployment recipes)."""
    sl, host = qwen3
    _properties(sl, host, n_decode=64, n_spot=48, seed=4, mids=(160, 512, 900, 1500), half=True)


def test_qwen3_full_size_skewed_routing(qwen3):
    """+2.0 on the logits of 8 experts: a few experts get thousands of rows, most a handful."""
    sl, host = qwen3
    logits = sl.logits.clone()
    logits[:, torch.arange(8, device="cuda") * 16] += 2.0
    full = _run(sl, sl.x, logits)
    idx = torch.arange(0, sl.x.shape[0], 171, device="cuda")[:48]
    assert np.array_equal(bits(full[idx]), _oracle(sl, host, sl.x[idx], logits[idx]))


def test_dsv3_full_size(dsv3):
    """DeepSeek-V3 shape: 256 experts + shared, sigmoid grouped top-8, hidden 7168, intermediate 2048;
    4096 and 128 tokens."""
    sl, host = dsv3
    _properties(sl, host, n_decode=128, n_spot=16, seed=2, mids=(320, 352, 1024, 1536, 1600))


def test_dsv3_full_size_float16(dsv3):
    sl, host = dsv3
    _properties(sl, host, n_decode=128, n_spot=12, seed=5, mids=(352, 1536, 1800), half=True)


def _fp8_oracle(sl, host, x, logits):
    w13, w13_s, w2, w2_s, sh = host
    s = sl.shape
    u8 = lambda t: t.view(torch.uint8).numpy()  # noqa: E731
    shared = None if sh is None else (u8(sh[0]), sh[1].numpy(), u8(sh[2]), sh[3].numpy())
    return co.forward_fp8(bits(x), _host(logits).numpy(), u8(w13), w13_s.numpy(), u8(w2), w2_s.numpy(), s.K, s.scoring,
                          True, s.n_group, s.topk_group, s.routed_scale, _host(sl.bias).numpy(), shared)


def _routing_ids(sl, M):
    m, s = sl.layer.quant_method, sl.shape
    ids = m.last_workspace[m.last_layout.topk_ids: m.last_layout.topk_ids + 4 * M * s.K].view(torch.int32)
    return ids.view(M, s.K)


def _fp8_checks(sl, host, n_decode, n_spot):
    """fp8 block-scaled layer: the prefill batch on a sample of its tokens and the decode batch in full
    against the C oracle within the fp8 tolerance (MFMA and oracle sum in different orders); routing ids
    bit-exact; the decode batch (16-row LDS-staged kernel + a shared-expert pass of its own) against the
    same tokens inside the prefill batch (tile kernel, shared expert folded in) within that tolerance."""
    from conftest import from_bits, rel_l2
    s = sl.shape
    full = _run(sl, sl.x, sl.logits)
    assert bool(torch.isfinite(full.float()).all())
    idx = torch.arange(5, s.M, 257, device="cuda")[:n_spot]
    ids = _routing_ids(sl, s.M)[idx].cpu().numpy()
    assert rel_l2(full[idx], from_bits(_fp8_oracle(sl, host, sl.x[idx], sl.logits[idx]))) <= REL_L2_FP8
    _, ids_ref = co.sigmoid_group_topk_norm(_host(sl.logits[idx]).numpy(), _host(sl.bias).numpy(), s.K, s.n_group,
                                            s.topk_group, s.routed_scale)
    assert np.array_equal(ids, ids_ref)
    x, logits = sl.x[:n_decode].contiguous(), sl.logits[:n_decode].contiguous()
    dec = _run(sl, x, logits)
    ids = _routing_ids(sl, n_decode).cpu().numpy()
    assert bool(torch.isfinite(dec.float()).all())
    assert rel_l2(dec, from_bits(_fp8_oracle(sl, host, x, logits))) <= REL_L2_FP8, "fp8 decode batch vs C oracle"
    _, ids_ref = co.sigmoid_group_topk_norm(_host(logits).numpy(), _host(sl.bias).numpy(), s.K, s.n_group,
                                            s.topk_group, s.routed_scale)
    assert np.array_equal(ids, ids_ref)
    assert rel_l2(dec, full[:n_decode]) <= REL_L2_FP8, "fp8 decode and prefill kernels disagree"


def test_dsv3_fp8_full_size():
    """The fp8 block-scaled layer at the DeepSeek-V3 shape: 4096 tokens (sample) and 128 tokens (in full)."""
    from vllm_kunlun_amd import synth
    sl = synth.make_fp8_layer(synth.SHAPES["dsv3-fp8-prefill"], "cuda", seed=0)
    _fp8_checks(sl, sl.host_weights(), n_decode=128, n_spot=16)


def test_kimi_k2_full_size_int8():
    """Kimi-K2 shape (384 experts + shared, sigmoid top-8 without groups, hidden 7168, intermediate 2048),
    int8: 4096 and 128 tokens, bit for bit."""
    from vllm_kunlun_amd import synth
    sl = synth.make_w8a8_layer(synth.SHAPES["kimi-prefill"], "cuda", seed=0)
    _properties(sl, sl.host_weights(), n_decode=128, n_spot=12, seed=3, mids=(480, 528))


def test_kimi_k2_full_size_fp8():
    """Kimi-K2 shape with fp8 block-scaled weights: 4096 tokens (sample) and 128 tokens (in full)."""
    from vllm_kunlun_amd import synth
    sl = synth.make_fp8_layer(synth.SHAPES["kimi-fp8-prefill"], "cuda", seed=0)
    _fp8_checks(sl, sl.host_weights(), n_decode=128, n_spot=12)
