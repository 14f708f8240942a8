"""HIP-graph capture of the layer and of the dense W8A8 op: what a serving engine does with the
decode step. Each graph is replayed several times with new inputs and with eager work and
synchronisations of the process between the replays; every replay must give the bits of the eager call."""
import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu


def _eager_noise():
    a = torch.randn(256, 256, device="cuda")
    (a @ a).sum().item()


def _replays(graph, static_inputs, fresh_inputs, static_out, eager):
    for fresh in fresh_inputs:
        for dst, src in zip(static_inputs, fresh):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        got = static_out.clone()
        _eager_noise()
        want = eager(*fresh)
        torch.cuda.synchronize()
        assert torch.equal(got, want)


def test_apply_monolithic_under_graph_capture():
    from vllm_kunlun_amd import synth
    shape = synth.scaled(synth.SHAPES["dsv3-decode"], M=48, H=1024, E=32, K=4, I=256, n_group=4, topk_group=2,
                         I_shared=256)
    sl = synth.make_w8a8_layer(shape, "cuda", seed=5)
    method, kw = sl.layer.quant_method, sl.apply_kwargs()
    x, logits = sl.x.clone(), sl.logits.clone()
    eager = lambda xx, ll: method.apply_monolithic(sl.layer, xx, ll, **kw)  # noqa: E731
    eager(x, logits)                                   # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = method.apply_monolithic(sl.layer, x, logits, **kw)
    g = torch.Generator(device="cuda").manual_seed(9)
    fresh = [(torch.randn(shape.M, shape.H, generator=g, device="cuda").bfloat16(),
              torch.randn(shape.M, shape.E, generator=g, device="cuda")) for _ in range(4)]
    _replays(graph, (x, logits), fresh, out, eager)


@pytest.mark.parametrize("side", [False, True], ids=["one-stream", "side-stream"])
@pytest.mark.parametrize("quant", ["int8", "fp8"])
def test_shared_expert_on_the_side_stream_under_graph_capture(quant, side):
    """A shared expert of another width (int8) and the fp8 decode layer run their shared MLP in launches of its own:
    on the caller's stream by default, and with KMOE_FLAG_SIDE_STREAM (the method's side_stream) on the library's
    second stream, forked from and joined into the caller's. Both settings, eager and captured (the fork and join
    become graph edges): same bits every time (int8: the oracle's)."""
    from vllm_kunlun_amd import synth
    base = "dsv3-decode" if quant == "int8" else "dsv3-fp8-decode"
    shape = synth.scaled(synth.SHAPES[base], M=40, H=512, E=32, K=4, I=128, n_group=4, topk_group=2,
                         I_shared=384 if quant == "int8" else 128)
    sl = synth.make_layer(shape, "cuda", seed=7)
    method, kw = sl.layer.quant_method, sl.apply_kwargs()
    method.side_stream = side
    x, logits = sl.x.clone(), sl.logits.clone()
    eager = lambda xx, ll: method.apply_monolithic(sl.layer, xx, ll, **kw)  # noqa: E731
    first = eager(x, logits)                           # creates the second stream (never inside a capture)
    torch.cuda.synchronize()
    if quant == "int8":  # the overlapped pass gives the oracle's bits
        import numpy as np
        from oracle import c_oracle as co
        b16 = lambda t: t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)  # noqa: E731
        w13, w13_max, w2, w2_max, shared = sl.host_weights()
        ref = co.forward_w8a8(b16(x), logits.cpu().numpy(), w13.numpy(), w13_max.numpy(), w2.numpy(), w2_max.numpy(),
                              shape.K, shape.scoring, True, shape.n_group, shape.topk_group, shape.routed_scale,
                              sl.bias.cpu().numpy(), tuple(t.numpy() for t in shared))
        assert np.array_equal(b16(first), ref)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = method.apply_monolithic(sl.layer, x, logits, **kw)
    g = torch.Generator(device="cuda").manual_seed(12)
    fresh = [(torch.randn(shape.M, shape.H, generator=g, device="cuda").bfloat16(),
              torch.randn(shape.M, shape.E, generator=g, device="cuda")) for _ in range(4)]
    _replays(graph, (x, logits), fresh, out, eager)


def test_static_workspace_forward_under_graph_capture():
    from vllm_kunlun_amd import _lib as L
    from vllm_kunlun_amd import synth
    from vllm_kunlun_amd._plan import make_moe_plan
    shape = synth.scaled(synth.SHAPES["qwen3-decode"], M=32, H=512, E=16, K=4, I=128)
    sl = synth.make_w8a8_layer(shape, "cuda", seed=6)
    lay = sl.layer
    x, logits = sl.x.clone(), sl.logits.clone()
    out = torch.empty_like(x)
    plan = make_moe_plan(L.KMOE_FMT_INT8, x, logits, out, shape.K, lay.w13_weight, lay.w2_weight, lay.w13_weight_scale,
                         lay.w2_weight_scale, "softmax", True)
    call = lambda: L.check(L.lib.kmoe_moe_forward_static(C.byref(plan.args), L.stream()))  # noqa: E731
    # one call on the GPU outside a capture (here of the workspace entry point) has to come first: it looks up the
    # built-in buffer's device address, which a captured call may not do
    plan()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    method = lay.quant_method
    g = torch.Generator(device="cuda").manual_seed(10)
    fresh = [(torch.randn(shape.M, shape.H, generator=g, device="cuda").bfloat16(),
              torch.randn(shape.M, shape.E, generator=g, device="cuda")) for _ in range(3)]
    _replays(graph, (x, logits), fresh, out, lambda xx, ll: method.apply_monolithic(lay, xx, ll))


def test_dense_matmul_op_under_graph_capture():
    import vllm_kunlun_amd  # noqa: F401  (registers torch.ops._C.*)
    M, n, k = 24, 256, 512
    g = torch.Generator(device="cuda").manual_seed(11)
    w = torch.randint(-127, 128, (n, k), generator=g, device="cuda", dtype=torch.int8)
    w_max = torch.rand(n, 1, generator=g, device="cuda") + 0.5
    x = torch.randint(-127, 128, (M, k), generator=g, device="cuda", dtype=torch.int8)
    x_max = torch.rand(M, 1, generator=g, device="cuda") + 0.5
    eager = lambda xx, mm: torch.ops._C.matmul(xx, w, torch.bfloat16, x_pc_max=mm, w_pc_max=w_max)  # noqa: E731
    eager(x, x_max)                                    # uploads the {0, M} row range once
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = eager(x, x_max)
    fresh = [(torch.randint(-127, 128, (M, k), generator=g, device="cuda", dtype=torch.int8),
              torch.rand(M, 1, generator=g, device="cuda") + 0.5) for _ in range(3)]
    _replays(graph, (x, x_max), fresh, out, eager)


def test_two_threads_share_the_side_stream():
    """Two host threads, each with a stream and a layer of its own whose shared expert runs on the library's second
    stream (one per GPU: both threads fork to it and join from it), calling at the same time: every call gives the
    bits the layer gives alone."""
    import threading
    from vllm_kunlun_amd import synth
    shapes = [synth.scaled(synth.SHAPES["dsv3-decode"], M=24 + 8 * i, H=512, E=32, K=4, I=128, n_group=4, topk_group=2,
                           I_shared=256 + 128 * i) for i in range(2)]
    layers = [synth.make_layer(sh, "cuda", seed=20 + i) for i, sh in enumerate(shapes)]
    for sl in layers:
        sl.layer.quant_method.side_stream = True
    want = []
    for sl in layers:
        want.append(sl.layer.quant_method.apply_monolithic(sl.layer, sl.x, sl.logits, **sl.apply_kwargs()).clone())
    torch.cuda.synchronize()
    errors = []

    def worker(i):
        try:
            sl = layers[i]
            stream = torch.cuda.Stream()
            stream.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(stream):
                for it in range(40):
                    out = sl.layer.quant_method.apply_monolithic(sl.layer, sl.x, sl.logits, **sl.apply_kwargs())
                    if it % 8 == 7:
                        stream.synchronize()
                        if not torch.equal(out, want[i]):
                            errors.append((i, it))
                stream.synchronize()
                if not torch.equal(out, want[i]):
                    errors.append((i, "last"))
        except Exception as ex:  # noqa: BLE001
            errors.append((i, repr(ex)))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors


def test_tile_height_chosen_on_the_device_under_graph_replay():
    """Variant 17 of the int8 GEMM enqueues a tall-tile launch and a 128-row-tile launch; the row counts decide in
    each launch's prologue which of the two works. Captured once, the pair is replayed with row counts that suit
    the tall tile and with counts that overflow it: every replay gives the bits of the 128-row-tile kernel."""
    from vllm_kunlun_amd import _lib as L
    E, n, k, rows = 20, 256, 384, 3000
    g = torch.Generator(device="cuda").manual_seed(3)
    a = torch.randint(-127, 128, (rows, k), generator=g, dtype=torch.int8, device="cuda")
    a_max = torch.rand(rows, generator=g, device="cuda") + 0.1
    w = torch.randint(-127, 128, (E, n, k), generator=g, dtype=torch.int8, device="cuda")
    w_max = torch.rand(E, n, generator=g, device="cuda") + 0.1
    wt = torch.empty_like(w)
    L.check(L.lib.kmoe_tile_weights_i8(w.data_ptr(), wt.data_ptr(), E, n, k, L.stream()))

    def lod_of(counts):
        assert sum(counts) == rows
        return torch.tensor([0] + list(torch.tensor(counts).cumsum(0)), dtype=torch.int32, device="cuda")

    even = [150] * E                                              # every expert fits a 192-row tile
    skew = [400, 20, 390, 10, 380, 30, 370, 40] + [113] * 11 + [117]  # a fifth of them overflows it
    lods = [lod_of(even), lod_of(skew), lod_of(even[::-1]), lod_of(skew[::-1])]
    lod = lods[0].clone()
    y = torch.zeros(rows, n, dtype=torch.bfloat16, device="cuda")
    args = L.GemmI8Args()
    args.a, args.lda, args.a_max, args.src_div = a.data_ptr(), k, a_max.data_ptr(), 1
    args.w, args.w_max, args.lod = wt.data_ptr(), w_max.data_ptr(), lod.data_ptr()
    args.E, args.n, args.k, args.rows = E, n, k, rows
    args.y, args.ldy, args.act, args.w_layout = y.data_ptr(), n, 0, L.KMOE_W_TILED

    def run(variant):
        args.variant = variant
        L.check(L.lib.kmoe_grouped_gemm_i8(args, L.stream()))

    run(17)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run(17)
    for fresh in lods:
        lod.copy_(fresh)
        y.fill_(7.0)
        graph.replay()
        torch.cuda.synchronize()
        got = y.clone()
        _eager_noise()
        y.fill_(7.0)
        run(6)
        torch.cuda.synchronize()
        assert torch.equal(got, y)
