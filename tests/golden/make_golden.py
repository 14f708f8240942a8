#!/usr/bin/env python3
"""Writes the golden fixtures in this directory from the CPU oracles.

The reference holds no vectors for the MoE path (its kernels are closed), so the
fixtures are produced here, by the oracle whose functions tests/test_oracle_pins.py
pins, and committed as data. They freeze today's oracle against accidental change
and give the GPU tests inputs/outputs that need no oracle build.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import c_oracle as co  # noqa: E402
from oracle import torch_moe as tm  # noqa: E402


def bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def main():
    g = torch.Generator().manual_seed(20240)
    # 1. routing
    logits = torch.randn(16, 32, generator=g)
    logits[0, :5] = 5.0  # exact ties above everything else: the lowest ids must win
    bias = torch.randn(32, generator=g) * 0.01
    w_sm, ids_sm = co.softmax_topk(logits.numpy(), 4, True)
    w_sg, ids_sg = co.sigmoid_group_topk_norm(logits.numpy(), bias.numpy(), 4, 4, 2, 2.5)
    np.savez_compressed(os.path.join(HERE, "routing.npz"), logits=logits.numpy(), bias=bias.numpy(), softmax_w=w_sm,
                        softmax_ids=ids_sm, sigmoid_w=w_sg, sigmoid_ids=ids_sg)
    # 2. a tiny W8A8 layer with a shared expert and all intermediates
    M, H, E, K, I, Is = 8, 64, 4, 2, 32, 32
    x = torch.randn(M, H, generator=g).bfloat16()
    lg = torch.randn(M, E, generator=g)
    w13, s13 = tm.quantize_weight_per_channel(torch.randn(E, 2 * I, H, generator=g) * 0.02)
    w2, s2 = tm.quantize_weight_per_channel(torch.randn(E, H, I, generator=g) * 0.02)
    a, sa = tm.quantize_weight_per_channel(torch.randn(2 * Is, H, generator=g) * 0.02)
    b, sb = tm.quantize_weight_per_channel(torch.randn(H, Is, generator=g) * 0.02)
    shared = (a.numpy(), (sa * 127).reshape(-1).numpy(), b.numpy(), (sb * 127).reshape(-1).numpy())
    out, inter = co.forward_w8a8(bits(x), lg.numpy(), w13.numpy(), (s13 * 127).numpy(), w2.numpy(),
                                 (s2 * 127).numpy(), K, shared=shared, out_scale=2.5, intermediates=True)
    np.savez_compressed(os.path.join(HERE, "w8a8_tiny_layer.npz"), x=bits(x), logits=lg.numpy(), w13=w13.numpy(),
                        w13_max=(s13 * 127).numpy(), w2=w2.numpy(), w2_max=(s2 * 127).numpy(), ws13=shared[0],
                        ws13_max=shared[1], ws2=shared[2], ws2_max=shared[3], K=K, out_scale=2.5, out=out, **inter)
    # 3. fp8 group quantisation edge values
    edge = torch.zeros(3, 128)
    edge[0, :8] = torch.tensor([0.0, 448.0, -448.0, 2.0 ** -9, 2.0 ** -10, 224.0, 1.0, -3.5])
    edge[1] = torch.linspace(-1, 1, 128)
    edge[2, 5] = 1e-3
    q, s = co.quant_fp8_group128(bits(edge.bfloat16()))
    np.savez_compressed(os.path.join(HERE, "fp8_group_quant.npz"), x=bits(edge.bfloat16()), q=q, scale=s)
    # 4. a tiny unquantized layer through the reference's torch expert loop (bf16)
    w13f = (torch.randn(E, 2 * I, H, generator=g) * 0.05).bfloat16()
    w2f = (torch.randn(E, H, I, generator=g) * 0.05).bfloat16()
    ref = tm.bf16_moe(x, lg, w13f, w2f, K, True)
    np.savez_compressed(os.path.join(HERE, "bf16_tiny_layer.npz"), x=bits(x), logits=lg.numpy(), w13=bits(w13f),
                        w2=bits(w2f), K=K, out=bits(ref))
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()
