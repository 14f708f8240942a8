"""The C ABI without a GPU: libkmoe.so loads, exports every function that
include/kmoe.h declares, and rejects bad arguments with status codes before any
HIP call (so these run on a CPU-only host). No compute call is made here."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def L():
    from vllm_kunlun_amd import _lib
    return _lib


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "kmoe.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(kmoe_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_functions():
    names = _declared_functions()
    assert "kmoe_moe_forward" in names and "kmoe_grouped_gemm_i8" in names and len(names) >= 15


def test_library_exports_every_declared_symbol(L):
    for name in _declared_functions():
        assert hasattr(L.lib, name), f"{name} is declared in include/kmoe.h but not exported by libkmoe.so"
    assert set(_declared_functions()) == set(L.EXPORTS), "the ctypes binding must cover exactly the declared ABI"
    assert b"gfx950" in L.lib.kmoe_version()


def test_struct_layouts_match_the_header(L, tmp_path):
    """The ctypes mirrors against the C declarations themselves: a C program that includes include/kmoe.h
    prints sizeof and the offsets of a few late fields of every argument struct (gcc, host only)."""
    import subprocess
    structs = {"kmoe_gemm_i8_args": (L.GemmI8Args, ["lod", "acc_out", "w_tail", "tail_src0", "act_dtype"]),
               "kmoe_gemm_bf16_args": (L.GemmBf16Args, ["lod", "y", "bias", "act_limit"]),
               "kmoe_gemm_fp8_args": (L.GemmFp8Args, ["w_scale", "y", "w_tail", "tail_src0"]),
               "kmoe_gemm_w4_args": (L.GemmW4Args, ["w_scale", "lod", "y", "w_layout"]),
               "kmoe_moe_args": (L.MoEArgs, ["logits", "I_shared", "out", "w_gate", "ws_layout", "group_size",
                                             "act_dtype", "shared_scale", "tile_variant", "first_expert", "flags"]),
               "kmoe_moe_layout": (L.MoELayout, ["align_ws", "down", "sh_out", "n_logit_planes"])}
    lines = ["#include <stdio.h>", "#include <stddef.h>", '#include "kmoe.h"', "int main(void) {"]
    for name, (_, fields) in structs.items():
        lines.append(f'  printf("{name} %zu", sizeof({name}));')
        for f in fields:
            lines.append(f'  printf(" %zu", offsetof({name}, {f}));')
        lines.append('  printf("\\n");')
    lines += ["  return 0;", "}"]
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split("\n")
    for line in filter(None, out):
        name, size, *offsets = line.split()
        cls, fields = structs[name]
        assert C.sizeof(cls) == int(size), name
        assert [getattr(cls, f).offset for f in fields] == [int(o) for o in offsets], name


def test_null_and_shape_errors_are_status_codes(L):
    lib = L.lib
    assert lib.kmoe_softmax_topk(None, 4, 8, 2, 1, None, None, None) == -1
    assert b"NULL" in lib.kmoe_last_error()
    one = C.c_void_p(0x1000)  # never dereferenced: validation fails first
    assert lib.kmoe_softmax_topk(one, 4, 0, 2, 1, one, one, None) == -2
    assert lib.kmoe_clock_probe(None, 1, 8, None) == -1
    assert lib.kmoe_clock_probe(one, 0, 8, None) == -2 and lib.kmoe_clock_probe(one, 1, 1, None) == -2
    assert lib.kmoe_softmax_topk(one, 4, 8, 9, 1, one, one, None) == -2          # K > E
    assert lib.kmoe_softmax_topk(one, 4, 2048, 8, 1, one, one, None) == -2       # E too large
    assert lib.kmoe_sigmoid_group_topk_norm(one, None, 4, 30, 4, 4, 2, 1.0, one, one, None) == -2  # E % n_group
    assert lib.kmoe_sigmoid_group_topk_norm(one, None, 4, 8, 4, 8, 2, 1.0, one, one, None) == -2   # groups of 1
    assert lib.kmoe_sigmoid_group_topk_norm(one, None, 4, 32, 8, 8, 1, 1.0, one, one, None) == -2  # K > kept experts
    assert lib.kmoe_align(one, 10, 4096, one, one, one, one, None, 0, None) == -2
    assert lib.kmoe_align(one, 100000, 64, one, one, one, one, None, 0, None) == -4  # needs a workspace
    assert b"workspace" in lib.kmoe_last_error()
    assert lib.kmoe_quant_i8_rows(one, 100, 4, 100, one, 100, one, None) == -2     # C % 8
    assert lib.kmoe_quant_fp8_group128(one, 200, 4, 200, one, 200, one, None) == -2
    assert lib.kmoe_silu_and_mul(one, 20, 4, 10, one, 10, None) == -2
    assert lib.kmoe_combine(one, 64, one, one, None, 4, 65, 64, 1.0, None, 0, one, 64, None) == -2  # K > 64
    assert lib.kmoe_grouped_gemm_i8(None, None) == -1


def test_gemm_argument_validation(L):
    g = L.GemmI8Args()
    assert L.lib.kmoe_grouped_gemm_i8(g, None) == -1
    for f in ("a", "a_max", "w", "w_max", "lod", "y"):
        setattr(g, f, 0x1000)
    g.E, g.n, g.k, g.rows, g.lda, g.ldy, g.src_div = 4, 64, 100, 10, 112, 64, 1
    assert L.lib.kmoe_grouped_gemm_i8(g, None) == -2 and b"k=100" in L.lib.kmoe_last_error()
    g.k, g.lda, g.act = 128, 128, 7
    assert L.lib.kmoe_grouped_gemm_i8(g, None) == -3
    g.act, g.n = 1, 48
    assert L.lib.kmoe_grouped_gemm_i8(g, None) == -2   # SwiGLU needs n % 32 == 0
    g.n, g.act, g.a = 64, 0, 0x1001
    assert L.lib.kmoe_grouped_gemm_i8(g, None) == -2 and b"misaligned" in L.lib.kmoe_last_error()
    # the tile kernel (variants 5-11) moves K in 128-byte chunks: a single 64-byte step is refused, not run
    g.a, g.k, g.lda, g.w_layout, g.variant = 0x1000, 64, 64, L.KMOE_W_TILED, 5
    assert L.lib.kmoe_grouped_gemm_i8(g, None) == -3 and b"k >= 128" in L.lib.kmoe_last_error()


def test_forward_validation_and_workspace_layout(L):
    a = L.MoEArgs()
    lay = L.MoELayout()
    a.M, a.H, a.E, a.K, a.I = 64, 2048, 128, 8, 768
    assert L.lib.kmoe_moe_workspace_layout(a, lay) == 0
    P = 64 * 8
    assert lay.total_bytes >= P * 2048 * 2 + P * 768 * 3 + 64 * 2048
    offs = [getattr(lay, n) for n, _ in L.MoELayout._fields_[1:-3]] + [lay.logit_planes]
    assert offs == sorted(offs) and all(o % 256 == 0 for o in offs)
    a.K = 200
    assert L.lib.kmoe_moe_workspace_layout(a, lay) == -2
    a.K = 8
    assert L.lib.kmoe_moe_forward(a, None, 0, None) == -1        # tensor pointers missing
    for f in ("logits", "x", "w13", "w13_max", "w2", "w2_max", "out"):
        setattr(a, f, 0x1000)
    assert L.lib.kmoe_moe_forward(a, None, 0, None) == -4        # no workspace
    assert L.lib.kmoe_moe_forward(a, C.c_void_p(0x10000), 16, None) == -4
    a.scoring = 9
    assert L.lib.kmoe_moe_forward(a, C.c_void_p(0x10000), 1 << 40, None) == -3


def test_python_errors_follow_the_reference_convention(L):
    with pytest.raises(ValueError):
        L.check(-2)
    with pytest.raises(NotImplementedError):
        L.check(-3)
    with pytest.raises(RuntimeError):
        L.check(-5)


def test_method_selection_mirrors_reference():
    """get_moe_method: same scheme for gate/up/down, None -> unquantized, dynamic-token
    W8A8 -> the int8 method, anything else -> RuntimeError (reference:
    compressed_tensors_moe.py:43-108)."""
    import torch
    from vllm_kunlun_amd.ops.fused_moe.layer import FusedMoEConfig, KunlunUnquantizedFusedMoEMethod
    from vllm_kunlun_amd.quantization.compressed_tensors.compressed_tensors_moe import (
        KunlunCompressedTensorsMoEMethod, KunlunCompressedTensorsW8A8Int8MoEMethod)

    class Cfg:
        def __init__(self, schemes):
            self.schemes = schemes

        def get_scheme_dict(self, layer, name):
            return self.schemes[name.rsplit(".", 1)[-1]]

    layer = torch.nn.Module()
    layer.moe_config = FusedMoEConfig(experts_per_token=2)
    w8 = {"weights": dict(num_bits=8, strategy="channel", symmetric=True, dynamic=False),
          "input_activations": dict(num_bits=8, strategy="token", symmetric=True, dynamic=True), "format": "int-quantized"}
    m = KunlunCompressedTensorsMoEMethod.get_moe_method(Cfg(dict(gate_proj=w8, up_proj=w8, down_proj=w8)), layer, "l.e")
    assert isinstance(m, KunlunCompressedTensorsW8A8Int8MoEMethod) and m.is_monolithic
    m = KunlunCompressedTensorsMoEMethod.get_moe_method(Cfg(dict(gate_proj=None, up_proj=None, down_proj=None)), layer,
                                                       "l.e")
    assert isinstance(m, KunlunUnquantizedFusedMoEMethod)
    with pytest.raises(ValueError):
        KunlunCompressedTensorsMoEMethod.get_moe_method(Cfg(dict(gate_proj=w8, up_proj=None, down_proj=w8)), layer, "l.e")
    static = dict(w8, input_activations=dict(num_bits=8, strategy="tensor", symmetric=True, dynamic=False))
    with pytest.raises(RuntimeError):
        KunlunCompressedTensorsMoEMethod.get_moe_method(Cfg(dict(gate_proj=static, up_proj=static, down_proj=static)),
                                                       layer, "l.e")


def test_process_weights_after_loading_turns_scales_into_maxes():
    import torch
    from vllm_kunlun_amd import synth
    shape = synth.scaled(synth.SHAPES["qwen3-decode"], M=4, H=64, E=4, K=2, I=32)
    sl = synth.make_w8a8_layer(shape, "cpu", seed=0)
    w13 = sl.layer.w13_weight.float()
    mx = sl.layer.w13_weight_scale
    assert mx.shape == (4, 64, 1) and torch.all(mx > 0)
    assert torch.all(w13.abs().amax(-1, keepdim=True) == 127)      # per-channel quantisation reaches +-127
    before = mx.clone()
    sl.layer.quant_method.process_weights_after_loading(sl.layer)  # a second call multiplies again: it is in place
    assert torch.allclose(sl.layer.w13_weight_scale, before * 127.0)


def test_static_workspace_forward_refuses_what_does_not_fit(L):
    a = L.MoEArgs()
    a.M, a.H, a.E, a.K, a.I = 4096, 7168, 256, 8, 2048  # needs ~0.9 GB of intermediates
    a.format = L.KMOE_FMT_INT8
    assert L.lib.kmoe_moe_forward_static(C.byref(a), None) == -4
    assert b"built-in buffer" in L.lib.kmoe_last_error()


def test_kernel_trace_record_is_per_thread_and_empty_without_launches(L):
    lib = L.lib
    lib.kmoe_trace_kernels(1)
    assert lib.kmoe_traced_kernels() == b""
    lib.kmoe_trace_kernels(0)
    assert lib.kmoe_traced_kernels() == b""
