"""Argument blocks for kmoe_moe_forward: one filled `kmoe_moe_args` + its workspace.

A plan binds fixed device buffers (x, logits, out, weights); calling it enqueues
the whole layer on the current HIP stream without allocating or synchronising,
so a serving loop — or a HIP-graph capture — can replay it. A plan belongs to the
stream that was current when it was built (its workspace is that stream's) and
refuses to launch on another.
"""
from __future__ import annotations

import collections
import weakref
from typing import Optional

import torch

from . import _lib as L


def _current_stream_id(device: torch.device) -> int:
    return int(torch.cuda.current_stream(device).cuda_stream)


class _Workspace:
    """Scratch buffers that only grow, one per (device, stream) (plays the role of vLLM's
    current_workspace_manager(), reference: vllm_kunlun/ops/_kunlun_ops.py:528-531). Work queued on one
    stream runs in order, so the calls of a stream can share a buffer; two streams cannot, and a buffer is
    only ever used on the stream it was allocated on (the caching allocator's own rule for reuse).
    At most MAX_STREAMS buffers are kept, least recently used first out: a process that makes and destroys
    streams does not keep a buffer per handle it has ever seen. A dropped buffer goes back to torch's
    allocator, which hands its memory out again only in the order of the stream it was allocated on, and a
    plan keeps its own reference to the buffer it was built with."""

    MAX_STREAMS = 8

    def __init__(self):
        self._buf = collections.OrderedDict()

    def get(self, nbytes: int, device: torch.device, stream_id: int) -> torch.Tensor:
        key = (device.type, device.index, stream_id)
        buf = self._buf.get(key)
        if buf is None or buf.numel() < nbytes:
            # allocated with the launching stream current, so the allocator ties the block to that stream
            buf = torch.empty(nbytes, dtype=torch.uint8, device=device)
            self._buf[key] = buf
        self._buf.move_to_end(key)
        while len(self._buf) > self.MAX_STREAMS:
            self._buf.popitem(last=False)
        return buf


WORKSPACE = _Workspace()


class MoEPlan:
    """A filled kmoe_moe_args block and its workspace, bound to the stream it was built on."""

    def __init__(self, args, layout, workspace, keepalive, stream_id=None):
        self.args, self.layout, self.workspace, self._keep = args, layout, workspace, keepalive
        self.stream_id = stream_id

    def __call__(self) -> None:
        if self.stream_id is not None:
            now = _current_stream_id(self.workspace.device)
            if now != self.stream_id:
                raise RuntimeError(
                    f"this MoE plan was built on stream {self.stream_id:#x} and is being launched on stream "
                    f"{now:#x}: its workspace belongs to the first stream (two streams sharing it would race). "
                    "Build the plan with the launching stream current (inside `with torch.cuda.stream(s)` or the "
                    "graph capture that will run it).")
        L.check(L.lib.kmoe_moe_forward(self.args, L.ptr(self.workspace), self.workspace.numel(), L.stream()))

    def view(self, name: str, count: int, dtype: torch.dtype) -> torch.Tensor:
        """An intermediate of the last call, e.g. view("topk_ids", M*K, torch.int32)."""
        off = getattr(self.layout, name)
        nbytes = count * torch.empty(0, dtype=dtype).element_size()
        return self.workspace[off: off + nbytes].view(dtype)


# Which device memory holds re-tiled weights. The mark belongs to the STORAGE (keyed by the address of
# torch's StorageImpl, dropped when the storage dies), not to a tensor object: views, `.data`, `.detach()`,
# `.t()` and a Parameter wrapped around the same memory all see it.
_TILED: dict[int, tuple[int, int]] = {}  # storage -> (n, bytes of k) of the tiles it holds


def _mark_tiled(w: torch.Tensor, n: int, k_bytes: int) -> None:
    storage = w.untyped_storage()
    key = storage._cdata
    _TILED[key] = (n, k_bytes)
    weakref.finalize(storage, _TILED.pop, key, None)


def is_tiled(w: torch.Tensor) -> bool:
    """True if the memory behind this tensor was re-arranged by tile_int8_weights_ (whatever view of it
    the tensor is)."""
    return w.untyped_storage()._cdata in _TILED


def weight_layout(w: torch.Tensor) -> int:
    """KMOE_W_TILED or KMOE_W_ROWMAJOR for a weight handed to an operator. A tensor over tiled memory must
    be the contiguous [..., n, k] tensor that was tiled (or a leading-dimension slice of it): any other
    view (a transpose, a column slice) would read scrambled values, so it is refused."""
    tiles = _TILED.get(w.untyped_storage()._cdata)
    if tiles is None:
        return L.KMOE_W_ROWMAJOR
    if w.dim() < 2 or not w.is_contiguous() or (w.shape[-2], w.shape[-1] * w.element_size()) != tiles:
        raise ValueError(f"this tensor {tuple(w.shape)} is a view of weights that were re-tiled as "
                         f"[..., {tiles[0]}, {tiles[1]} bytes]: pass the contiguous [..., n, k] tensor itself")
    return L.KMOE_W_TILED


_TILEABLE = (torch.int8, torch.uint8, torch.float8_e4m3fn, torch.bfloat16, torch.float16)


def tile_int8_weights_(w: torch.Tensor) -> bool:
    """Re-arranges weights [..., n, k] (int8, e4m3 codes, or bf16 — the kernel moves BYTES: a
    1 KB block is 16 channels x 64 bytes of K) IN PLACE into the MFMA-ready blocks of
    kmoe_tile_weights_i8 (one expert at a time through a scratch copy) and marks the memory as tiled.
    Returns False and leaves the tensor alone when the shape does not allow it (n % 16,
    64 bytes of K)."""
    data = w.data
    if data.dtype not in _TILEABLE or not data.is_cuda or not data.is_contiguous():
        return False
    n, k = data.shape[-2], data.shape[-1] * data.element_size()  # k in bytes
    if n % 16 or k % 64:
        return False
    if is_tiled(w):
        return True
    flat = data.view(torch.int8).view(-1, n, k)
    tmp = torch.empty_like(flat[0])
    for e in range(flat.shape[0]):
        L.check(L.lib.kmoe_tile_weights_i8(L.ptr(flat[e]), L.ptr(tmp), 1, n, k, L.stream()))
        flat[e].copy_(tmp)
    _mark_tiled(data, n, k)
    return True


_SCALES_FRAG16: dict = {}  # storage -> (n, groups) of 4-bit group scales re-arranged by tile_w4_scales_


def tile_w4_scales_(scale: torch.Tensor) -> bool:
    """Re-arranges the group scales [E, n, groups] of packed 4-bit weights IN PLACE (one expert at a time through
    a scratch copy) into the per-16-channel [groups][16] form of kmoe_tile_scales_w4 and marks the memory.
    Returns False and leaves the tensor alone when the shape does not allow it."""
    data = scale.data
    if data.dtype not in (torch.bfloat16, torch.float16) or not data.is_cuda or not data.is_contiguous() or data.dim() != 3:
        return False
    E, n, groups = data.shape
    if n % 16:
        return False
    key = data.untyped_storage()._cdata
    if key in _SCALES_FRAG16:
        return True
    tmp = torch.empty_like(data[0])
    for e in range(E):
        L.check(L.lib.kmoe_tile_scales_w4(L.ptr(data[e]), L.ptr(tmp), 1, n, groups, L.stream()))
        data[e].copy_(tmp)
    storage = data.untyped_storage()
    _SCALES_FRAG16[key] = (n, groups)
    weakref.finalize(storage, _SCALES_FRAG16.pop, key, None)
    return True


def scale_layout(scale: torch.Tensor) -> int:
    """KMOE_S_FRAG16 or KMOE_S_ROWMAJOR for the group scales of packed 4-bit weights handed to an operator; as
    for weights, only the contiguous [..., n, groups] tensor that was re-arranged may stand for its memory."""
    dims = _SCALES_FRAG16.get(scale.untyped_storage()._cdata)
    if dims is None:
        return L.KMOE_S_ROWMAJOR
    if scale.dim() < 2 or not scale.is_contiguous() or tuple(scale.shape[-2:]) != dims:
        raise ValueError(f"this tensor {tuple(scale.shape)} is a view of group scales that were re-arranged as "
                         f"[..., {dims[0]}, {dims[1]}]: pass the contiguous tensor itself")
    return L.KMOE_S_FRAG16


def rowmajor_w4_scales(scale: torch.Tensor) -> torch.Tensor:
    """A row-major [..., n, groups] COPY of group scales, undoing tile_w4_scales_ if it was applied."""
    if scale.untyped_storage()._cdata not in _SCALES_FRAG16:
        return scale.data.clone()
    n, groups = scale.shape[-2:]
    lead = scale.shape[:-2]
    return scale.data.reshape(-1, n // 16, groups, 16).permute(0, 1, 3, 2).reshape(*lead, n, groups).contiguous()


def can_tile(w: torch.Tensor) -> bool:
    d = w.data
    return (d.dtype in _TILEABLE and d.is_cuda and d.is_contiguous() and d.shape[-2] % 16 == 0
            and (d.shape[-1] * d.element_size()) % 64 == 0)


def tile_pair_(w13: torch.Tensor, w2: torch.Tensor) -> bool:
    """Tiles the two weights of an MLP, or neither (a launch takes one layout for both)."""
    if not (can_tile(w13) and can_tile(w2)):
        return False
    return tile_int8_weights_(w13) and tile_int8_weights_(w2)


def rowmajor_int8_weights(w: torch.Tensor) -> torch.Tensor:
    """A row-major [..., n, k] COPY of int8 weights, undoing tile_int8_weights_ if it was applied."""
    if not is_tiled(w):
        return w.data.clone()
    n, k = w.shape[-2], w.shape[-1] * w.element_size()  # k in bytes
    lead = w.shape[:-2]
    t = w.data.view(torch.int8).reshape(-1, n // 16, k // 64, 4, 16, 16).permute(0, 1, 4, 2, 3, 5)
    return t.reshape(*lead, n, k).contiguous().view(w.dtype)


_WEIGHT_DTYPE = {L.KMOE_FMT_INT8: (torch.int8,), L.KMOE_FMT_FP8_BLOCK: (torch.float8_e4m3fn, torch.uint8),
                 L.KMOE_FMT_BF16: (torch.bfloat16, torch.float16), L.KMOE_FMT_W4A16: (torch.uint8,)}


def make_moe_plan(fmt: int, x: torch.Tensor, logits: torch.Tensor, out: torch.Tensor, top_k: int,
                  w13: torch.Tensor, w2: torch.Tensor, w13_aux: Optional[torch.Tensor], w2_aux: Optional[torch.Tensor],
                  scoring_func: str = "softmax", renormalize: bool = True, num_expert_group: Optional[int] = None,
                  topk_group: Optional[int] = None, routed_scaling_factor: float = 1.0,
                  e_score_correction_bias: Optional[torch.Tensor] = None, shared_expert=None, out_scale: float = 1.0,
                  stage_events=None, w_layout: Optional[int] = None,
                  router_weight: Optional[torch.Tensor] = None, w13_bias: Optional[torch.Tensor] = None,
                  w2_bias: Optional[torch.Tensor] = None, activation: str = "silu", act_alpha: float = 1.702,
                  act_limit: float = 7.0, group_size: Optional[int] = None, tile_variant: int = 0,
                  shared_scale: float = 1.0, first_expert: int = 0, side_stream: bool = False) -> MoEPlan:
    """x bf16 [M,H] (or float16 with int8 or unquantized weights, the latter then float16 too), logits f32 [M,E], out [M,H] like x; w13 [E,2I,H], w2 [E,H,I] in the
    format's dtype; w13_aux/w2_aux: per-channel maxes (int8) or block scales (fp8), None for bf16.
    shared_expert: (ws13 [2Is,H], ws13_aux, ws2 [H,Is], ws2_aux) in the same format.
    logits may be None when router_weight (bf16 [E,H], the gate projection) is given: the
    layer then computes the router logits itself. bf16 only: w13_bias [E,2I] / w2_bias [E,H] (bf16)
    and activation "swigluoai" (gate and up rows of w13 interleaved) select the expert-bias branch.
    KMOE_FMT_W4A16: w13 [E,2I,H/2] and w2 [E,H,I/2] uint8 (two 4-bit codes per byte), tiled;
    w13_aux/w2_aux their group scales [E,2I,H/group_size], [E,H,I/group_size] in x's dtype.
    shared_scale multiplies the shared expert's output before it is added (the float16 form of the caller's
    epilogue, models/deepseek_v2.py:286-292). tile_variant: a tuning variant of the int8 / fp8 tile kernel for the routed GEMMs (kmoe_moe_args.tile_variant).
    An expert-parallel share (ops/_kunlun_ops.py:640-696): logits [M,E_global] (correction bias [E_global], router
    weight [E_global,H]) with more experts than the weights hold, and first_expert = ep_rank * E: the routing runs
    over all of them, the pairs routed to [first_expert, first_expert + E) are computed, the others add nothing.
    side_stream: let a shared expert that cannot ride in the routed launches run on the library's second stream
    beside them (KMOE_FLAG_SIDE_STREAM); by default every launch goes to the current stream.
    The plan is bound to the stream that is current when it is built and refuses to run on another one; a plan that
    a HIP graph is to replay must be built INSIDE the capture (a plan built before torch.cuda.graph() sits on
    another stream than the capture's and raises when called inside it)."""
    if scoring_func not in ("softmax", "sigmoid"):
        raise ValueError(f"Unsupported scoring_func: {scoring_func}")
    if logits is None and router_weight is None:
        raise ValueError("moe plan: either router logits or the router weight is needed")
    tensors = [x, logits, out, w13, w2, w13_aux, w2_aux, e_score_correction_bias, router_weight]
    L.require_device(*tensors)
    L.require_contig(*tensors)
    dt = L.act_dtype(x, "moe plan")
    if fmt == L.KMOE_FMT_BF16 and w13.dtype != x.dtype:
        raise ValueError(f"moe plan: unquantized weights ({w13.dtype}) must have the activations' dtype ({x.dtype})")
    if fmt == L.KMOE_FMT_BF16 and dt == L.KMOE_DT_F16 and (w13_bias is not None or w2_bias is not None
                                                           or activation == "swigluoai"):
        raise NotImplementedError("moe plan: expert biases and swigluoai are built for bfloat16 only")
    if out.dtype != x.dtype or (logits is not None and logits.dtype != torch.float32):
        raise ValueError("moe plan: out must have x's dtype and logits must be float32")
    if w13.dtype not in _WEIGHT_DTYPE[fmt] or w2.dtype != w13.dtype:
        raise ValueError(f"moe plan: weight dtype {w13.dtype} does not fit the layer format")
    E, two_i, H = w13.shape
    w4 = fmt == L.KMOE_FMT_W4A16
    if w4:
        H *= 2  # two codes per byte
    M = x.shape[0]
    Eg = logits.shape[-1] if logits is not None else router_weight.shape[0]  # experts the routing runs over
    if tuple(x.shape) != (M, H) or tuple(out.shape) != (M, H) or (logits is not None and tuple(logits.shape) != (M, Eg)):
        raise ValueError("moe plan: x/out must be [M,H] and logits [M,E]")
    if logits is None and (router_weight.dtype != x.dtype or tuple(router_weight.shape) != (Eg, H)):
        raise ValueError("moe plan: router_weight must be [E,H] in the activations' dtype")
    if Eg < E or first_expert < 0 or first_expert + E > Eg or (Eg == E and first_expert):
        raise ValueError(f"moe plan: the weights' {E} experts from {first_expert} on are not among the {Eg} the "
                         "routing runs over")
    if e_score_correction_bias is not None and e_score_correction_bias.numel() != Eg:
        raise ValueError(f"moe plan: the correction bias must have one entry per routed expert ({Eg})")
    if tuple(w2.shape) != (E, H, two_i // (4 if w4 else 2)):
        raise ValueError("moe plan: w2 must be [E,H,I] for w13 [E,2I,H]")
    if w4:
        gs = int(group_size or 0)
        if w13_aux is None or w2_aux is None or w13_aux.dtype != x.dtype or w2_aux.dtype != x.dtype:
            raise ValueError("moe plan: 4-bit weights need group scales in the activations' dtype")
        if gs < 32 or gs % 32 or H % gs or (two_i // 2) % gs:
            raise ValueError(f"moe plan: group_size={group_size} must be a multiple of 32 dividing H and I")
        if tuple(w13_aux.shape) != (E, two_i, H // gs) or tuple(w2_aux.shape) != (E, H, two_i // 2 // gs):
            raise ValueError("moe plan: group scales must be [E,2I,H/group_size] and [E,H,I/group_size]")
        if shared_expert is not None:
            raise NotImplementedError("moe plan: no shared expert with 4-bit weights")
    a = L.MoEArgs()
    a.M, a.H, a.E, a.K, a.I = M, H, E, int(top_k), two_i // 2
    a.E_global, a.first_expert = (Eg, int(first_expert)) if Eg > E else (0, 0)
    a.format = fmt
    a.scoring = L.KMOE_SCORE_SOFTMAX if scoring_func == "softmax" else L.KMOE_SCORE_SIGMOID
    a.renormalize = int(bool(renormalize))
    a.n_group = int(num_expert_group or 1)
    a.topk_group = int(topk_group or 1)
    a.routed_scale = float(routed_scaling_factor)
    a.logits = 0 if logits is None else logits.data_ptr()
    a.w_gate = 0 if logits is not None or router_weight is None else router_weight.data_ptr()
    a.bias = 0 if e_score_correction_bias is None else e_score_correction_bias.data_ptr()
    a.x = x.data_ptr()
    a.w13, a.w2 = w13.data_ptr(), w2.data_ptr()
    if w4:
        a.w13_scale, a.w2_scale, a.group_size = w13_aux.data_ptr(), w2_aux.data_ptr(), int(group_size)
        a.w_scale_layout = scale_layout(w13_aux)
        if scale_layout(w2_aux) != a.w_scale_layout:
            raise ValueError("moe plan: the group scales of w13 and w2 must be in one layout (tile_w4_scales_ on both, or none)")
    else:
        a.w13_max = 0 if w13_aux is None else w13_aux.data_ptr()
        a.w2_max = 0 if w2_aux is None else w2_aux.data_ptr()
    keep = list(tensors)
    if shared_expert is not None:
        ws13, ws13_aux, ws2, ws2_aux = shared_expert
        L.require_device(ws13, ws13_aux, ws2, ws2_aux)
        L.require_contig(ws13, ws13_aux, ws2, ws2_aux)
        a.I_shared = ws13.shape[0] // 2
        a.ws13, a.ws2 = ws13.data_ptr(), ws2.data_ptr()
        a.ws13_max = 0 if ws13_aux is None else ws13_aux.data_ptr()
        a.ws2_max = 0 if ws2_aux is None else ws2_aux.data_ptr()
        keep.append(shared_expert)
    if activation not in ("silu", "swigluoai"):
        raise ValueError(f"Unsupported activation: {activation}")
    if (w13_bias is not None or w2_bias is not None or activation == "swigluoai") and fmt != L.KMOE_FMT_BF16:
        raise NotImplementedError("moe plan: expert biases and swigluoai go with bf16 weights only")
    for b, cols in ((w13_bias, two_i), (w2_bias, H)):
        if b is not None:
            L.require_device(b)
            L.require_contig(b)
            if b.dtype != torch.bfloat16 or tuple(b.shape) != (E, cols):
                raise ValueError(f"moe plan: expert bias must be bfloat16 [{E},{cols}]")
            keep.append(b)
    a.w13_bias = 0 if w13_bias is None else w13_bias.data_ptr()
    a.w2_bias = 0 if w2_bias is None else w2_bias.data_ptr()
    a.activation = L.KMOE_ACT_SWIGLUOAI if activation == "swigluoai" else L.KMOE_ACT_SWIGLU
    a.act_alpha, a.act_limit = float(act_alpha), float(act_limit)
    a.out_scale = float(out_scale)
    a.tile_variant = int(tile_variant)
    a.act_dtype = dt
    a.shared_scale = float(shared_scale)
    a.flags = L.KMOE_FLAG_SIDE_STREAM if side_stream else 0
    a.out = out.data_ptr()
    if w_layout is None:  # per group of weights: tiled if both of its tensors have been tiled
        w_layout = L.KMOE_W_TILED if is_tiled(w13) and is_tiled(w2) else L.KMOE_W_ROWMAJOR
        if w_layout == L.KMOE_W_ROWMAJOR and (is_tiled(w13) or is_tiled(w2)):
            raise ValueError("moe plan: w13 and w2 must be either both tiled or both row-major")
    ws_layout = L.KMOE_W_ROWMAJOR
    if shared_expert is not None:
        ws_tiled = [is_tiled(shared_expert[0]), is_tiled(shared_expert[2])]
        if any(ws_tiled) and not all(ws_tiled):
            raise ValueError("moe plan: the shared expert's two weights must be either both tiled or both row-major")
        ws_layout = L.KMOE_W_TILED if all(ws_tiled) else L.KMOE_W_ROWMAJOR
    a.ws_layout = int(ws_layout)
    a.w_layout = int(w_layout)
    if stage_events is not None:
        a.stage_events = stage_events
        keep.append(stage_events)
    lay = L.MoELayout()
    L.check(L.lib.kmoe_moe_workspace_layout(a, lay))
    stream_id = _current_stream_id(x.device)
    if torch.cuda.is_current_stream_capturing():
        # memory allocated during a capture belongs to the graph's pool: the plan owns this buffer, it is
        # not shared with later plans
        ws = torch.empty(max(int(lay.total_bytes), 1), dtype=torch.uint8, device=x.device)
    else:
        ws = WORKSPACE.get(lay.total_bytes, x.device, stream_id)
    return MoEPlan(a, lay, ws, keep, stream_id)
