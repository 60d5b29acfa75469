"""``torch.autograd.Function`` front end of the HIP attention path.

``PackedDocAttention`` takes what maester's ``GemmaAttention.forward`` holds right after the qkv
split (maester/models/gemma/model.py:358-364) -- ``xq [B,S,Hq,D]``, ``xk/xv [B,S,Hkv,D]`` (strided
views are fine), the stored QK-norm weights, RoPE tables, ``position_ids``, ``document_ids`` -- and
returns the attention output in ``[B,S,Hq,D]``, i.e. model.py:366-438 in one call.  The two stages
are also exposed on their own (``qk_norm_rope``, ``doc_masked_attention``).

Everything runs in the HIP library; there is no PyTorch fallback.
"""
from __future__ import annotations

import warnings
from ctypes import byref

import torch

from . import _lib
from .tile_map import TileMap, build_tile_map


# ------------------------------------------------------------------------------------------------
# raw stage wrappers (no autograd)
# ------------------------------------------------------------------------------------------------
def _check_qkv(xq, xk, xv=None):
    if xq.dim() != 4 or xk.dim() != 4:
        raise ValueError("expected [B,S,H,D] tensors")
    B, S, Hq, D = xq.shape
    if xk.shape[0] != B or xk.shape[1] != S or xk.shape[3] != D:
        raise ValueError(f"q {tuple(xq.shape)} and k {tuple(xk.shape)} disagree")
    if xv is not None and xv.shape != xk.shape:
        raise ValueError(f"k {tuple(xk.shape)} and v {tuple(xv.shape)} disagree")
    if xk.dtype != xq.dtype or (xv is not None and xv.dtype != xq.dtype):
        raise TypeError("q, k, v must share one dtype")
    return B, S, Hq, xk.shape[2], D


def _rowmajor(t: torch.Tensor) -> torch.Tensor:
    return t if t.stride(-1) == 1 else t.contiguous()


def _ids(t: torch.Tensor | None, B: int, S: int, name: str):
    if t is None:
        return None
    if tuple(t.shape) != (B, S):
        raise ValueError(f"{name} shape {tuple(t.shape)} != {(B, S)}")
    return t.detach().to(torch.long).contiguous()


def prologue_forward(xq, xk, q_w, k_w, cos, sin, position_ids, eps=1e-6, add_unit_offset=True):
    """Returns (q, k, q_rstd, k_rstd); q/k are new contiguous [B,S,H,D] tensors."""
    _lib.require_gpu(xq, "prologue_forward")
    B, S, Hq, Hkv, D = _check_qkv(xq, xk)
    xq, xk = _rowmajor(xq), _rowmajor(xk)
    dev = xq.device
    q = torch.empty((B, S, Hq, D), dtype=xq.dtype, device=dev)
    k = torch.empty((B, S, Hkv, D), dtype=xk.dtype, device=dev)
    qw = None if q_w is None else q_w.detach().float().contiguous()
    kw = None if k_w is None else k_w.detach().float().contiguous()
    q_rstd = torch.empty((B, S, Hq), dtype=torch.float32, device=dev) if qw is not None else None
    k_rstd = torch.empty((B, S, Hkv), dtype=torch.float32, device=dev) if kw is not None else None
    pos = _ids(position_ids, B, S, "position_ids")
    cos, sin = cos.contiguous(), sin.contiguous()
    if cos.dtype != torch.float32 or cos.shape != sin.shape or cos.shape[-1] != D // 2:
        raise ValueError(f"rope tables must be fp32 [P,{D // 2}], got {tuple(cos.shape)} {cos.dtype}")
    with torch.cuda.device(dev):
        rc = _lib.lib().ma_prologue_fwd(
            byref(_lib.tensor4(xq)), byref(_lib.tensor4(xk)), byref(_lib.tensor4(q)), byref(_lib.tensor4(k)),
            _lib.ptr(qw), _lib.ptr(kw), _lib.ptr(cos), _lib.ptr(sin), cos.shape[0], _lib.ptr(pos), float(eps),
            1 if add_unit_offset else 0, _lib.ptr(q_rstd), _lib.ptr(k_rstd), _lib.dtype_code(xq.dtype), B, S, Hq,
            Hkv, D, _lib.current_stream(dev))
    _lib.check(rc)
    return q, k, q_rstd, k_rstd


def prologue_backward(xq, xk, dq, dk, q_w, k_w, cos, sin, position_ids, q_rstd, k_rstd, add_unit_offset=True,
                      inplace=False):
    """Gradients w.r.t. the prologue inputs: (dxq, dxk, dq_w fp32|None, dk_w fp32|None).
    With ``inplace`` the incoming ``dq``/``dk`` buffers are overwritten with the result."""
    B, S, Hq, Hkv, D = _check_qkv(dq, dk)
    dev = dq.device
    dq, dk = _rowmajor(dq), _rowmajor(dk)
    dxq = dq if inplace else torch.empty((B, S, Hq, D), dtype=dq.dtype, device=dev)
    dxk = dk if inplace else torch.empty((B, S, Hkv, D), dtype=dk.dtype, device=dev)
    L = _lib.lib()
    qw = None if q_w is None else q_w.detach().float().contiguous()
    kw = None if k_w is None else k_w.detach().float().contiguous()
    dqw = torch.empty(D, dtype=torch.float32, device=dev) if qw is not None else None
    dkw = torch.empty(D, dtype=torch.float32, device=dev) if kw is not None else None
    ws_bytes = L.ma_prologue_bwd_workspace_bytes(B, S, Hq, Hkv, D)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
    pos = _ids(position_ids, B, S, "position_ids")
    xq_d = byref(_lib.tensor4(_rowmajor(xq))) if qw is not None else None
    xk_d = byref(_lib.tensor4(_rowmajor(xk))) if kw is not None else None
    with torch.cuda.device(dev):
        rc = L.ma_prologue_bwd(
            xq_d, xk_d, byref(_lib.tensor4(dq)), byref(_lib.tensor4(dk)), byref(_lib.tensor4(dxq)),
            byref(_lib.tensor4(dxk)), _lib.ptr(qw), _lib.ptr(kw), _lib.ptr(cos), _lib.ptr(sin), cos.shape[0],
            _lib.ptr(pos), 1 if add_unit_offset else 0, _lib.ptr(q_rstd), _lib.ptr(k_rstd), _lib.ptr(dqw),
            _lib.ptr(dkw), _lib.ptr(ws), ws_bytes, _lib.dtype_code(dq.dtype), B, S, Hq, Hkv, D,
            _lib.current_stream(dev))
    _lib.check(rc)
    return dxq, dxk, dqw, dkw


def _resolve_map(tile_map, document_ids, B, S, causal, window, device) -> TileMap:
    if tile_map is None:
        return build_tile_map(document_ids, B, S, causal, window, device=device)
    if tile_map.seq_len != S or tile_map.kv_num_blocks.shape[0] != B:
        raise ValueError("tile_map was built for another batch/sequence shape")
    if tile_map.causal != bool(causal) or tile_map.window != window:
        raise ValueError("tile_map was built for another mask (causal/sliding_window)")
    return tile_map


def attention_forward(q, k, v, tile_map: TileMap, document_ids, scale, causal=True, window=None):
    """Returns (out [B,S,Hq,D], lse [B,Hq,S] fp32)."""
    _lib.require_gpu(q, "attention_forward")
    B, S, Hq, Hkv, D = _check_qkv(q, k, v)
    q, k, v = _rowmajor(q), _rowmajor(k), _rowmajor(v)
    dev = q.device
    out = torch.empty((B, S, Hq, D), dtype=q.dtype, device=dev)
    lse = torch.empty((B, Hq, S), dtype=torch.float32, device=dev)
    doc = _ids(document_ids, B, S, "document_ids")
    cs = tile_map.c_struct()
    tile_map.order_on_current_stream(dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().ma_attn_fwd(
            byref(_lib.tensor4(q)), byref(_lib.tensor4(k)), byref(_lib.tensor4(v)), byref(_lib.tensor4(out)),
            _lib.ptr(lse), byref(cs), _lib.ptr(doc), 1 if causal else 0, -1 if window is None else int(window),
            float(scale), _lib.dtype_code(q.dtype), B, S, Hq, Hkv, D, _lib.current_stream(dev))
    _lib.check(rc)
    return out, lse


# Largest workspace the backward takes for handing dS from the dK/dV kernel to the dQ kernel (bytes), as a
# fraction of the memory that is available when the choice is made; above it the dQ kernel recomputes S and dP.
DS_WORKSPACE_LIMIT = 64 << 30
DS_WORKSPACE_FREE_FRACTION = 0.5
# The two backward paths agree to rounding, not bit for bit, so the choice between them must not move while a
# run is under way.  ``HAND_OVER_DEFAULT`` True / False fixes it for the process; None decides it ONCE per
# (device, batch shape) from the memory available at that moment and keeps the decision for every later tile
# map of that shape (``_HAND_OVER_DECISIONS``).  A decision for the hand-over whose workspace then cannot be
# allocated is withdrawn for good, with a warning -- never silently and never back and forth.
HAND_OVER_DEFAULT: bool | None = None
_HAND_OVER_DECISIONS: dict = {}


def _available_bytes(device) -> int:
    """Memory a new torch allocation can draw on: what the driver reports free plus what torch's caching
    allocator has reserved but not handed out."""
    if torch.device(device).type != "cuda":
        return 0
    free = torch.cuda.mem_get_info(device)[0]
    cached = torch.cuda.memory_reserved(device) - torch.cuda.memory_allocated(device)
    return int(free + max(cached, 0))


def decide_hand_over(B, S, Hq, dtype, tile_map: TileMap | None, hand_over=None) -> bool:
    """Whether ``attention_backward`` hands dS from the dK/dV kernel to the dQ kernel for this tile map.
    Explicit ``hand_over`` wins, then ``HAND_OVER_DEFAULT``, then the decision already taken for this map or
    for this (device, B, S, Hq); only the first call for a shape looks at the memory."""
    if dtype != torch.bfloat16 or tile_map is None or tile_map.tile_slot is None:
        return False
    if hand_over is None:
        hand_over = HAND_OVER_DEFAULT
    if hand_over is not None:
        return bool(hand_over)
    if tile_map._hand_over is not None:
        return tile_map._hand_over
    dev = tile_map.tile_slot.device
    key = (dev.index, B, S, Hq)
    if key not in _HAND_OVER_DECISIONS:
        large = _lib.lib().ma_attn_bwd_ds_workspace_bytes(B, S, Hq, tile_map.visited_tiles())
        ok = 0 < large <= DS_WORKSPACE_LIMIT and large <= DS_WORKSPACE_FREE_FRACTION * _available_bytes(dev)
        _HAND_OVER_DECISIONS[key] = bool(ok)
    tile_map._hand_over = _HAND_OVER_DECISIONS[key]
    return tile_map._hand_over


def backward_workspace_bytes(B, S, Hq, Hkv, D, dtype, hand_over=None, tile_map: TileMap | None = None) -> int:
    """Workspace of ``attention_backward``: delta alone, or delta plus one 32 KB dS slot per query head and
    VISITED tile of ``tile_map`` (bf16 only) when the hand-over is taken (``decide_hand_over``)."""
    L = _lib.lib()
    small = L.ma_attn_bwd_workspace_bytes(B, S, Hq, Hkv, D)
    if not decide_hand_over(B, S, Hq, dtype, tile_map, hand_over):
        return small
    large = L.ma_attn_bwd_ds_workspace_bytes(B, S, Hq, tile_map.visited_tiles())
    return large if large else small


def attention_backward(q, k, v, out, dout, lse, tile_map: TileMap, document_ids, scale, causal=True, window=None,
                       stages=_lib.MA_BWD_ALL, buffers=None, hand_over=None):
    """Returns (dq, dk, dv) as new contiguous [B,S,H,D] tensors.  ``stages`` restricts the call to
    some of its kernels (see ``ma_attn_bwd_stages``); ``buffers`` = (dq, dk, dv, workspace) reuses
    tensors from an earlier call, which staged calls need.  ``hand_over``: see ``decide_hand_over``.
    The path the call took is left in ``tile_map.last_backward_path`` ("hand_over" / "recompute")."""
    B, S, Hq, Hkv, D = _check_qkv(q, k, v)
    q, k, v, out, dout = (_rowmajor(t) for t in (q, k, v, out, dout))
    dev = q.device
    L = _lib.lib()
    small = L.ma_attn_bwd_workspace_bytes(B, S, Hq, Hkv, D)
    if buffers is None:
        dq = torch.empty((B, S, Hq, D), dtype=q.dtype, device=dev)
        dk = torch.empty((B, S, Hkv, D), dtype=q.dtype, device=dev)
        dv = torch.empty((B, S, Hkv, D), dtype=q.dtype, device=dev)
        ws_bytes = backward_workspace_bytes(B, S, Hq, Hkv, D, q.dtype, hand_over, tile_map)
        try:
            ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
        except torch.cuda.OutOfMemoryError:
            if ws_bytes <= small or hand_over is True or HAND_OVER_DEFAULT is True:
                raise                            # (an explicit request for the hand-over is not overruled)
            # the dS slots did not fit after all: withdraw the decision for this shape, for the rest of the process
            warnings.warn(f"maester_amd: no room for the {ws_bytes >> 20} MiB dS workspace of the attention backward; "
                          f"B={B} S={S} Hq={Hq} recompute S and dP in the dQ kernel from now on (gradients agree with "
                          "the hand-over path to rounding, not bit for bit)", RuntimeWarning, stacklevel=2)
            _HAND_OVER_DECISIONS[(dev.index, B, S, Hq)] = False
            tile_map._hand_over = False
            ws_bytes = small
            ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
    else:
        dq, dk, dv, ws = buffers
        ws_bytes = ws.numel() * ws.element_size()
    doc = _ids(document_ids, B, S, "document_ids")
    cs = tile_map.c_struct()
    tile_map.order_on_current_stream(dev)
    with torch.cuda.device(dev):
        rc = L.ma_attn_bwd_stages(
            byref(_lib.tensor4(q)), byref(_lib.tensor4(k)), byref(_lib.tensor4(v)), byref(_lib.tensor4(out)),
            byref(_lib.tensor4(dout)), _lib.ptr(lse), byref(_lib.tensor4(dq)), byref(_lib.tensor4(dk)),
            byref(_lib.tensor4(dv)), byref(cs), _lib.ptr(doc), 1 if causal else 0,
            -1 if window is None else int(window), float(scale), _lib.ptr(ws), ws_bytes,
            _lib.dtype_code(q.dtype), B, S, Hq, Hkv, D, int(stages), _lib.current_stream(dev))
    _lib.check(rc)
    # (the library takes the hand-over when the map carries the numbering and the workspace holds every visited tile)
    vis = tile_map._visited or 0
    took = q.dtype == torch.bfloat16 and tile_map.tile_slot is not None and vis > 0 and \
        ws_bytes >= L.ma_attn_bwd_ds_workspace_bytes(B, S, Hq, vis)
    tile_map.last_backward_path = "hand_over" if took else "recompute"
    return dq, dk, dv


# ------------------------------------------------------------------------------------------------
# autograd
# ------------------------------------------------------------------------------------------------
def _wgrad(g, w):
    return None if (g is None or w is None) else g.to(w.dtype)


class _QKNormRope(torch.autograd.Function):
    @staticmethod
    def forward(ctx, xq, xk, q_w, k_w, cos, sin, position_ids, eps, add_unit_offset):
        q, k, q_rstd, k_rstd = prologue_forward(xq, xk, q_w, k_w, cos, sin, position_ids, eps, add_unit_offset)
        ctx.save_for_backward(xq, xk, q_w, k_w, cos, sin, position_ids, q_rstd, k_rstd)
        ctx.add_unit_offset = add_unit_offset
        return q, k

    @staticmethod
    def backward(ctx, dq, dk):
        xq, xk, q_w, k_w, cos, sin, position_ids, q_rstd, k_rstd = ctx.saved_tensors
        dxq, dxk, dqw, dkw = prologue_backward(xq, xk, dq, dk, q_w, k_w, cos, sin, position_ids, q_rstd, k_rstd,
                                               ctx.add_unit_offset)
        return dxq, dxk, _wgrad(dqw, q_w), _wgrad(dkw, k_w), None, None, None, None, None


class _DocMaskedAttention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, document_ids, scale, causal, window, tile_map):
        B, S = q.shape[0], q.shape[1]
        tile_map = _resolve_map(tile_map, document_ids, B, S, causal, window, q.device)
        out, lse = attention_forward(q, k, v, tile_map, document_ids, scale, causal, window)
        ctx.save_for_backward(q, k, v, out, lse, document_ids)
        ctx.tile_map, ctx.scale, ctx.causal, ctx.window = tile_map, scale, causal, window
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, out, lse, document_ids = ctx.saved_tensors
        dq, dk, dv = attention_backward(q, k, v, out, dout, lse, ctx.tile_map, document_ids, ctx.scale, ctx.causal,
                                        ctx.window)
        return dq, dk, dv, None, None, None, None, None


# What the autograd Function keeps for its backward, beyond its inputs (which autograd holds anyway):
#   "all"        q, k after the prologue, the output, LSE, the norms' rstd -- nothing is redone
#   "attention"  the output and LSE only; the prologue (elementwise, one pass) is redone.  This is
#                what the reference's op-level selective checkpointing keeps: outputs of matmuls and
#                attention, everything elementwise recomputed (maester/parallelisms/parallelize_gemma.py:181-232)
#   "inputs"     nothing; prologue and attention forward are redone (full checkpointing of the op,
#                parallelize_gemma.py:195-196, without re-running the surrounding module)
SAVE_POLICIES = ("all", "attention", "inputs")


class PackedDocAttention(torch.autograd.Function):
    """QK-RMSNorm -> RoPE -> document-masked GQA attention, forward and backward in HIP.

    ``apply(xq, xk, xv, q_norm_w, k_norm_w, rope_cos, rope_sin, position_ids, document_ids, scale,
    causal, sliding_window, eps, tile_map)`` -> ``out [B,S,Hq,D]`` (dtype of ``xq``).

    ``q_norm_w`` / ``k_norm_w`` are the *stored* Gemma parameters (effective scale ``1 + w``,
    maester/models/gemma/model.py:146,163-164) or ``None`` (``use_qk_norm=False``).  Gradients are
    returned for xq, xk, xv and the two weights."""

    @staticmethod
    def forward(ctx, xq, xk, xv, q_norm_w, k_norm_w, rope_cos, rope_sin, position_ids, document_ids, scale,
                causal=True, sliding_window=None, eps=1e-6, tile_map=None, save="all"):
        if save not in SAVE_POLICIES:
            raise ValueError(f"save={save!r}: expected one of {SAVE_POLICIES}")
        B, S = xq.shape[0], xq.shape[1]
        tile_map = _resolve_map(tile_map, document_ids, B, S, causal, sliding_window, xq.device)
        q, k, q_rstd, k_rstd = prologue_forward(xq, xk, q_norm_w, k_norm_w, rope_cos, rope_sin, position_ids, eps,
                                                True)
        out, lse = attention_forward(q, k, xv, tile_map, document_ids, scale, causal, sliding_window)
        kept = {"all": (q, k, out, lse, q_rstd, k_rstd), "attention": (out, lse), "inputs": ()}[save]
        ctx.save_for_backward(xq, xk, xv, q_norm_w, k_norm_w, rope_cos, rope_sin, position_ids, document_ids, *kept)
        ctx.tile_map, ctx.scale, ctx.causal, ctx.window, ctx.eps, ctx.save = tile_map, scale, causal, sliding_window, eps, save
        return out

    @staticmethod
    def backward(ctx, dout):
        xq, xk, xv, q_w, k_w, cos, sin, position_ids, document_ids = ctx.saved_tensors[:9]
        kept = ctx.saved_tensors[9:]
        if ctx.save == "all":
            q, k, out, lse, q_rstd, k_rstd = kept
        else:  # the prologue is one HBM-bound pass: cheaper to redo than to keep q and k
            q, k, q_rstd, k_rstd = prologue_forward(xq, xk, q_w, k_w, cos, sin, position_ids, ctx.eps, True)
            if ctx.save == "attention":
                out, lse = kept
            else:
                out, lse = attention_forward(q, k, xv, ctx.tile_map, document_ids, ctx.scale, ctx.causal, ctx.window)
        dq, dk, dv = attention_backward(q, k, xv, out, dout, lse, ctx.tile_map, document_ids, ctx.scale, ctx.causal,
                                        ctx.window)
        dxq, dxk, dqw, dkw = prologue_backward(xq, xk, dq, dk, q_w, k_w, cos, sin, position_ids, q_rstd, k_rstd, True,
                                               inplace=True)
        return (dxq, dxk, dv, _wgrad(dqw, q_w), _wgrad(dkw, k_w), None, None, None, None, None, None, None, None,
                None, None)


def packed_doc_attention(xq, xk, xv, q_norm_w=None, k_norm_w=None, rope_cos=None, rope_sin=None, position_ids=None,
                         document_ids=None, scale=None, causal=True, sliding_window=None, eps=1e-6, tile_map=None,
                         save="all"):
    """Keyword-friendly wrapper of ``PackedDocAttention.apply``; ``scale`` defaults to ``D**-0.5``;
    ``save`` picks what is kept for the backward (``SAVE_POLICIES``)."""
    if scale is None:
        scale = xq.shape[-1] ** -0.5
    return PackedDocAttention.apply(xq, xk, xv, q_norm_w, k_norm_w, rope_cos, rope_sin, position_ids, document_ids,
                                    float(scale), bool(causal), sliding_window, float(eps), tile_map, save)


def qk_norm_rope(xq, xk, q_norm_w, k_norm_w, rope_cos, rope_sin, position_ids=None, eps=1e-6, add_unit_offset=True):
    """The prologue on its own (differentiable): returns (q, k) in [B,S,H,D]."""
    return _QKNormRope.apply(xq, xk, q_norm_w, k_norm_w, rope_cos, rope_sin, position_ids, float(eps),
                             bool(add_unit_offset))


def doc_masked_attention(q, k, v, document_ids=None, scale=None, causal=True, sliding_window=None, tile_map=None):
    """The attention on its own (differentiable): q [B,S,Hq,D], k/v [B,S,Hkv,D] -> [B,S,Hq,D]."""
    if scale is None:
        scale = q.shape[-1] ** -0.5
    return _DocMaskedAttention.apply(q, k, v, document_ids, float(scale), bool(causal), sliding_window, tile_map)
