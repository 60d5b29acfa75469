"""Dense (closed-form) document-masked GQA attention, restated in torch (CPU or any device).
Test infrastructure only.

Follows the semantics the reference obtains from torch FlexAttention
(maester/models/gemma/model.py:384-396; third-party torch/_higher_order_ops/flex_attention.py
``math_attention`` 159-267, ``sdpa_dense_backward`` 825-993) and that its own "naive" branch
restates (model.py:397-432):
    S = (Q K^T) * scale (fp32), masked -> -inf, P = softmax(S), O = P V;
    q-head h uses kv-head h // (Hq/Hkv).
Backward comes from torch autograd through this closed form.
"""
from __future__ import annotations

import torch

from . import masks


def dense_attention(q, k, v, document_ids, scale, causal=True, window=None, compute_dtype=torch.float32,
                    return_lse=False):
    """q [B,S,Hq,D], k/v [B,S,Hkv,D] (the layout GemmaAttention holds before its transposes).
    Returns out [B,S,Hq,D] in ``compute_dtype`` (and LSE [B,Hq,S], natural log).  Processes one
    (batch row, kv head) slice at a time so the live score tensor is G*S*S elements."""
    B, S, Hq, D = q.shape
    Hkv = k.shape[2]
    G = Hq // Hkv
    out = torch.empty(B, S, Hq, D, dtype=compute_dtype, device=q.device)
    lse = torch.empty(B, Hq, S, dtype=compute_dtype, device=q.device)
    for b in range(B):
        ids_b = None if document_ids is None else document_ids[b:b + 1]
        m = masks.dense_mask(ids_b, 1, S, causal, window, device=q.device)[0, 0]  # [S,S]
        for hk in range(Hkv):
            qs = q[b, :, hk * G:(hk + 1) * G].to(compute_dtype).transpose(0, 1)      # [G,S,D]
            ks = k[b, :, hk].to(compute_dtype)                                          # [S,D]
            vs = v[b, :, hk].to(compute_dtype)
            s = torch.matmul(qs, ks.t()) * scale
            s = s.masked_fill(~m, float("-inf"))
            l = torch.logsumexp(s, dim=-1)
            p = torch.exp(s - l[..., None])
            o = torch.matmul(p, vs)                                                      # [G,S,D]
            out[b, :, hk * G:(hk + 1) * G] = o.transpose(0, 1)
            lse[b, hk * G:(hk + 1) * G] = l
    return (out, lse) if return_lse else out


def dense_attention_fwd_bwd(q, k, v, dout, document_ids, scale, causal=True, window=None,
                            compute_dtype=torch.float32):
    """Forward + autograd backward of the closed form, sliced per (row, kv head).
    Returns out, dq, dk, dv in ``compute_dtype`` with the [B,S,H,D] layout."""
    B, S, Hq, D = q.shape
    Hkv = k.shape[2]
    G = Hq // Hkv
    dev = q.device
    out = torch.empty(B, S, Hq, D, dtype=compute_dtype, device=dev)
    dq = torch.empty(B, S, Hq, D, dtype=compute_dtype, device=dev)
    dk = torch.empty(B, S, Hkv, D, dtype=compute_dtype, device=dev)
    dv = torch.empty(B, S, Hkv, D, dtype=compute_dtype, device=dev)
    for b in range(B):
        ids_b = None if document_ids is None else document_ids[b:b + 1]
        m = masks.dense_mask(ids_b, 1, S, causal, window, device=dev)[0, 0]
        for hk in range(Hkv):
            qs = q[b, :, hk * G:(hk + 1) * G].to(compute_dtype).transpose(0, 1).detach().requires_grad_(True)
            ks = k[b, :, hk].to(compute_dtype).detach().requires_grad_(True)
            vs = v[b, :, hk].to(compute_dtype).detach().requires_grad_(True)
            s = torch.matmul(qs, ks.t()) * scale
            s = s.masked_fill(~m, float("-inf"))
            p = torch.softmax(s, dim=-1)
            o = torch.matmul(p, vs)
            go = dout[b, :, hk * G:(hk + 1) * G].to(compute_dtype).transpose(0, 1)
            gq, gk, gv = torch.autograd.grad(o, (qs, ks, vs), go)
            out[b, :, hk * G:(hk + 1) * G] = o.detach().transpose(0, 1)
            dq[b, :, hk * G:(hk + 1) * G] = gq.transpose(0, 1)
            dk[b, :, hk] = gk
            dv[b, :, hk] = gv
    return out, dq, dk, dv


def flex_attention_cpu(q, k, v, document_ids, scale, causal=True, window=None, compiled=False):
    """torch's own FlexAttention on CPU with the restated mask mod -- the same call
    GemmaAttention.forward makes (model.py:384-396).  q/k/v in [B,S,H,D]; returns [B,S,Hq,D]."""
    from torch.nn.attention.flex_attention import create_block_mask, flex_attention
    B, S, Hq, D = q.shape
    Hkv = k.shape[2]
    mod = masks.make_mask_mod(document_ids, causal, window)
    bm = create_block_mask(mod, B, None, S, S, device="cpu")
    fn = torch.compile(flex_attention, fullgraph=True) if compiled else flex_attention
    o = fn(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), block_mask=bm, scale=scale,
           enable_gqa=(Hq != Hkv))
    return o.transpose(1, 2)


def full_path(xq, xk, xv, q_w, k_w, cos, sin, position_ids, document_ids, scale, causal=True, window=None,
              eps=1e-6, compute_dtype=torch.float32):
    """Prologue + attention in ``compute_dtype`` end to end, differentiable w.r.t. its tensor inputs
    (used by tests through torch autograd for dW of the norms)."""
    from . import prologue as P
    wd = compute_dtype
    q = P.rope_apply(P.rms_norm(xq.to(wd), q_w, eps), cos, sin, position_ids)
    k = P.rope_apply(P.rms_norm(xk.to(wd), k_w, eps), cos, sin, position_ids)
    B, S, Hq, D = q.shape
    Hkv = k.shape[2]
    G = Hq // Hkv
    outs = []
    for b in range(B):
        ids_b = None if document_ids is None else document_ids[b:b + 1]
        m = masks.dense_mask(ids_b, 1, S, causal, window, device=q.device)[0, 0]
        kb = k[b].repeat_interleave(G, dim=1).transpose(0, 1)     # [Hq,S,D]
        vb = xv[b].to(wd).repeat_interleave(G, dim=1).transpose(0, 1)
        s = torch.matmul(q[b].transpose(0, 1), kb.transpose(1, 2)) * scale
        s = s.masked_fill(~m, float("-inf"))
        outs.append(torch.matmul(torch.softmax(s, -1), vb).transpose(0, 1))
    return torch.stack(outs)
