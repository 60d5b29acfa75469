"""The reference-side binding, executed: a module whose ``forward`` has the signature of maester's
``GemmaAttention.forward`` (maester/models/gemma/model.py:344-356: ``hidden_states, freqs_cis, mask,
local_mask, dense_mask, dense_local_mask``) plus the per-step ``hip`` inputs, with a third backend
``"hip"`` that calls ``packed_doc_attention`` the way the integration notes tell a maintainer to patch
model.py:339-342 / 366-438, and the per-step dictionary built as the patch to model.py:694-747 builds
it.  Its ``"naive"`` backend is the dense-mask formulation of the same layer (norm, RoPE through the
gathered complex table, masked softmax) written with the oracle's pieces; the two backends are run on
the same weights and inputs and compared.

CPU: the patched module constructs, keeps the reference's signature and attribute names, validates
backends as the reference does (ValueError), and the hip backend refuses CPU tensors (no fallback).
GPU: hip backend vs naive backend, outputs and the gradients of every parameter."""
import inspect

import pytest
import torch
from torch import nn

from maester_amd import build_tile_map, packed_doc_attention, precompute_rope_tables
from oracle import masks as M
from oracle import prologue as P


class _Norm(nn.Module):                       # parameter name and zero init of the reference's RMSNorm (model.py:135-172)
    def __init__(self, dim, eps):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.zeros(dim))


class PatchedGemmaAttention(nn.Module):
    """Constructor attributes of model.py:284-337; ``forward`` = the reference's signature + ``hip``."""

    def __init__(self, dim, n_heads, n_kv_heads, head_dim, attn_type, sliding_window_size, use_qk_norm=True, eps=1e-6):
        super().__init__()
        self.num_heads, self.num_kv_heads, self.head_dim, self.hidden_size = n_heads, n_kv_heads, head_dim, dim
        self.num_queries_per_kv = n_heads // n_kv_heads
        self.q_size, self.kv_size = n_heads * head_dim, n_kv_heads * head_dim
        self.scaling = head_dim ** -0.5
        self.qkv_proj = nn.Linear(dim, (n_heads + 2 * n_kv_heads) * head_dim, bias=False)
        self.o_proj = nn.Linear(n_heads * head_dim, dim, bias=False)
        self.query_norm = _Norm(head_dim, eps) if use_qk_norm else None
        self.key_norm = _Norm(head_dim, eps) if use_qk_norm else None
        self.attn_type, self.sliding_window_size = attn_type, sliding_window_size
        self.attention_backend = "naive"

    def set_backend(self, backend: str) -> None:
        if backend not in {"flex", "naive", "hip"}:
            raise ValueError(f"Unsupported attention backend: {backend}")
        self.attention_backend = backend

    def forward(self, hidden_states, freqs_cis, mask, local_mask=None, dense_mask=None, dense_local_mask=None, hip=None):
        batch_size, input_len, _ = hidden_states.shape
        qkv = self.qkv_proj(hidden_states)
        xq, xk, xv = qkv.split([self.q_size, self.kv_size, self.kv_size], dim=-1)
        xq = xq.view(batch_size, -1, self.num_heads, self.head_dim)
        xk = xk.view(batch_size, -1, self.num_kv_heads, self.head_dim)
        xv = xv.view(batch_size, -1, self.num_kv_heads, self.head_dim)
        if self.attention_backend == "hip":
            use_local = self.attn_type == "local_sliding" and self.sliding_window_size is not None
            cos, sin = hip["local_rope"] if self.attn_type == "local_sliding" else hip["global_rope"]
            out = packed_doc_attention(
                xq, xk, xv,
                self.query_norm.weight if self.query_norm is not None else None,
                self.key_norm.weight if self.key_norm is not None else None,
                cos, sin, hip["position_ids"], hip["document_ids"], self.scaling, causal=True,
                sliding_window=self.sliding_window_size if use_local else None,
                eps=self.query_norm.eps if self.query_norm is not None else 1e-6,
                tile_map=hip["local_map"] if use_local else hip["global_map"])
            return self.o_proj(out.view(batch_size, input_len, -1))
        if self.attention_backend != "naive":
            raise NotImplementedError("this stand-in carries the naive and the hip backend")
        # dense formulation in fp32: norm, rotation by the gathered complex table, masked softmax
        f = torch.float32
        qw = None if self.query_norm is None else self.query_norm.weight.to(f)
        kw = None if self.key_norm is None else self.key_norm.weight.to(f)
        eps = 1e-6 if self.query_norm is None else self.query_norm.eps
        rot = lambda x: torch.cat([x[..., : self.head_dim // 2] * freqs_cis.real[:, :, None] - x[..., self.head_dim // 2:] * freqs_cis.imag[:, :, None],
                                   x[..., : self.head_dim // 2] * freqs_cis.imag[:, :, None] + x[..., self.head_dim // 2:] * freqs_cis.real[:, :, None]], -1)
        q = rot(P.rms_norm(xq.to(f), qw, eps)).transpose(1, 2)
        k = rot(P.rms_norm(xk.to(f), kw, eps)).transpose(1, 2).repeat_interleave(self.num_queries_per_kv, dim=1)
        v = xv.to(f).transpose(1, 2).repeat_interleave(self.num_queries_per_kv, dim=1)
        use_local = self.attn_type == "local_sliding" and self.sliding_window_size is not None and dense_local_mask is not None
        keep = dense_local_mask if use_local else dense_mask
        s = (q @ k.transpose(-1, -2)) * self.scaling
        s = s.masked_fill(~keep, float("-inf"))
        out = (torch.softmax(s, -1) @ v).transpose(1, 2).reshape(batch_size, input_len, -1)
        return self.o_proj(out.to(hidden_states.dtype))


def _step_inputs(position_ids, document_ids, head_dim, max_seq_len, window, device, with_maps):
    """What the patched GemmaTextModel.forward builds once per step (hip) and what the reference builds (dense masks,
    gathered freqs_cis) -- model.py:694-747."""
    B, S = document_ids.shape
    grope = precompute_rope_tables(head_dim, 2 * max_seq_len, 1_000_000.0, 1.0, device=device)
    lrope = precompute_rope_tables(head_dim, 2 * max_seq_len, 10_000.0, 1.0, device=device)
    hip = {"position_ids": position_ids, "document_ids": document_ids, "global_rope": grope, "local_rope": lrope,
           "global_map": None, "local_map": None}
    if with_maps:
        hip["global_map"] = build_tile_map(document_ids, B, S, causal=True, sliding_window=None, device=device)
        hip["local_map"] = build_tile_map(document_ids, B, S, True, window, device=device)
    dense = M.dense_mask(document_ids.cpu(), B, S, True, None).to(device)
    dense_local = M.dense_mask(document_ids.cpu(), B, S, True, window).to(device)
    cis = {k: torch.complex(c[position_ids], s[position_ids]) for k, (c, s) in (("global", grope), ("local_sliding", lrope))}
    return hip, dense, dense_local, cis


def _ids(B, S):
    g = torch.Generator().manual_seed(3)
    doc = torch.zeros(B, S, dtype=torch.long)
    pos = torch.zeros(B, S, dtype=torch.long)
    for b in range(B):
        at, d = 0, 0
        while at < S:
            n = min(int(torch.randint(20, 200, (1,), generator=g)), S - at)
            doc[b, at:at + n] = d
            pos[b, at:at + n] = torch.arange(n)
            at, d = at + n, d + 1
    return pos, doc


def test_patched_module_keeps_the_reference_interface():
    ref_params = ["self", "hidden_states", "freqs_cis", "mask", "local_mask", "dense_mask", "dense_local_mask"]
    assert list(inspect.signature(PatchedGemmaAttention.forward).parameters) == ref_params + ["hip"]
    attn = PatchedGemmaAttention(64, 4, 2, 64, "global", 32)
    assert {"qkv_proj.weight", "o_proj.weight", "query_norm.weight", "key_norm.weight"} == set(attn.state_dict())
    with pytest.raises(ValueError):
        attn.set_backend("cuda")
    attn.set_backend("hip")
    pos, doc = _ids(1, 128)
    hip, dense, dense_local, cis = _step_inputs(pos, doc, 64, 128, 32, "cpu", with_maps=False)
    with pytest.raises(RuntimeError, match="no CPU fallback"):        # the binding reaches the library boundary and is refused there
        attn(torch.randn(1, 128, 64), cis["global"], None, None, dense, dense_local, hip=hip)
    attn.set_backend("naive")                                          # the comparator runs anywhere
    assert attn(torch.randn(1, 128, 64), cis["global"], None, None, dense, dense_local).shape == (1, 128, 64)


@pytest.mark.gpu
@pytest.mark.parametrize("attn_type", ["global", "local_sliding"])
def test_hip_backend_of_the_patched_module_matches_its_dense_backend(gpu, attn_type):
    torch.manual_seed(1)
    B, S, dim, Hq, Hkv, D, window = 2, 700, 256, 4, 2, 128, 96
    pos, doc = _ids(B, S)
    pos, doc = pos.to(gpu), doc.to(gpu)
    hip, dense, dense_local, cis = _step_inputs(pos, doc, D, 1024, window, gpu, with_maps=True)
    attn = PatchedGemmaAttention(dim, Hq, Hkv, D, attn_type, window).to(gpu)
    with torch.no_grad():
        attn.qkv_proj.weight.normal_(0, 0.05)
        attn.o_proj.weight.normal_(0, 0.05)
        attn.query_norm.weight.normal_(0, 0.1)
        attn.key_norm.weight.normal_(0, 0.1)
    attn = attn.to(torch.bfloat16)
    h = (0.5 * torch.randn(B, S, dim, device=gpu)).to(torch.bfloat16)
    dy = (0.1 * torch.randn(B, S, dim, device=gpu)).to(torch.bfloat16)
    results = {}
    for backend in ("naive", "hip"):
        attn.set_backend(backend)
        attn.zero_grad()
        y = attn(h, cis[attn_type], None, None, dense, dense_local, hip=hip)
        y.backward(dy)
        results[backend] = (y.detach().float(), {n: p.grad.float().clone() for n, p in attn.named_parameters()})
    rel = lambda a, b: float((a - b).norm() / b.norm())
    y_n, g_n = results["naive"]
    y_h, g_h = results["hip"]
    assert float((y_h - y_n).abs().max()) <= 2e-2 and rel(y_h, y_n) <= 1e-2, (float((y_h - y_n).abs().max()), rel(y_h, y_n))
    for name in g_n:        # parameter gradients are sums over B*S rows of bf16 products: relative L2 (both sides round in bf16)
        assert rel(g_h[name], g_n[name]) <= 2e-2, (name, rel(g_h[name], g_n[name]))
