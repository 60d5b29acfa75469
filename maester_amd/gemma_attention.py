"""A ``GemmaAttention``-compatible module whose attention core runs in the HIP library.

Mirrors maester's ``GemmaAttention`` (maester/models/gemma/model.py:283-444): same parameters
(``qkv_proj``, ``o_proj``, ``query_norm.weight``, ``key_norm.weight``), same scaling rule
(``query_pre_attn_scalar**-0.5`` else ``head_dim**-0.5``, model.py:304-307), same GQA mapping and
the same choice of the local (sliding-window) mask on ``local_sliding`` layers (model.py:375-381).
The reference's backend switch ``set_backend({"flex","naive"})`` (model.py:339-342) gains a third
value, ``"hip"``, which is the only one implemented here; the others raise.

The projections stay ordinary ``torch.nn.functional.linear`` GEMMs (rocBLAS/hipBLASLt): they are
outside this path.  What the reference passes as per-step ``BlockMask``s and gathered ``freqs_cis``
is passed here as ``TileMap``s (built once per step by ``build_step_inputs``) and the RoPE tables
plus ``position_ids``.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import torch
import torch.nn as nn
import torch.nn.functional as F

from .attention import packed_doc_attention
from .rope import precompute_rope_tables
from .tile_map import TileMap, build_tile_map


@dataclass
class GemmaAttentionConfig:
    """The fields of maester's Gemma ``ModelArgs`` that the attention reads
    (maester/models/gemma/model.py:14-57, maester/models/gemma/__init__.py:5-105)."""
    dim: int = 2560
    n_heads: int = 8
    num_key_value_heads: int = 4
    head_dim: int = 256
    max_seq_len: int = 8192
    rms_norm_eps: float = 1e-6
    use_qk_norm: bool = True
    query_pre_attn_scalar: float | None = None
    sliding_window_size: int | None = 1024
    rope_wave_length: dict = field(default_factory=lambda: {"local_sliding": 10_000, "global": 1_000_000})
    rope_scaling: dict | None = None


class _StoredNormWeight(nn.Module):
    """Holds the ``weight`` parameter of a Gemma RMSNorm (zeros-initialised, effective scale 1+w;
    model.py:135-147) under the same attribute path as the reference (``query_norm.weight``)."""

    def __init__(self, dim: int, eps: float):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.zeros(dim))


@dataclass
class StepInputs:
    """Per-step, layer-independent inputs (what GemmaTextModel.forward builds at model.py:680-747)."""
    position_ids: torch.Tensor | None
    document_ids: torch.Tensor | None
    global_map: TileMap
    local_map: TileMap | None


def build_step_inputs(config: GemmaAttentionConfig, batch_size: int, seq_len: int, position_ids=None,
                      document_ids=None, device=None) -> StepInputs:
    """Build the global and (if the model has a sliding window) local tile maps once per step, for
    reuse by every layer."""
    gmap = build_tile_map(document_ids, batch_size, seq_len, True, None, device=device)
    lmap = None
    if config.sliding_window_size:
        lmap = build_tile_map(document_ids, batch_size, seq_len, True, int(config.sliding_window_size), device=device)
    return StepInputs(position_ids, document_ids, gmap, lmap)


class GemmaAttention(nn.Module):
    def __init__(self, config: GemmaAttentionConfig, attn_type: str = "global"):
        super().__init__()
        self.num_heads = config.n_heads
        self.num_kv_heads = config.num_key_value_heads
        assert self.num_heads % self.num_kv_heads == 0
        self.num_queries_per_kv = self.num_heads // self.num_kv_heads
        self.hidden_size = config.dim
        self.head_dim = config.head_dim
        self.q_size = self.num_heads * self.head_dim
        self.kv_size = self.num_kv_heads * self.head_dim
        if config.query_pre_attn_scalar is not None:
            self.scaling = config.query_pre_attn_scalar ** -0.5
        else:
            self.scaling = self.head_dim ** -0.5
        self.qkv_proj = nn.Linear(self.hidden_size, (self.num_heads + 2 * self.num_kv_heads) * self.head_dim,
                                  bias=False)
        self.o_proj = nn.Linear(self.num_heads * self.head_dim, self.hidden_size, bias=False)
        self.query_norm = _StoredNormWeight(self.head_dim, config.rms_norm_eps) if config.use_qk_norm else None
        self.key_norm = _StoredNormWeight(self.head_dim, config.rms_norm_eps) if config.use_qk_norm else None
        self.eps = config.rms_norm_eps
        self.attn_type = attn_type
        self.sliding_window_size = config.sliding_window_size
        self.attention_backend = "hip"
        self.saved_for_backward = "all"   # see maester_amd.attention.SAVE_POLICIES
        # RoPE tables (model.py:588-623): 2*max_seq_len rows; scaling factor on the global table only
        wl = config.rope_wave_length or {}
        if attn_type == "local_sliding":
            theta, factor = wl.get("local_sliding", 10_000), 1.0
        else:
            theta = wl.get("global", 10_000)
            factor = (config.rope_scaling or {}).get("factor", 1) if config.rope_scaling else 1.0
        # kept out of the module's buffers on purpose: ``module.to(torch.bfloat16)`` must not round the
        # tables (the reference's table is complex64 whatever the dtype of the weights)
        self._rope_cpu = precompute_rope_tables(self.head_dim, 2 * config.max_seq_len, theta, factor)
        self._rope_dev: dict = {}

    def _rope(self, device) -> tuple:
        device = torch.device(device)
        if device not in self._rope_dev:
            self._rope_dev[device] = tuple(t.to(device) for t in self._rope_cpu)
        return self._rope_dev[device]

    @property
    def rope_cos(self) -> torch.Tensor:
        """fp32 ``[2*max_seq_len, head_dim/2]`` on the device of the weights."""
        return self._rope(self.qkv_proj.weight.device)[0]

    @property
    def rope_sin(self) -> torch.Tensor:
        return self._rope(self.qkv_proj.weight.device)[1]

    def set_backend(self, backend: str) -> None:
        if backend not in {"flex", "naive", "hip"}:
            raise ValueError(f"Unsupported attention backend: {backend}")
        if backend != "hip":
            raise NotImplementedError(
                f"backend {backend!r} is the reference's torch path; this module only carries the 'hip' backend")
        self.attention_backend = backend

    def init_weights(self, init_std: float):
        nn.init.normal_(self.qkv_proj.weight, mean=0.0, std=init_std)
        nn.init.normal_(self.o_proj.weight, mean=0.0, std=init_std)

    def forward(self, hidden_states: torch.Tensor, step: StepInputs) -> torch.Tensor:
        assert hidden_states.dim() == 3
        batch_size, input_len, _ = hidden_states.shape
        qkv = self.qkv_proj(hidden_states)
        xq, xk, xv = qkv.split([self.q_size, self.kv_size, self.kv_size], dim=-1)
        xq = xq.view(batch_size, -1, self.num_heads, self.head_dim)
        xk = xk.view(batch_size, -1, self.num_kv_heads, self.head_dim)
        xv = xv.view(batch_size, -1, self.num_kv_heads, self.head_dim)
        use_local = (self.attn_type == "local_sliding" and self.sliding_window_size is not None
                     and step.local_map is not None)
        tile_map = step.local_map if use_local else step.global_map
        out = packed_doc_attention(
            xq, xk, xv,
            self.query_norm.weight if self.query_norm is not None else None,
            self.key_norm.weight if self.key_norm is not None else None,
            self.rope_cos, self.rope_sin, step.position_ids, step.document_ids, self.scaling,
            causal=True, sliding_window=int(self.sliding_window_size) if use_local else None, eps=self.eps,
            tile_map=tile_map, save=self.saved_for_backward)
        out = out.view(batch_size, input_len, -1)   # already [B,S,Hq*D]: no transposed copy
        return self.o_proj(out)
