"""The decoder layer and the layer stack around the attention path.

Counterparts of ``GemmaMLP`` (maester/models/gemma/model.py:177-199), ``Gemma2DecoderLayer``
(model.py:446-513) and ``GemmaModel`` (model.py:524-560) with the orchestration of
``GemmaTextModel.forward`` (model.py:654-757) reduced to what concerns this path: the tile maps and
ids of a step are built once (``build_step_inputs``) and handed to every layer; local and global
layers alternate as ``attn_types`` says; the four sandwich norms run as fused kernels, the two
post-norms with their residual add folded in.  The projections and the MLP stay torch GEMMs.
``GemmaTextModel`` puts the token embedding in front and the tied-embedding loss behind
(model.py:570-769): ``forward(tokens, labels, position_ids, document_ids)`` returns the loss of the
fused linear + cross-entropy, or the logits without labels.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch
import torch.nn.functional as F
from torch import nn

from .gemma_attention import GemmaAttention, GemmaAttentionConfig, StepInputs, build_step_inputs
from .linear_ce import linear_cross_entropy
from .rmsnorm import RMSNorm


@dataclass
class GemmaLayerConfig(GemmaAttentionConfig):
    """``GemmaAttentionConfig`` plus the fields of the reference's ``ModelArgs`` that the layer and
    the stack read (model.py:14-60)."""
    intermediate_size: int = 0
    n_layers: int = 1
    attn_types: tuple | None = None          # e.g. ("local_sliding",) * 5 + ("global",)
    use_pre_ffw_norm: bool = True
    use_post_ffw_norm: bool = True
    vocab_size: int = 0                      # GemmaTextModel only


class GemmaMLP(nn.Module):
    def __init__(self, hidden_size: int, intermediate_size: int):
        super().__init__()
        self.gate_proj = nn.Linear(hidden_size, intermediate_size, bias=False)
        self.up_proj = nn.Linear(hidden_size, intermediate_size, bias=False)
        self.down_proj = nn.Linear(intermediate_size, hidden_size, bias=False)

    def forward(self, x):
        return self.down_proj(F.gelu(self.gate_proj(x), approximate="tanh") * self.up_proj(x))

    def init_weights(self, init_std: float):
        for lin in (self.gate_proj, self.up_proj, self.down_proj):
            nn.init.normal_(lin.weight, mean=0.0, std=init_std)


class Gemma2DecoderLayer(nn.Module):
    """Same parameters and the same arithmetic as the reference layer; ``forward(hidden_states, step)``
    takes the step's shared inputs in place of the masks and rope tables."""

    def __init__(self, config: GemmaLayerConfig, attn_type: str):
        super().__init__()
        self.attn_type = attn_type
        self.self_attn = GemmaAttention(config, attn_type)
        self.mlp = GemmaMLP(config.dim, config.intermediate_size)
        self.input_layernorm = RMSNorm(config.dim, config.rms_norm_eps)
        self.post_attention_layernorm = RMSNorm(config.dim, config.rms_norm_eps)
        self.pre_feedforward_layernorm = RMSNorm(config.dim, config.rms_norm_eps) if config.use_pre_ffw_norm else None
        self.post_feedforward_layernorm = RMSNorm(config.dim, config.rms_norm_eps) if config.use_post_ffw_norm else None

    def forward(self, hidden_states: torch.Tensor, step: StepInputs) -> torch.Tensor:
        residual = hidden_states
        attn = self.self_attn(self.input_layernorm(hidden_states), step)
        hidden_states = self.post_attention_layernorm(attn, residual=residual)      # residual + norm(attn), one pass
        residual = hidden_states
        x = hidden_states if self.pre_feedforward_layernorm is None else self.pre_feedforward_layernorm(hidden_states)
        x = self.mlp(x)
        if self.post_feedforward_layernorm is None:
            return residual + x
        return self.post_feedforward_layernorm(x, residual=residual)

    def init_weights(self, init_std: float):
        for norm in (self.input_layernorm, self.post_attention_layernorm, self.pre_feedforward_layernorm,
                     self.post_feedforward_layernorm):
            if norm is not None:
                norm.reset_parameters()
        self.self_attn.init_weights(init_std)
        self.mlp.init_weights(init_std)


class GemmaModel(nn.Module):
    """The stack of decoder layers and the final norm; ``forward(hidden_states, position_ids,
    document_ids)`` builds the step's tile maps once for all layers (two builds: global and local)."""

    def __init__(self, config: GemmaLayerConfig):
        super().__init__()
        self.config = config
        kinds = config.attn_types
        self.layers = nn.ModuleList(
            Gemma2DecoderLayer(config, kinds[i % len(kinds)] if kinds is not None else "global") for i in range(config.n_layers))
        self.norm = RMSNorm(config.dim, config.rms_norm_eps)

    def forward(self, hidden_states: torch.Tensor, position_ids=None, document_ids=None, step: StepInputs | None = None):
        if step is None:
            B, S, _ = hidden_states.shape
            step = build_step_inputs(self.config, B, S, position_ids, document_ids, device=hidden_states.device)
        for layer in self.layers:
            hidden_states = layer(hidden_states, step)
        return self.norm(hidden_states)

    def init_weights(self, init_std: float):
        for layer in self.layers:
            layer.init_weights(init_std)
        self.norm.reset_parameters()


class GemmaTextModel(nn.Module):
    """Counterpart of the reference's ``GemmaTextModel`` (model.py:570-769) with the same parameter
    names (``tok_embeddings.weight``, ``model.layers.*``, ``model.norm.weight``) and the same
    ``forward(tokens, labels=None, position_ids=None, document_ids=None)``: embeddings scaled by
    sqrt(dim) (the factor rounded to the activation dtype, as there), the layer stack on one step's
    tile maps, then the loss against the tied embedding table (``labels`` given, -100 ignored) or the
    logits."""

    def __init__(self, config: GemmaLayerConfig):
        super().__init__()
        if config.vocab_size <= 0:
            raise ValueError("GemmaTextModel needs config.vocab_size")
        self.config = config
        self.model_args = config
        self.vocab_size = config.vocab_size
        self.n_layers = config.n_layers
        self.tok_embeddings = nn.Embedding(config.vocab_size, config.dim)
        self.model = GemmaModel(config)

    def init_weights(self, init_std: float = 0.02):
        nn.init.normal_(self.tok_embeddings.weight, std=init_std)
        self.model.init_weights(init_std)

    def forward(self, tokens: torch.Tensor, labels: torch.Tensor | None = None, position_ids=None, document_ids=None):
        hidden_states = self.tok_embeddings(tokens)
        normalizer = torch.tensor(self.config.dim ** 0.5, dtype=hidden_states.dtype, device=hidden_states.device)
        hidden_states = self.model(hidden_states * normalizer, position_ids, document_ids)
        weight = self.tok_embeddings.weight
        if labels is not None:
            return linear_cross_entropy(hidden_states, weight, labels)
        return torch.matmul(hidden_states, weight.t())
