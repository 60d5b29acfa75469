"""MI355X (gfx950) implementation of maester's packed-SFT document-masked attention path.

Drop-in for what sits between the qkv split and ``o_proj`` in maester's ``GemmaAttention.forward``
(maester/models/gemma/model.py:364-439) and for the per-step ``create_block_mask`` calls of
``GemmaTextModel.forward`` (model.py:694-730): a block-sparse tile map built on the GPU from
``document_ids``, a fused QK-RMSNorm + RoPE prologue over per-document ``position_ids``, and a GQA
flash-style forward/backward -- all hand-written HIP kernels behind a C ABI
(``include/maester_attn.h``), driven from PyTorch-ROCm through ``ctypes``.
"""
from .tile_map import TileMap, build_tile_map
from .rope import precompute_rope_tables
from .attention import (PackedDocAttention, packed_doc_attention, qk_norm_rope, doc_masked_attention)
from .gemma_attention import GemmaAttention, GemmaAttentionConfig
from .rmsnorm import RMSNorm, rms_norm
from .linear_ce import ce_rows, linear_cross_entropy
from .gemma_layers import GemmaLayerConfig, GemmaMLP, Gemma2DecoderLayer, GemmaModel, GemmaTextModel
from .packed_ids import (generate_position_ids, generate_document_ids, packed_collate_ids, boundaries_to_tensors,
                         device_packed_ids)

__all__ = [
    "TileMap", "build_tile_map", "precompute_rope_tables", "PackedDocAttention", "packed_doc_attention",
    "qk_norm_rope", "doc_masked_attention", "GemmaAttention", "GemmaAttentionConfig",
    "generate_position_ids", "generate_document_ids", "packed_collate_ids", "boundaries_to_tensors",
    "device_packed_ids", "RMSNorm", "rms_norm", "ce_rows", "linear_cross_entropy", "GemmaLayerConfig", "GemmaMLP", "Gemma2DecoderLayer", "GemmaModel", "GemmaTextModel",
]
