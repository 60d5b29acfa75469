"""CPU-side checks: the C-ABI library loads, exports every symbol the header declares, and rejects
bad arguments before any launch; workload generators reproduce the survey's census."""
import ctypes
import os
import re

import pytest
import torch

from maester_amd import _lib, workloads
from maester_amd._lib import MaTensor4, MaTileMap

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "maester_attn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ma_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = _lib.lib()
    names = _declared_symbols()
    assert set(names) == set(_lib.EXPORTS), (names, _lib.EXPORTS)
    for n in names:
        assert hasattr(L, n), n
    assert L.ma_version() == _lib.MA_ABI_VERSION   # the binding refuses a library built from another header
    assert L.ma_last_error() is not None


def _t4(ptr=0x1000, sb=1 << 20, ss=1024, sh=256):
    return MaTensor4(ptr, sb, ss, sh)


def _map(ok=True):
    return MaTileMap(*([0x1000] * 8 if ok else [0] * 8))


def _err():
    return _lib.lib().ma_last_error().decode()


def test_workspace_sizes():
    L = _lib.lib()
    # class byte per tile + (min, max) int64 per tile row + counter + list of tiles to count exactly
    assert L.ma_tile_map_workspace_bytes(4, 8192) == 4 * 64 * 64 + 4 * 64 * 16 + 16 + 4 * 64 * 64 * 4
    assert L.ma_tile_map_workspace_bytes(1, 129) == 16 + 2 * 16 + 16 + 4 * 4   # T = 2: 4 class bytes rounded up to 16
    assert L.ma_tile_map_workspace_bytes(0, 10) == 0
    assert L.ma_attn_bwd_workspace_bytes(4, 8192, 8, 4, 256) == 4 * 8 * 8192 * 4
    # with room for dS: delta (rounded up to 256 bytes) + one 32 KB slot per (batch row, query head, q tile, kv tile)
    # delta, then one 32 KB slot per query head and VISITED tile (config 2 visits 1698 of its 16384 tiles)
    assert L.ma_attn_bwd_ds_workspace_bytes(4, 8192, 8, 1698) == 4 * 8 * 8192 * 4 + 8 * 1698 * 32768
    assert L.ma_attn_bwd_ds_workspace_bytes(1, 130, 2, 3) == 1280 + 2 * 3 * 32768     # 1040 bytes of delta -> 1280
    assert L.ma_attn_bwd_ds_workspace_bytes(0, 8192, 8, 10) == 0 and L.ma_attn_bwd_ds_workspace_bytes(4, 8192, 8, 0) == 0
    assert L.ma_prologue_bwd_workspace_bytes(4, 8192, 8, 4, 256) > 0


def test_tile_map_argument_errors():
    L = _lib.lib()
    m = _map()
    assert L.ma_tile_map_build(None, 0, 128, 1, -1, ctypes.byref(m), 0x1000, 1 << 20, None) == _lib.MA_ERR_BAD_ARG
    assert "positive" in _err()
    assert L.ma_tile_map_build(None, 1, 128, 2, -1, ctypes.byref(m), 0x1000, 1 << 20, None) == _lib.MA_ERR_BAD_ARG
    assert L.ma_tile_map_build(None, 1, 128, 1, -5, ctypes.byref(m), 0x1000, 1 << 20, None) == _lib.MA_ERR_BAD_ARG
    assert "window" in _err()
    assert L.ma_tile_map_build(None, 1, 128, 1, -1, None, 0x1000, 1 << 20, None) == _lib.MA_ERR_BAD_ARG
    bad = _map(False)
    assert L.ma_tile_map_build(None, 1, 128, 1, -1, ctypes.byref(bad), 0x1000, 1 << 20, None) == _lib.MA_ERR_BAD_ARG
    assert L.ma_tile_map_build(None, 1, 1024, 1, -1, ctypes.byref(m), 0x1000, 8, None) == _lib.MA_ERR_BAD_ARG
    assert "workspace" in _err()
    assert L.ma_tile_map_build(None, 1, 1024, 1, -1, ctypes.byref(m), None, 1 << 20, None) == _lib.MA_ERR_BAD_ARG
    # tiles are numbered in 32 bits: B * T * T must stay below 2^31 (B = 1 at S = 128 * 46341 is just above)
    assert L.ma_tile_map_build(None, 1, 128 * 46341, 1, -1, ctypes.byref(m), 0x1000, 1 << 62, None) == _lib.MA_ERR_UNSUPPORTED
    assert "2^31" in _err()
    # the build on the library's own scratch: the same argument checks, and sizes beyond the scratch are refused
    assert L.ma_tile_map_build_static(None, 0, 128, 1, -1, ctypes.byref(m), None) == _lib.MA_ERR_BAD_ARG
    assert L.ma_tile_map_build_static(None, 1, 128, 1, -1, None, None) == _lib.MA_ERR_BAD_ARG
    assert L.ma_tile_map_workspace_bytes(16, 65536) > _lib.MA_TILE_MAP_STATIC_BYTES
    assert L.ma_tile_map_build_static(None, 16, 65536, 1, -1, ctypes.byref(m), None) == _lib.MA_ERR_UNSUPPORTED
    assert "scratch" in _err()


def test_packed_ids_argument_errors():
    L = _lib.lib()
    ok = (0x1000, 0x1000, 0x1000)
    assert L.ma_packed_ids_build(*ok, 0, 4, 128, 0x1000, 0x1000, None) == _lib.MA_ERR_BAD_ARG
    assert L.ma_packed_ids_build(0x1000, 0x1000, None, 1, 4, 128, 0x1000, 0x1000, None) == _lib.MA_ERR_BAD_ARG and "counts" in _err()
    assert L.ma_packed_ids_build(None, 0x1000, 0x1000, 1, 4, 128, 0x1000, 0x1000, None) == _lib.MA_ERR_BAD_ARG and "starts" in _err()
    assert L.ma_packed_ids_build(*ok, 1, -1, 128, 0x1000, 0x1000, None) == _lib.MA_ERR_BAD_ARG
    assert L.ma_packed_ids_build(*ok, 1, 4, 128, None, None, None) == _lib.MA_ERR_BAD_ARG and "outputs" in _err()


def test_rmsnorm_argument_errors():
    L = _lib.lib()
    P_ = 0x1000

    def fwd(x=P_, res=None, w=P_, out=P_, rstd=P_, rows=8, dim=256, eps=1e-6, dtype=1):
        return L.ma_rmsnorm_fwd(x, res, w, out, rstd, rows, dim, eps, 1, dtype, None)

    assert fwd(dim=100) == _lib.MA_ERR_UNSUPPORTED and "multiple of 8" in _err()
    assert fwd(dim=16384) == _lib.MA_ERR_UNSUPPORTED
    assert fwd(rows=0) == _lib.MA_ERR_BAD_ARG
    assert fwd(x=None) == _lib.MA_ERR_BAD_ARG and "NULL" in _err()
    assert fwd(out=0x1004) == _lib.MA_ERR_BAD_ARG and "aligned" in _err()
    assert fwd(dtype=9) == _lib.MA_ERR_BAD_ARG
    assert fwd(eps=-1.0) == _lib.MA_ERR_BAD_ARG
    assert L.ma_rmsnorm_bwd_workspace_bytes(0, 256) == 0
    rc = L.ma_rmsnorm_bwd(P_, P_, P_, P_, P_, P_, P_, 8, 64, 256, 1, 1, None)
    assert rc == _lib.MA_ERR_BAD_ARG and "workspace" in _err()
    rc = L.ma_rmsnorm_bwd(P_, P_, None, P_, P_, P_, P_, 1 << 30, 64, 256, 1, 1, None)
    assert rc == _lib.MA_ERR_BAD_ARG and "rstd" in _err()


def test_attention_argument_errors():
    L = _lib.lib()
    t, m = _t4(), _map()
    r = ctypes.byref

    def fwd(q=t, k=t, v=t, o=t, lse=0x1000, mp=m, causal=1, window=-1, scale=0.1, dtype=1, B=1, S=256, Hq=4, Hkv=2, D=256):
        return L.ma_attn_fwd(r(q), r(k), r(v), r(o), lse, r(mp), None, causal, window, scale, dtype, B, S, Hq, Hkv, D, None)

    assert fwd(D=96) == _lib.MA_ERR_UNSUPPORTED and "head_dim" in _err()
    assert fwd(Hq=5) == _lib.MA_ERR_BAD_ARG and "multiple" in _err()
    assert fwd(dtype=7) == _lib.MA_ERR_BAD_ARG
    assert fwd(scale=0.0) == _lib.MA_ERR_BAD_ARG and "scale" in _err()
    assert fwd(scale=float("nan")) == _lib.MA_ERR_BAD_ARG
    assert fwd(lse=None) == _lib.MA_ERR_BAD_ARG and "lse" in _err()
    assert fwd(q=_t4(ptr=0)) == _lib.MA_ERR_BAD_ARG and "NULL" in _err()
    assert fwd(q=_t4(ptr=0x1004)) == _lib.MA_ERR_BAD_ARG and "aligned" in _err()
    assert fwd(k=_t4(ss=1023)) == _lib.MA_ERR_BAD_ARG and "strides" in _err()
    assert fwd(mp=_map(False)) == _lib.MA_ERR_BAD_ARG and "tile map" in _err()
    assert fwd(causal=3) == _lib.MA_ERR_BAD_ARG
    assert fwd(B=0) == _lib.MA_ERR_BAD_ARG
    assert fwd(S=1 << 24) == _lib.MA_ERR_UNSUPPORTED and "2^24" in _err()
    assert fwd(Hq=66, Hkv=2) == _lib.MA_ERR_UNSUPPORTED and "per kv head" in _err()
    # backward: workspace too small, invalid stages
    rc = L.ma_attn_bwd(r(t), r(t), r(t), r(t), r(t), 0x1000, r(t), r(t), r(t), r(m), None, 1, -1, 0.1, 0x1000, 16, 1,
                       1, 256, 4, 2, 256, None)
    assert rc == _lib.MA_ERR_BAD_ARG and "workspace" in _err()
    rc = L.ma_attn_bwd_stages(r(t), r(t), r(t), r(t), r(t), 0x1000, r(t), r(t), r(t), r(m), None, 1, -1, 0.1, 0x1000,
                              1 << 30, 1, 1, 256, 4, 2, 256, 9, None)
    assert rc == _lib.MA_ERR_BAD_ARG and "stages" in _err()


def test_prologue_argument_errors():
    L = _lib.lib()
    t = _t4()
    r = ctypes.byref
    rc = L.ma_prologue_fwd(r(t), r(t), r(t), r(t), None, None, None, 0x1000, 100, None, 1e-6, 1, None, None, 1, 1, 64, 4,
                           2, 256, None)
    assert rc == _lib.MA_ERR_BAD_ARG and "rope" in _err()
    rc = L.ma_prologue_fwd(r(t), r(t), r(t), r(t), None, None, 0x1000, 0x1000, 10, None, 1e-6, 1, None, None, 1, 1, 64,
                           4, 2, 256, None)
    assert rc == _lib.MA_ERR_BAD_ARG and "n_pos" in _err()
    rc = L.ma_prologue_fwd(r(t), r(t), r(t), r(t), 0x1000, None, 0x1000, 0x1000, 100, None, 1e-6, 1, None, None, 1, 1,
                           64, 4, 2, 256, None)
    assert rc == _lib.MA_ERR_BAD_ARG and "q_rstd" in _err()
    rc = L.ma_prologue_fwd(r(t), r(t), r(t), r(t), None, None, 0x1000, 0x1000, 100, None, 1e-6, 1, None, None, 1, 1, 64,
                           4, 2, 100, None)
    assert rc == _lib.MA_ERR_UNSUPPORTED


def test_python_front_end_refuses_cpu_tensors():
    from maester_amd import build_tile_map, doc_masked_attention
    q = torch.zeros(1, 128, 2, 64)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        doc_masked_attention(q, q, q, torch.zeros(1, 128, dtype=torch.long))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        build_tile_map(torch.zeros(1, 128, dtype=torch.long), 1, 128)
    with pytest.raises(TypeError):
        _lib.dtype_code(torch.float16)


def test_workload_census_matches_survey():
    want = {"c1": 278607, "c2": 21977636, "c3": 17311446, "c4": 138550011, "c5": 44817787}
    for name, pairs in want.items():
        sp = workloads.spec(name)
        rows = workloads.document_lengths(sp)
        assert all(sum(r) == sp.S for r in rows)
        assert workloads.count_pairs(rows, sp.window) == pairs
    # the closed form equals a brute-force count on a small window case
    from oracle import tile_map as otm
    wl = workloads.make("c3", B=2, S=2048)
    assert wl.n_pairs == otm.count_pairs(wl.document_ids.numpy(), 2, 2048, True, 1024)
    assert (wl.position_ids[wl.document_ids == 0][:5] == torch.arange(5)).all()
    assert wl.xq.dtype == torch.bfloat16 and wl.q_w.shape == (256,)
    wlp = workloads.make("c2", B=1, S=1024, pad_tail=100)
    assert (wlp.document_ids[:, -100:] == -1).all() and (wlp.position_ids[:, -100:] == 0).all()


def test_gemma_module_mirrors_reference_interface():
    from maester_amd import GemmaAttention, GemmaAttentionConfig
    cfg = GemmaAttentionConfig(dim=64, n_heads=2, num_key_value_heads=1, head_dim=64, max_seq_len=128,
                               sliding_window_size=32, query_pre_attn_scalar=256)
    attn = GemmaAttention(cfg, "local_sliding")
    assert attn.scaling == 256 ** -0.5
    assert attn.rope_cos.shape == (256, 32)
    assert set(dict(attn.named_parameters())) == {"qkv_proj.weight", "o_proj.weight", "query_norm.weight", "key_norm.weight"}
    assert float(attn.query_norm.weight.abs().sum()) == 0.0          # zeros-initialised, scale 1+w
    with pytest.raises(ValueError):
        attn.set_backend("triton")
    with pytest.raises(NotImplementedError):
        attn.set_backend("flex")
    attn.set_backend("hip")


def test_tile_map_struct_matches_the_header():
    """The ctypes mirror of ma_tile_map has the header's fields, in the header's order."""
    import os
    import re
    hdr = open(os.path.join(os.path.dirname(__file__), "..", "include", "maester_attn.h")).read()
    body = hdr[hdr.index("typedef struct ma_tile_map {"):hdr.index("} ma_tile_map;")]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    fields = re.findall(r"\b(?:int32_t|int64_t)\s*\*?\s*(\w+)\s*;", body)       # 14 device pointers, then the host count
    assert fields == [n for n, _ in MaTileMap._fields_] and len(fields) == 15
    assert int(re.search(r"#define MA_WORK_COUNTERS (\d+)", hdr).group(1)) == _lib.MA_WORK_COUNTERS
    assert int(re.search(r"#define MA_DOC_BLOCK (\d+)", hdr).group(1)) == _lib.MA_DOC_BLOCK


def test_backward_workspace_choice():
    import torch
    from maester_amd import attention as A
    from maester_amd.tile_map import TileMap
    L = _lib.lib()
    z = torch.zeros(1, dtype=torch.int32)
    tm = TileMap(*([z] * 8), seq_len=8192, causal=True, window=None, tile_slot=z, tile_count=torch.tensor([1698], dtype=torch.int32))
    assert tm.visited_tiles() == 1698
    small, large = L.ma_attn_bwd_workspace_bytes(4, 8192, 8, 4, 256), L.ma_attn_bwd_ds_workspace_bytes(4, 8192, 8, 1698)
    assert large - small == 8 * 1698 * 32768                                                 # 0.45 GB, a tenth of one slot per tile
    assert A.backward_workspace_bytes(4, 8192, 8, 4, 256, torch.bfloat16, True, tm) == large
    assert A.backward_workspace_bytes(4, 8192, 8, 4, 256, torch.float32, True, tm) == small  # the hand-over is a bf16 path
    assert A.backward_workspace_bytes(4, 8192, 8, 4, 256, torch.bfloat16, False, tm) == small
    assert A.backward_workspace_bytes(4, 8192, 8, 4, 256, torch.bfloat16, True, None) == small   # no map, no slots
    # a map without visited tiles, or slots beyond the limit: the dQ kernel recomputes instead
    tm._visited = 0
    assert A.backward_workspace_bytes(4, 8192, 8, 4, 256, torch.bfloat16, True, tm) == small
    tm._visited = 8 * 1024 * 1024
    assert L.ma_attn_bwd_ds_workspace_bytes(8, 131072, 8, tm._visited) > A.DS_WORKSPACE_LIMIT
    assert A.backward_workspace_bytes(8, 131072, 8, 4, 256, torch.bfloat16, None, tm) == L.ma_attn_bwd_workspace_bytes(8, 131072, 8, 4, 256)


def test_backward_path_is_decided_once_per_shape(monkeypatch):
    """The two backward paths differ in the last bits, so the choice between them must not follow the free
    memory from call to call: the first map of a shape decides, later maps inherit, an explicit setting wins."""
    import torch
    from maester_amd import attention as A
    from maester_amd.tile_map import TileMap
    L = _lib.lib()
    z = torch.zeros(1, dtype=torch.int32)
    mk = lambda: TileMap(*([z] * 8), seq_len=8192, causal=True, window=None, tile_slot=z, tile_count=torch.tensor([1698], dtype=torch.int32))
    small, large = L.ma_attn_bwd_workspace_bytes(4, 8192, 8, 4, 256), L.ma_attn_bwd_ds_workspace_bytes(4, 8192, 8, 1698)
    monkeypatch.setattr(A, "_HAND_OVER_DECISIONS", {})
    asked = []
    monkeypatch.setattr(A, "_available_bytes", lambda dev: asked.append(1) or 10 * large)
    a = mk()
    assert A.backward_workspace_bytes(4, 8192, 8, 4, 256, torch.bfloat16, None, a) == large and a._hand_over is True
    monkeypatch.setattr(A, "_available_bytes", lambda dev: asked.append(1) or 0)          # memory gets tight later on
    b = mk()
    assert A.backward_workspace_bytes(4, 8192, 8, 4, 256, torch.bfloat16, None, b) == large and len(asked) == 1
    assert A.backward_workspace_bytes(4, 8192, 8, 4, 256, torch.bfloat16, None, a) == large
    assert A.backward_workspace_bytes(4, 8192, 8, 4, 256, torch.bfloat16, False, a) == small   # explicit wins, and is not remembered
    assert A.backward_workspace_bytes(4, 8192, 8, 4, 256, torch.bfloat16, None, a) == large
    monkeypatch.setattr(A, "HAND_OVER_DEFAULT", False)
    assert A.backward_workspace_bytes(4, 8192, 8, 4, 256, torch.bfloat16, None, mk()) == small
    monkeypatch.setattr(A, "HAND_OVER_DEFAULT", None)
    c = mk()                                                                               # another shape decides afresh
    assert A.backward_workspace_bytes(2, 8192, 8, 4, 256, torch.bfloat16, None, c) == L.ma_attn_bwd_workspace_bytes(2, 8192, 8, 4, 256)
    assert c._hand_over is False and len(asked) == 2


def test_text_model_mirrors_reference_parameter_names():
    # maester/models/gemma/model.py:570-585 (tok_embeddings, model), 524-540 (layers, norm), 446-476 (the layer's modules)
    from maester_amd.gemma_layers import GemmaLayerConfig, GemmaTextModel
    cfg = GemmaLayerConfig(dim=64, n_heads=2, num_key_value_heads=1, head_dim=64, max_seq_len=128, sliding_window_size=32,
                           intermediate_size=128, n_layers=2, attn_types=("local_sliding", "global"), vocab_size=100)
    keys = set(GemmaTextModel(cfg).state_dict())
    for name in ("tok_embeddings.weight", "model.norm.weight", "model.layers.1.self_attn.qkv_proj.weight",
                 "model.layers.0.self_attn.o_proj.weight", "model.layers.0.self_attn.query_norm.weight",
                 "model.layers.0.mlp.gate_proj.weight", "model.layers.0.mlp.up_proj.weight", "model.layers.0.mlp.down_proj.weight",
                 "model.layers.0.input_layernorm.weight", "model.layers.0.post_attention_layernorm.weight",
                 "model.layers.0.pre_feedforward_layernorm.weight", "model.layers.0.post_feedforward_layernorm.weight"):
        assert name in keys, name
    with pytest.raises(ValueError):
        GemmaTextModel(GemmaLayerConfig(dim=64, n_heads=2, num_key_value_heads=1, head_dim=64, max_seq_len=128,
                                        intermediate_size=128))
