"""The GemmaAttention-compatible module end to end on the GPU (counterpart of
maester/models/gemma/model.py:344-440 with the per-step inputs of 654-757): q/k/v are strided views
of the fused qkv projection, one step's tile maps serve a global and a local layer, gradients reach
the projection and norm weights.  Checked against the oracle fed with the same projections."""
import pytest
import torch

from conftest import max_abs, rel_l2
from maester_amd import GemmaAttention, GemmaAttentionConfig, packed_ids
from maester_amd.gemma_attention import build_step_inputs
from oracle import attention as A

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda", 0)


def _reference(attn, h, step, window):
    """The same layer through the oracle in fp32 (projection weights and norm weights of ``attn``)."""
    B, S, _ = h.shape
    w_qkv = attn.qkv_proj.weight.detach().float().cpu().requires_grad_()
    w_o = attn.o_proj.weight.detach().float().cpu().requires_grad_()
    qw = attn.query_norm.weight.detach().float().cpu().requires_grad_()
    kw = attn.key_norm.weight.detach().float().cpu().requires_grad_()
    qkv = h.float().cpu() @ w_qkv.t()
    xq, xk, xv = qkv.split([attn.q_size, attn.kv_size, attn.kv_size], dim=-1)
    xq = xq.view(B, S, attn.num_heads, attn.head_dim)
    xk = xk.view(B, S, attn.num_kv_heads, attn.head_dim)
    xv = xv.view(B, S, attn.num_kv_heads, attn.head_dim)
    o = A.full_path(xq, xk, xv, qw, kw, attn.rope_cos.float().cpu(), attn.rope_sin.float().cpu(), step.position_ids.cpu(),
                    step.document_ids.cpu(), attn.scaling, True, window)
    return o.reshape(B, S, -1) @ w_o.t(), (w_qkv, w_o, qw, kw)


def test_global_and_local_layer_share_one_steps_inputs(gpu):
    torch.manual_seed(0)
    cfg = GemmaAttentionConfig(dim=256, n_heads=4, num_key_value_heads=2, head_dim=128, max_seq_len=512,
                               sliding_window_size=96, rope_wave_length={"local_sliding": 10_000, "global": 1_000_000},
                               rope_scaling={"factor": 8})
    B, S = 2, 333
    rows = [[(0, 0, 100), (1, 100, 150), (2, 250, 60)], [(3, 0, 333)]]      # (conversation, start, length); row 0 ends in padding
    pos, doc = packed_ids.packed_collate_ids(rows, S)
    step = build_step_inputs(cfg, B, S, pos.to(gpu), doc.to(gpu))
    assert step.local_map is not None and step.local_map is not step.global_map
    h = (0.5 * torch.randn(B, S, cfg.dim)).to(torch.bfloat16).to(gpu)
    dy = (0.1 * torch.randn(B, S, cfg.dim)).to(torch.bfloat16).to(gpu)
    for kind, window in (("global", None), ("local_sliding", 96)):
        attn = GemmaAttention(cfg, kind).to(gpu).to(torch.bfloat16)
        attn.init_weights(0.05)
        with torch.no_grad():                                              # non-trivial norm weights
            attn.query_norm.weight.copy_(0.1 * torch.randn(cfg.head_dim))
            attn.key_norm.weight.copy_(0.1 * torch.randn(cfg.head_dim))
        y = attn(h, step)
        y.backward(dy)
        want, leaves = _reference(attn, h, step, window)
        want.backward(dy.float().cpu())
        scale = max(1.0, float(want.detach().abs().max()))
        assert max_abs(y.float().cpu(), want.detach()) <= 2e-2 * scale and rel_l2(y.float().cpu(), want.detach()) <= 1e-2, kind
        got = (attn.qkv_proj.weight.grad, attn.o_proj.weight.grad, attn.query_norm.weight.grad, attn.key_norm.weight.grad)
        for name, g, leaf in zip(("qkv_proj", "o_proj", "query_norm", "key_norm"), got, leaves):
            assert rel_l2(g.float().cpu(), leaf.grad) <= 2e-2, (kind, name, rel_l2(g.float().cpu(), leaf.grad))
