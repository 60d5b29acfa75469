"""The GemmaAttention-compatible module end to end on the GPU (counterpart of
maester/models/gemma/model.py:344-440 with the per-step inputs of 654-757): q/k/v are strided views
of the fused qkv projection, one step's tile maps serve a global and a local layer, gradients reach
the projection and norm weights.  Checked against the oracle fed with the same projections."""
import pytest
import torch

from conftest import check_bf16, max_abs, rel_l2
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
        check_bf16(y, want, ("module output", kind))
        got = (attn.qkv_proj.weight.grad, attn.o_proj.weight.grad, attn.query_norm.weight.grad, attn.key_norm.weight.grad)
        for name, g, leaf in zip(("qkv_proj", "o_proj", "query_norm", "key_norm"), got, leaves):
            assert rel_l2(g.float().cpu(), leaf.grad) <= 2e-2, (kind, name, rel_l2(g.float().cpu(), leaf.grad))


def _reference_layer(layer, h, step, window):
    """One decoder layer in fp32 on the CPU: the oracle's norm and attention path, torch GEMMs."""
    from oracle import prologue as P

    def w(mod):
        return mod.weight.detach().float().cpu()
    a = layer.self_attn
    B, S, _ = h.shape
    x = P.rms_norm(h, w(layer.input_layernorm))
    qkv = x @ w(a.qkv_proj).t()
    xq, xk, xv = qkv.split([a.q_size, a.kv_size, a.kv_size], dim=-1)
    o = A.full_path(xq.view(B, S, a.num_heads, a.head_dim), xk.view(B, S, a.num_kv_heads, a.head_dim),
                    xv.view(B, S, a.num_kv_heads, a.head_dim), w(a.query_norm), w(a.key_norm), a.rope_cos.float().cpu(),
                    a.rope_sin.float().cpu(), step.position_ids.cpu(), step.document_ids.cpu(), a.scaling, True, window)
    h = h + P.rms_norm(o.reshape(B, S, -1) @ w(a.o_proj).t(), w(layer.post_attention_layernorm))
    x = P.rms_norm(h, w(layer.pre_feedforward_layernorm))
    m = layer.mlp
    x = (torch.nn.functional.gelu(x @ w(m.gate_proj).t(), approximate="tanh") * (x @ w(m.up_proj).t())) @ w(m.down_proj).t()
    return h + P.rms_norm(x, w(layer.post_feedforward_layernorm))


def test_layer_stack_shares_the_steps_tile_maps(gpu):
    """A local and a global decoder layer plus the final norm (counterpart of GemmaModel.forward,
    maester/models/gemma/model.py:524-560) against the same stack in fp32 on the CPU."""
    from maester_amd.gemma_layers import GemmaLayerConfig, GemmaModel
    from oracle import prologue as P
    torch.manual_seed(1)
    cfg = GemmaLayerConfig(dim=256, n_heads=4, num_key_value_heads=2, head_dim=128, max_seq_len=512, sliding_window_size=64,
                           intermediate_size=512, n_layers=2, attn_types=("local_sliding", "global"))
    B, S = 2, 290
    rows = [[(0, 0, 90), (1, 90, 200)], [(2, 0, 150), (3, 150, 100)]]
    pos, doc = packed_ids.packed_collate_ids(rows, S)
    model = GemmaModel(cfg).to(gpu).to(torch.bfloat16)
    model.init_weights(0.06)
    with torch.no_grad():
        for p in model.parameters():
            if p.dim() == 1:
                p.copy_(0.1 * torch.randn_like(p))           # non-trivial norm weights
    assert [l.attn_type for l in model.layers] == ["local_sliding", "global"]
    h = torch.randn(B, S, cfg.dim).to(torch.bfloat16)
    y = model(h.to(gpu), pos.to(gpu), doc.to(gpu))
    step = build_step_inputs(cfg, B, S, pos.to(gpu), doc.to(gpu))
    ref = h.float()
    for layer, window in zip(model.layers, (64, None)):
        ref = _reference_layer(layer, ref, step, window)
    ref = P.rms_norm(ref, model.norm.weight.detach().float().cpu())
    assert rel_l2(y.float().cpu(), ref) <= 2e-2, rel_l2(y.float().cpu(), ref)
    # gradients flow to every parameter, through both layers
    y.float().pow(2).mean().backward()
    assert all(p.grad is not None and torch.isfinite(p.grad.float()).all() and float(p.grad.float().abs().sum()) > 0
               for p in model.parameters())


def test_text_model_tokens_to_loss(gpu):
    """Tokens in, loss out (counterpart of GemmaTextModel.forward with labels, maester/models/gemma/model.py:654-769):
    embedding, two layers on one step's tile maps, final norm, fused linear + cross-entropy against the tied
    embedding table -- against the same computation in fp32 on the CPU with the oracle's pieces."""
    from maester_amd.gemma_layers import GemmaLayerConfig, GemmaTextModel
    from oracle import linear_ce as LCE
    from oracle import prologue as P
    torch.manual_seed(2)
    cfg = GemmaLayerConfig(dim=256, n_heads=4, num_key_value_heads=2, head_dim=128, max_seq_len=512, sliding_window_size=64,
                           intermediate_size=512, n_layers=2, attn_types=("local_sliding", "global"), vocab_size=1000)
    B, S = 2, 290
    rows = [[(0, 0, 90), (1, 90, 200)], [(2, 0, 150), (3, 150, 100)]]
    pos, doc = packed_ids.packed_collate_ids(rows, S)
    model = GemmaTextModel(cfg).to(gpu).to(torch.bfloat16)
    model.init_weights(0.06)
    assert {"tok_embeddings.weight", "model.norm.weight", "model.layers.0.self_attn.qkv_proj.weight"} <= set(model.state_dict())
    tokens = torch.randint(0, cfg.vocab_size, (B, S))
    labels = torch.roll(tokens, -1, 1)
    labels[:, :40] = -100                                      # prompt tokens masked
    labels[doc < 0] = -100                                     # padding
    loss = model(tokens.to(gpu), labels.to(gpu), pos.to(gpu), doc.to(gpu))
    assert loss.shape == () and loss.dtype == torch.float32

    step = build_step_inputs(cfg, B, S, pos.to(gpu), doc.to(gpu))
    emb = model.tok_embeddings.weight.detach().float().cpu()
    ref = emb[tokens] * float(torch.tensor(cfg.dim ** 0.5, dtype=torch.bfloat16))
    for layer, window in zip(model.model.layers, (64, None)):
        ref = _reference_layer(layer, ref, step, window)
    ref = P.rms_norm(ref, model.model.norm.weight.detach().float().cpu())
    want = LCE.linear_cross_entropy(ref.reshape(B * S, -1).numpy(), emb.numpy(), labels.reshape(-1).numpy())["loss"]
    assert abs(float(loss) - want) <= 2e-2 * max(1.0, abs(want)), (float(loss), want)

    loss.backward()
    assert all(p.grad is not None and torch.isfinite(p.grad.float()).all() and float(p.grad.float().abs().sum()) > 0
               for p in model.parameters())
    # the tied table gets gradient from both of its uses: the rows of tokens that were looked up and, through the loss, all rows
    logits = model(tokens.to(gpu), None, pos.to(gpu), doc.to(gpu))
    assert logits.shape == (B, S, cfg.vocab_size)
