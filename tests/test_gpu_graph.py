"""The attention launches under HIP graph capture: the library allocates nothing, never synchronises
and records no memset, and its work queues reset themselves on the device, so a training step's
attention can be captured once and replayed.  Every replay -- with eager work and synchronisations
between the replays -- must reproduce the eager result bit for bit."""
import pytest
import torch

from maester_amd import build_tile_map, workloads
from maester_amd.attention import attention_backward, attention_forward, backward_workspace_bytes

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name,B,S", [("c2", 2, 2048), ("c5", 1, 1536)])
def test_captured_step_replays_bit_for_bit(gpu, name, B, S):
    wl = workloads.make(name, B=B, S=S).to(gpu)
    sp = wl.spec
    q, k, v, do, ids = wl.xq, wl.xk, wl.xv, wl.dout, wl.document_ids
    tm = build_tile_map(ids, sp.B, sp.S, True, sp.window)
    ws = torch.empty(backward_workspace_bytes(sp.B, sp.S, sp.Hq, sp.Hkv, sp.D, q.dtype, True, tm), dtype=torch.uint8, device=gpu)
    bufs = (torch.empty_like(q), torch.empty_like(k), torch.empty_like(v), ws)

    def step():
        out, lse = attention_forward(q, k, v, tm, ids, wl.scale, True, sp.window)
        attention_backward(q, k, v, out, do, lse, tm, ids, wl.scale, True, sp.window, buffers=bufs)
        return out, lse

    out, lse = step()
    torch.cuda.synchronize()
    want = [t.clone() for t in (out, lse) + bufs[:3]]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g_out, g_lse = step()
    for rep in range(4):
        for t in (g_out, g_lse) + bufs[:3]:
            t.zero_()
        graph.replay()
        torch.cuda.synchronize()
        for name_, got, exp in zip(("out", "lse", "dq", "dk", "dv"), (g_out, g_lse) + bufs[:3], want):
            assert torch.equal(got, exp), (rep, name_)
        # the program's own eager work between the replays (same tile map, same work queues)
        e_out, _ = step()
        torch.cuda.synchronize()
        assert torch.equal(e_out, want[0])
    assert int(tm.work_counters.abs().sum()) == 0
