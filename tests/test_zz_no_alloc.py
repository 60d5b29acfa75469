"""``ma_tile_map_build_static`` (the entry point that allocates nothing: its scratch is a fixed array
inside the library) against ``ma_tile_map_build`` (caller-provided workspace), through the C ABI:
bit-exact on every output, on two calls in a row, the second on a smaller input (the scratch keeps
the first call's contents)."""
from ctypes import byref

import pytest
import torch

from maester_amd import _lib, build_tile_map, workloads

pytestmark = pytest.mark.gpu

FIELDS = ("kv_num_blocks", "kv_indices", "full_kv_num_blocks", "full_kv_indices", "q_num_blocks", "q_indices", "tile_slot", "tile_count",
          "full_q_num_blocks", "full_q_indices", "q_tile_order", "kv_tile_order", "block_doc_range", "work_counters")


def _same(a, b):
    for f in FIELDS:
        x, y = getattr(a, f), getattr(b, f)
        assert (x is None) == (y is None), f
        if x is not None:
            assert torch.equal(x, y), f


def test_static_scratch_build_matches_the_workspace_build_twice_in_a_row(gpu):
    big = workloads.make("c4").to(gpu)                      # B=2, S=16384: 164 KB of scratch
    small = workloads.make("c2", B=1, S=1000).to(gpu)       # ragged, a fraction of the first call's scratch
    for wl, window in ((big, None), (small, 300), (small, None)):
        sp = wl.spec
        want = build_tile_map(wl.document_ids, sp.B, sp.S, True, window)
        got = build_tile_map(wl.document_ids, sp.B, sp.S, True, window, static_scratch=True)
        torch.cuda.synchronize()
        _same(got, want)
    # no document ids (plain causal mask), still on the used scratch
    _same(build_tile_map(None, 2, 700, True, 64, device=gpu, static_scratch=True), build_tile_map(None, 2, 700, True, 64, device=gpu))


def test_static_scratch_build_rejects_what_does_not_fit(gpu):
    L = _lib.lib()
    B, S = 16, 65536                                        # 16 * 512^2 tiles: 21 MB of scratch
    assert L.ma_tile_map_workspace_bytes(B, S) > _lib.MA_TILE_MAP_STATIC_BYTES
    tm = build_tile_map(None, 1, 128, True, None, device=gpu)       # any valid struct: rejected before it is used
    rc = L.ma_tile_map_build_static(None, B, S, 1, -1, byref(tm.c_struct()), None)
    assert rc == _lib.MA_ERR_UNSUPPORTED and b"scratch" in L.ma_last_error()


def _poison(tm):
    for f in FIELDS:
        t = getattr(tm, f)
        if t is not None:
            t.fill_(-7)


def test_static_scratch_build_allocates_no_device_memory(gpu):
    """The entry point itself, called straight through the C ABI on outputs that exist already: neither the
    driver's free memory nor torch's allocator moves across the call, and the outputs are those of the
    workspace build."""
    L = _lib.lib()
    wl = workloads.make("c2", B=2, S=3000).to(gpu)
    sp = wl.spec
    want = build_tile_map(wl.document_ids, sp.B, sp.S, True, None)
    got = build_tile_map(wl.document_ids, sp.B, sp.S, True, None, static_scratch=True)   # outputs allocated here, by torch
    torch.cuda.synchronize()
    _poison(got)
    cs = got.c_struct()
    stream = _lib.current_stream(gpu)
    doc = wl.document_ids.contiguous()
    torch.cuda.synchronize()
    before = (torch.cuda.mem_get_info(gpu)[0], torch.cuda.memory_allocated(gpu), torch.cuda.memory_reserved(gpu))
    rc = L.ma_tile_map_build_static(_lib.ptr(doc), sp.B, sp.S, 1, -1, byref(cs), stream)
    torch.cuda.synchronize()
    after = (torch.cuda.mem_get_info(gpu)[0], torch.cuda.memory_allocated(gpu), torch.cuda.memory_reserved(gpu))
    assert rc == _lib.MA_OK, L.ma_last_error()
    assert before == after, (before, after)
    _same(got, want)


def test_static_scratch_build_under_graph_capture(gpu):
    """What the entry point is for: recorded into a HIP graph (after one call outside it, which is where the
    library looks up its scratch address), replayed on fresh inputs with eager work in between; every replay
    gives the bits of the workspace build of the ids the replay saw."""
    L = _lib.lib()
    B, S = 2, 2500
    wls = [workloads.make(n, B=B, S=S).to(gpu) for n in ("c2", "c5", "c4")]     # three document laws
    doc = wls[0].document_ids.clone().contiguous()
    got = build_tile_map(doc, B, S, True, 512, static_scratch=True)        # warm: scratch address, outputs
    torch.cuda.synchronize()
    cs = got.c_struct()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rc = L.ma_tile_map_build_static(_lib.ptr(doc), B, S, 1, 512, byref(cs), _lib.current_stream(gpu))
    assert rc == _lib.MA_OK, L.ma_last_error()
    for wl in wls[1:] + wls[:1]:
        doc.copy_(wl.document_ids)
        _poison(got)
        graph.replay()
        torch.cuda.synchronize()
        want = build_tile_map(wl.document_ids, B, S, True, 512)              # eager work between the replays
        torch.cuda.synchronize()
        _same(got, want)
