"""Block-sparse tile map (torch ``BlockMask`` format) built on the GPU from ``document_ids``.

Replaces the two per-step ``create_block_mask(make_document_mask_wrapper(...), B, None, S, S)``
calls of maester/models/gemma/model.py:694-730.
"""
from __future__ import annotations

from dataclasses import dataclass
from ctypes import byref, c_void_p

import torch

from . import _lib

TILE = _lib.MA_TILE


@dataclass
class TileMap:
    """The eight ``BlockMask`` tensors (head dim 1) plus the mask parameters they were built for.

    Field names, shapes ([B,1,T] / [B,1,T,T]) and dtype (int32) are those of
    ``torch.nn.attention.flex_attention.BlockMask``; ``BLOCK_SIZE`` is (128, 128)."""
    kv_num_blocks: torch.Tensor
    kv_indices: torch.Tensor
    full_kv_num_blocks: torch.Tensor
    full_kv_indices: torch.Tensor
    q_num_blocks: torch.Tensor
    q_indices: torch.Tensor
    full_q_num_blocks: torch.Tensor
    full_q_indices: torch.Tensor
    seq_len: int
    causal: bool
    window: int | None
    BLOCK_SIZE: tuple = (TILE, TILE)
    # launch schedules (not part of BlockMask): tile rows b*T+i by descending work, int32 [B*T]
    q_tile_order: torch.Tensor | None = None
    kv_tile_order: torch.Tensor | None = None
    # (min, max) document id of every 32-row block, int64 [B, 2*ceil(S/64), 2]; None without document ids
    block_doc_range: torch.Tensor | None = None
    # work queues of the attention kernels, int32 [64], zeroed by the build (launches that share a
    # tile map must be stream-ordered); None = one workgroup per work item
    work_counters: torch.Tensor | None = None
    # compact numbering of the visited tiles, int32 [B,T,T] (-1: never visited), and their number, int32 [1]:
    # the backward indexes its dS workspace with it
    tile_slot: torch.Tensor | None = None
    tile_count: torch.Tensor | None = None
    _visited: int | None = None
    _hand_over: bool | None = None   # the backward's choice of path for this map (attention.decide_hand_over)
    last_backward_path: str | None = None
    _last_stream: object = None      # the torch stream of the last launch that used the work queues

    def order_on_current_stream(self, device) -> None:
        """The work queues are shared by every launch that uses this map, so two launches must never
        overlap.  Launches on one stream are ordered anyway; when a launch comes on another stream than the
        one before, that stream is made to wait for everything queued on the previous one."""
        if self.work_counters is None:
            return
        cur = torch.cuda.current_stream(device)
        last = self._last_stream
        if last is not None and last != cur and not torch.cuda.is_current_stream_capturing():
            cur.wait_stream(last)
        self._last_stream = cur

    NAMES = ("kv_num_blocks", "kv_indices", "full_kv_num_blocks", "full_kv_indices",
             "q_num_blocks", "q_indices", "full_q_num_blocks", "full_q_indices")

    def as_dict(self) -> dict:
        return {n: getattr(self, n) for n in self.NAMES}

    def c_struct(self) -> _lib.MaTileMap:
        ptrs = [c_void_p(getattr(self, n).data_ptr()) for n in self.NAMES]
        ptrs += [None if t is None else c_void_p(t.data_ptr()) for t in (self.q_tile_order, self.kv_tile_order, self.block_doc_range,
                                                                           self.work_counters, self.tile_slot, self.tile_count)]
        return _lib.MaTileMap(*ptrs, self._visited or 0)

    def visited_tiles(self) -> int:
        """Number of visited (partial or full) tiles, read back from the device on first use (one
        synchronisation per map; the map of a training step is shared by all layers) and kept."""
        if self._visited is None:
            if self.tile_count is None:
                self._visited = 0
            else:
                # the count is written by the build, on the stream the build ran on: wait for THAT stream (the
                # caller may be on another one, where .item() would read the count before it exists)
                if self._last_stream is not None and not torch.cuda.is_current_stream_capturing():
                    self._last_stream.synchronize()
                self._visited = int(self.tile_count.item())
        return self._visited

    @property
    def seq_lengths(self):
        return (self.seq_len, self.seq_len)

    def sparsity(self) -> float:
        """Fraction of tiles never visited (the skipped-tile ratio)."""
        B, _, T = self.kv_num_blocks.shape
        visited = int(self.kv_num_blocks.sum()) + int(self.full_kv_num_blocks.sum())
        return 1.0 - visited / float(B * T * T)


def build_tile_map(document_ids: torch.Tensor | None, batch_size: int, seq_len: int, causal: bool = True,
                   sliding_window: int | None = None, device=None, static_scratch: bool = False) -> TileMap:
    """``document_ids``: int64 [B,S] on the GPU, or ``None`` for the plain causal / sliding-window
    mask (maester/models/gemma/model.py:227-228).  ``sliding_window`` is inclusive (``q - kv <= W``,
    model.py:206-207) and implies causality.  ``static_scratch``: go through ``ma_tile_map_build_static``,
    whose scratch is a fixed array inside the library instead of a workspace allocated here (the
    output tensors are still torch's; the C entry point itself allocates nothing)."""
    if document_ids is not None:
        _lib.require_gpu(document_ids, "build_tile_map")
        if document_ids.shape != (batch_size, seq_len):
            raise ValueError(f"document_ids shape {tuple(document_ids.shape)} != {(batch_size, seq_len)}")
        document_ids = document_ids.detach().to(torch.long).contiguous()
        device = document_ids.device
    elif device is None:
        device = torch.device("cuda", torch.cuda.current_device())
    device = torch.device(device)
    L = _lib.lib()
    T = (seq_len + TILE - 1) // TILE
    nums = torch.empty(4, batch_size, 1, T, dtype=torch.int32, device=device)
    idxs = torch.empty(4, batch_size, 1, T, T, dtype=torch.int32, device=device)
    order = torch.empty(2, batch_size * T, dtype=torch.int32, device=device)
    tm = TileMap(nums[0], idxs[0], nums[1], idxs[1], nums[2], idxs[2], nums[3], idxs[3],
                 seq_len=seq_len, causal=bool(causal), window=sliding_window, q_tile_order=order[0],
                 kv_tile_order=order[1],
                 work_counters=torch.empty(_lib.MA_WORK_COUNTERS, dtype=torch.int32, device=device),
                 tile_slot=torch.empty(batch_size, T, T, dtype=torch.int32, device=device),
                 tile_count=torch.empty(1, dtype=torch.int32, device=device))
    if document_ids is not None:
        nblk = 2 * ((seq_len + 63) // 64)   # two 32-row blocks per 64-row step, the last step padded
        tm.block_doc_range = torch.empty(batch_size, nblk, 2, dtype=torch.int64, device=device)
    cs = tm.c_struct()
    tm._last_stream = torch.cuda.current_stream(device)
    if static_scratch:
        with torch.cuda.device(device):
            rc = L.ma_tile_map_build_static(_lib.ptr(document_ids), batch_size, seq_len, 1 if causal else 0,
                                            -1 if sliding_window is None else int(sliding_window), byref(cs),
                                            _lib.current_stream(device))
        _lib.check(rc)
        return tm
    ws_bytes = L.ma_tile_map_workspace_bytes(batch_size, seq_len)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=device)
    with torch.cuda.device(device):
        rc = L.ma_tile_map_build(_lib.ptr(document_ids), batch_size, seq_len, 1 if causal else 0,
                                 -1 if sliding_window is None else int(sliding_window), byref(cs),
                                 _lib.ptr(ws), ws_bytes, _lib.current_stream(device))
    _lib.check(rc)
    return tm
