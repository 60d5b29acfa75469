"""ctypes binding of ``libmaester_attn.so`` (C ABI: ``include/maester_attn.h``).

The library is loaded from the package directory; there is no fallback: if it has not been built
(``python -m maester_amd.build``) every entry point raises.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import (POINTER, Structure, c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p)

import torch

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libmaester_attn.so")

MA_ABI_VERSION = 10200   # include/maester_attn.h: the struct layouts and signatures bound below
MA_OK = 0
MA_ERR_BAD_ARG = -1
MA_ERR_UNSUPPORTED = -2
MA_ERR_LAUNCH = -3
MA_DTYPE_F32 = 0
MA_DTYPE_BF16 = 1
MA_TILE = 128
MA_DOC_BLOCK = 32
MA_WORK_COUNTERS = 64
MA_TILE_MAP_STATIC_BYTES = 4 << 20
MA_BWD_DELTA, MA_BWD_DKV, MA_BWD_DQ, MA_BWD_ALL = 1, 2, 4, 7

EXPORTS = (
    "ma_version", "ma_last_error", "ma_probe_mfma", "ma_tile_map_workspace_bytes", "ma_tile_map_build", "ma_tile_map_build_static", "ma_packed_ids_build", "ma_rmsnorm_bwd_workspace_bytes", "ma_rmsnorm_fwd", "ma_rmsnorm_bwd", "ma_ce_valid_count", "ma_ce_rows", "ma_ce_loss_reduce", "ma_transpose", "ma_prologue_fwd",
    "ma_prologue_bwd_workspace_bytes", "ma_prologue_bwd", "ma_attn_fwd", "ma_attn_bwd_workspace_bytes", "ma_attn_bwd_ds_workspace_bytes",
    "ma_attn_bwd", "ma_attn_bwd_stages",
)


class MaTensor4(Structure):
    _fields_ = [("ptr", c_void_p), ("stride_b", c_int64), ("stride_s", c_int64), ("stride_h", c_int64)]


class MaTileMap(Structure):
    _fields_ = [(n, c_void_p) for n in (
        "kv_num_blocks", "kv_indices", "full_kv_num_blocks", "full_kv_indices",
        "q_num_blocks", "q_indices", "full_q_num_blocks", "full_q_indices", "q_tile_order", "kv_tile_order",
        "block_doc_range", "work_counters", "tile_slot", "tile_count")] + [("visited_tiles", c_int64)]


class MaesterAttnError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"libmaester_attn error {code}: {message}")
        self.code = code
        self.message = message


_lib = None


def lib() -> ctypes.CDLL:
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build the HIP library first (python -m maester_amd.build). "
            "There is no CPU or PyTorch fallback for this path.")
    L = ctypes.CDLL(LIB_PATH)
    T4 = POINTER(MaTensor4)
    TM = POINTER(MaTileMap)
    L.ma_version.restype = c_int
    L.ma_version.argtypes = []
    if L.ma_version() != MA_ABI_VERSION:
        raise RuntimeError(f"{LIB_PATH} was built from header version {L.ma_version()}, this binding is for "
                           f"{MA_ABI_VERSION}: rebuild the library (python -m maester_amd.build)")
    L.ma_last_error.restype = c_char_p
    L.ma_last_error.argtypes = []
    L.ma_probe_mfma.restype = c_int
    L.ma_probe_mfma.argtypes = [c_int, c_int, c_int, c_void_p, c_void_p]
    L.ma_tile_map_workspace_bytes.restype = c_size_t
    L.ma_tile_map_workspace_bytes.argtypes = [c_int, c_int]
    L.ma_tile_map_build.restype = c_int
    L.ma_tile_map_build.argtypes = [c_void_p, c_int, c_int, c_int, c_int64, TM, c_void_p, c_size_t, c_void_p]
    L.ma_tile_map_build_static.restype = c_int
    L.ma_tile_map_build_static.argtypes = [c_void_p, c_int, c_int, c_int, c_int64, TM, c_void_p]
    L.ma_packed_ids_build.restype = c_int
    L.ma_packed_ids_build.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]
    L.ma_rmsnorm_bwd_workspace_bytes.restype = c_size_t
    L.ma_rmsnorm_bwd_workspace_bytes.argtypes = [c_int64, c_int]
    L.ma_rmsnorm_fwd.restype = c_int
    L.ma_rmsnorm_fwd.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_float, c_int, c_int, c_void_p]
    L.ma_ce_valid_count.restype = c_int
    L.ma_ce_valid_count.argtypes = [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p]
    L.ma_ce_rows.restype = c_int
    L.ma_ce_rows.argtypes = [c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int64, c_float, c_void_p, c_void_p, c_void_p, c_int,
                             c_int, c_void_p]
    L.ma_transpose.restype = c_int
    L.ma_transpose.argtypes = [c_void_p, c_void_p, c_int64, c_int64, c_int, c_int, c_void_p]
    L.ma_ce_loss_reduce.restype = c_int
    L.ma_ce_loss_reduce.argtypes = [c_void_p, c_int64, c_void_p, c_void_p, c_void_p]
    L.ma_rmsnorm_bwd.restype = c_int
    L.ma_rmsnorm_bwd.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_int64, c_int,
                                 c_int, c_int, c_void_p]
    L.ma_prologue_fwd.restype = c_int
    L.ma_prologue_fwd.argtypes = [T4, T4, T4, T4, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_float,
                                  c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]
    L.ma_prologue_bwd_workspace_bytes.restype = c_size_t
    L.ma_prologue_bwd_workspace_bytes.argtypes = [c_int] * 5
    L.ma_prologue_bwd.restype = c_int
    L.ma_prologue_bwd.argtypes = [T4, T4, T4, T4, T4, T4, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p,
                                  c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_int, c_int,
                                  c_int, c_int, c_int, c_int, c_void_p]
    L.ma_attn_fwd.restype = c_int
    L.ma_attn_fwd.argtypes = [T4, T4, T4, T4, c_void_p, TM, c_void_p, c_int, c_int64, c_float, c_int, c_int, c_int,
                              c_int, c_int, c_int, c_void_p]
    L.ma_attn_bwd_workspace_bytes.restype = c_size_t
    L.ma_attn_bwd_workspace_bytes.argtypes = [c_int] * 5
    L.ma_attn_bwd_ds_workspace_bytes.restype = c_size_t
    L.ma_attn_bwd_ds_workspace_bytes.argtypes = [c_int, c_int, c_int, c_int64]
    L.ma_attn_bwd.restype = c_int
    L.ma_attn_bwd.argtypes = [T4, T4, T4, T4, T4, c_void_p, T4, T4, T4, TM, c_void_p, c_int, c_int64, c_float,
                              c_void_p, c_size_t, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]
    L.ma_attn_bwd_stages.restype = c_int
    L.ma_attn_bwd_stages.argtypes = L.ma_attn_bwd.argtypes[:-1] + [c_int, c_void_p]
    _lib = L
    return L


def check(rc: int) -> None:
    if rc != MA_OK:
        raise MaesterAttnError(rc, lib().ma_last_error().decode())


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.bfloat16:
        return MA_DTYPE_BF16
    if dtype == torch.float32:
        return MA_DTYPE_F32
    raise TypeError(f"maester_amd supports bfloat16 and float32 activations, got {dtype}")


def tensor4(t: torch.Tensor) -> MaTensor4:
    """Descriptor of a [B,S,H,D] tensor (any strides, last dim contiguous)."""
    if t.dim() != 4 or t.stride(3) != 1:
        raise ValueError(f"expected a [B,S,H,D] tensor with a contiguous last dim, got strides {t.stride()}")
    return MaTensor4(t.data_ptr(), t.stride(0), t.stride(1), t.stride(2))


def ptr(t: torch.Tensor | None):
    return None if t is None else c_void_p(t.data_ptr())


def current_stream(device) -> c_void_p:
    return c_void_p(torch.cuda.current_stream(device).cuda_stream)


def require_gpu(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(
            f"{what}: tensors must live on an MI355X (got device {t.device}); this path has no CPU fallback")
