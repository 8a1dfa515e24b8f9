"""ctypes binding of liblorafusion_hip.so (the C ABI declared in include/lorafusion_hip.h).

There is no fallback: if the shared library is missing, ``lib()`` raises.
"""

from __future__ import annotations

import ctypes
import os
from typing import Sequence

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liblorafusion_hip.so")

LF_BF16, LF_F16 = 0, 1
LF_MASK_BITS = 0x100  # OR into dtype: the call's keep-masks are bit-packed ([M, K/8] bytes, element k = bit k & 7 of byte k >> 3)
LF_MAX_SEG = 32
LF_OP_XA, LF_OP_DYS_DYB, LF_OP_DA, LF_OP_FWD, LF_OP_BWD, LF_OP_NF4_FWD, LF_OP_NF4_BWD = range(7)
LF_OK, LF_EINVAL, LF_ESHAPE, LF_EWORKSPACE, LF_ELAUNCH, LF_ELIMIT, LF_ESTATIC = 0, -1, -2, -3, -4, -5, -6
LF_STATIC_SCRATCH_BYTES = 32 << 20

EXPORTS = (
    "lf_version", "lf_strerror", "lf_workspace_bytes", "lf_lora_xa", "lf_lora_xw_sb", "lf_lora_dys_dyb",
    "lf_lora_da", "lf_lora_dyw_dsa", "lf_lora_fwd", "lf_lora_bwd", "lf_gemm", "lf_nf4_dequant", "lf_dropout_mask",
    "lf_lora_xa_seeded", "lf_lora_fwd_seeded", "lf_nf4_lora_fwd", "lf_nf4_lora_bwd", "lf_lora_bwd_static", "lf_set_tile_cfg", "lf_gemm_plan",
    "lf_rmsnorm_fwd", "lf_rmsnorm_bwd_workspace", "lf_rmsnorm_bwd", "lf_silu_mul_fwd", "lf_silu_mul_bwd",
    "lf_lora_xa_silu_mul", "lf_swiglu_lora_fwd", "lf_mask_pack", "lf_mask_unpack",
)


class Routing(ctypes.Structure):
    """struct lf_routing."""

    _fields_ = [
        ("n_seg", ctypes.c_int32),
        ("block_size_m", ctypes.c_int32),
        ("n_blocks", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
        ("block_table", ctypes.c_void_p),
        ("block_scale", ctypes.c_void_p),
        ("block_p", ctypes.c_void_p),
        ("scale", ctypes.c_float),
        ("p", ctypes.c_float),
        ("seg_first_block", ctypes.c_int32 * LF_MAX_SEG),
        ("seg_rank", ctypes.c_int32 * LF_MAX_SEG),
    ]


class NF4Weight(ctypes.Structure):
    """struct lf_nf4_weight."""

    _fields_ = [
        ("packed", ctypes.c_void_p),
        ("absmax", ctypes.c_void_p),
        ("code2", ctypes.c_void_p),
        ("absmax2", ctypes.c_void_p),
        ("offset", ctypes.c_void_p),
        ("blocksize", ctypes.c_int32),
        ("blocksize2", ctypes.c_int32),
        ("dense", ctypes.c_void_p),
        ("dense_valid", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
    ]


_lib = None


def lib() -> ctypes.CDLL:
    """Load the HIP library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} not found: build it with `python -m lorafusion_amd.csrc.build` "
            "(hipcc, gfx950). There is no non-HIP fallback."
        )
    l = ctypes.CDLL(LIB_PATH)
    vp, i, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
    rp = ctypes.POINTER(Routing)
    l.lf_version.restype = i
    l.lf_strerror.restype = ctypes.c_char_p
    l.lf_strerror.argtypes = [i]
    l.lf_workspace_bytes.restype = sz
    l.lf_workspace_bytes.argtypes = [i, i, i, i, i, rp]
    l.lf_lora_xa.argtypes = [vp, vp, vp, vp, vp, sz, i, i, i, rp, i, vp]
    l.lf_lora_xw_sb.argtypes = [vp, vp, vp, vp, vp, vp, i, i, i, i, rp, i, vp]
    l.lf_lora_dys_dyb.argtypes = [vp, vp, vp, vp, vp, vp, sz, i, i, i, rp, i, vp]
    l.lf_lora_da.argtypes = [vp, vp, vp, vp, vp, sz, i, i, i, rp, i, vp]
    l.lf_lora_dyw_dsa.argtypes = [vp, vp, vp, vp, vp, vp, i, i, i, i, rp, i, vp]
    l.lf_lora_fwd.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, vp, sz, i, i, i, i, rp, i, vp]
    l.lf_lora_bwd.argtypes = [vp] * 12 + [sz, i, i, i, i, rp, i, vp]
    l.lf_lora_bwd_static.argtypes = [vp] * 11 + [i, i, i, i, rp, i, vp]
    l.lf_gemm.argtypes = [vp, vp, vp, vp, i, i, i, i, i, i, vp]
    l.lf_set_tile_cfg.argtypes = [i]
    l.lf_gemm_plan.argtypes = [i, i, i, i, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int)]
    l.lf_nf4_dequant.argtypes = [vp, vp, vp, vp, vp, vp, ctypes.c_int64, i, i, i, vp]
    l.lf_dropout_mask.argtypes = [vp, i, i, ctypes.c_float, rp, ctypes.c_uint64, vp]
    l.lf_lora_xa_seeded.argtypes = [vp, vp, vp, vp, i, i, i, rp, ctypes.c_uint64, i, vp]
    l.lf_lora_fwd_seeded.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, vp, ctypes.c_size_t, i, i, i, i, rp, ctypes.c_uint64, i, vp]
    wp = ctypes.POINTER(NF4Weight)
    l.lf_nf4_lora_fwd.argtypes = [vp, wp, vp, vp, vp, vp, vp, vp, vp, sz, i, i, i, i, rp, i, vp]
    l.lf_nf4_lora_bwd.argtypes = [vp, vp, wp, vp, vp, vp, vp, vp, vp, vp, vp, vp, sz, i, i, i, i, rp, i, vp]
    i64, f32 = ctypes.c_int64, ctypes.c_float
    l.lf_rmsnorm_fwd.argtypes = [vp, vp, vp, vp, i, i, f32, i, vp]
    l.lf_rmsnorm_bwd_workspace.restype = sz
    l.lf_rmsnorm_bwd_workspace.argtypes = [i, i]
    l.lf_rmsnorm_bwd.argtypes = [vp, vp, vp, vp, vp, vp, i, i, i, vp, sz, vp]
    l.lf_silu_mul_fwd.argtypes = [vp, vp, vp, i, i, i64, i64, i64, i, vp]
    l.lf_silu_mul_bwd.argtypes = [vp, vp, vp, vp, vp, i, i, i64, i64, i64, i64, i64, i, vp]
    l.lf_lora_xa_silu_mul.argtypes = [vp, vp, i64, vp, vp, vp, ctypes.c_uint64, vp, vp, i, i, i, rp, i, vp]
    l.lf_swiglu_lora_fwd.argtypes = [vp, vp, i64, vp, vp, vp, vp, vp, ctypes.c_uint64, vp, vp, vp, vp, vp, ctypes.c_size_t, i, i, i, i, rp, i, vp]
    l.lf_mask_pack.argtypes = [vp, vp, i, i, vp]
    l.lf_mask_unpack.argtypes = [vp, vp, i, i, vp]
    for name in EXPORTS:
        if name not in ("lf_strerror", "lf_workspace_bytes", "lf_rmsnorm_bwd_workspace"):
            getattr(l, name).restype = i
    _lib = l
    return l


def check(rc: int, what: str) -> None:
    if rc != 0:
        raise RuntimeError(f"{what} failed: {lib().lf_strerror(rc).decode()} (code {rc})")


def dtype_id(dtype: torch.dtype) -> int:
    if dtype == torch.bfloat16:
        return LF_BF16
    if dtype == torch.float16:
        return LF_F16
    raise ValueError(f"Unsupported dtype: {dtype}; expected torch.bfloat16 or torch.float16.")


def ptr(t: torch.Tensor | None):
    return None if t is None else t.data_ptr()


def ptr_array(tensors: Sequence[torch.Tensor]):
    arr = (ctypes.c_void_p * len(tensors))()
    for k, t in enumerate(tensors):
        arr[k] = t.data_ptr()
    return arr


def stream_of(t: torch.Tensor):
    return torch.cuda.current_stream(t.device).cuda_stream


def require_gpu(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU (got device {t.device}); the HIP kernels have no CPU path.")


def workspace(nbytes: int, device) -> torch.Tensor | None:
    """Scratch memory for one call (torch's caching allocator keeps this cheap and stream-safe)."""
    if nbytes == 0:
        return None
    return torch.empty(nbytes, dtype=torch.uint8, device=device)


def single_routing(rank: int, scale: float, p: float) -> Routing:
    r = Routing()
    r.n_seg = 1
    r.block_size_m = 128
    r.n_blocks = 0
    r.block_table = None
    r.block_scale = None
    r.block_p = None
    r.scale = float(scale)
    r.p = float(p)
    r.seg_first_block[0] = 0
    r.seg_rank[0] = int(rank)
    return r


def multi_routing(padded_seq_len_list, rank_list, block_table, block_scale, block_p, block_size_m: int) -> Routing:
    if len(padded_seq_len_list) > LF_MAX_SEG:
        raise ValueError(f"At most {LF_MAX_SEG} adapter segments per call, got {len(padded_seq_len_list)}.")
    r = Routing()
    r.n_seg = len(padded_seq_len_list)
    r.block_size_m = int(block_size_m)
    r.n_blocks = int(block_table.shape[0])
    r.block_table = block_table.data_ptr()
    r.block_scale = block_scale.data_ptr()
    r.block_p = block_p.data_ptr()
    r.scale = 1.0
    r.p = 0.0
    fb = 0
    for k, (padded, rank) in enumerate(zip(padded_seq_len_list, rank_list, strict=True)):
        r.seg_first_block[k] = fb
        r.seg_rank[k] = int(rank)
        fb += int(padded) // int(block_size_m)
    return r


def round_rank(max_rank: int) -> int:
    """Columns of S / dS: the largest rank rounded up to the MFMA k-step of 16."""
    return (int(max_rank) + 15) // 16 * 16
