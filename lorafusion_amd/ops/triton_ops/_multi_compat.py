"""Reference call signatures of the multi-adapter kernel wrappers on top of the HIP ops.

The reference hands its kernels per-block device-pointer tables built from per-adapter tensors
(``construct_s_and_b_ptrs_list``, lorafusion/ops/triton_ops/fused_multi_lora_xw_sb.py:21-62); the HIP
kernels take the per-adapter tensors themselves, so the "pointer lists" here simply carry them.
"""

from __future__ import annotations

import torch

from lorafusion_amd.ops import hip_ops
from lorafusion_amd.ops.hip_ops import FUSED_MULTI_LORA_BLOCK_SIZE_M


class TensorPtrList(list):
    """What ``construct_*_ptrs_list`` returns in place of an int64 pointer tensor: the tensors."""


def _block_size(block_size_m, config):
    cfg_bs = getattr(config, "block_size_m", None) if config is not None else FUSED_MULTI_LORA_BLOCK_SIZE_M
    if cfg_bs is None:
        cfg_bs = FUSED_MULTI_LORA_BLOCK_SIZE_M
    if block_size_m is not None and block_size_m != cfg_bs:
        raise ValueError(
            f"lora_kernel_config.block_size_m != input block_size_m. lora_kernel_config.block_size_m: {cfg_bs}, "
            f"block_size_m: {block_size_m}."
        )
    if cfg_bs != FUSED_MULTI_LORA_BLOCK_SIZE_M:
        raise ValueError(f"the HIP kernels route in blocks of {FUSED_MULTI_LORA_BLOCK_SIZE_M} rows, got {cfg_bs}.")
    return cfg_bs


def _lists(ptrs_a, ptrs_b, raw_a, raw_b, what):
    if raw_a is not None and raw_b is not None:
        return list(raw_a), list(raw_b)
    if isinstance(ptrs_a, TensorPtrList) and isinstance(ptrs_b, TensorPtrList):
        return list(ptrs_a), list(ptrs_b)
    if ptrs_a is not None or ptrs_b is not None:
        raise ValueError(f"raw device-pointer tables are not supported; pass {what} or the lists returned by construct_*_ptrs_list.")
    raise ValueError(f"Either {what} or the pointer lists must be provided.")


def _routing(row_tensors, rank_list, table, block_scale, block_p, M, bs):
    padded = [int(t.shape[0]) for t in row_tensors]
    for n in padded:
        if n % bs != 0:
            raise ValueError(f"every per-adapter tensor must cover whole blocks of {bs} rows, got {n}.")
    if sum(padded) != M:
        raise ValueError(f"per-adapter rows {padded} do not add up to M = {M}.")
    dev = table.device
    if block_scale is None:
        block_scale = torch.ones(table.shape[0], dtype=torch.float32, device=dev)
    if block_p is None:
        block_p = torch.zeros(table.shape[0], dtype=torch.float32, device=dev)
    return hip_ops.MultiRouting(padded, rank_list, table, block_scale, block_p), padded


def _pack_rows(tensors, M, R, dtype, device):
    full = torch.zeros((M, R), dtype=dtype, device=device)
    cur = 0
    for t in tensors:
        full[cur:cur + t.shape[0], : t.shape[1]] = t
        cur += t.shape[0]
    return full


def construct_s_and_b_ptrs_list(raw_s_list, raw_b_list, block_size_m, *, return_tensor_list: bool = False):
    _block_size(block_size_m, None)
    s_list = b_list = None
    if return_tensor_list:
        s_list, b_list = [], []
        for s, b in zip(raw_s_list, raw_b_list, strict=True):
            nb = (s.shape[0] + block_size_m - 1) // block_size_m
            s_list.extend([s] * nb)
            b_list.extend([b] * nb)
    return TensorPtrList(raw_s_list), TensorPtrList(raw_b_list), s_list, b_list


def construct_ds_and_a_ptrs_list(raw_ds_list, raw_a_list, block_size_m, *, return_tensor_list: bool = False):
    return construct_s_and_b_ptrs_list(raw_ds_list, raw_a_list, block_size_m, return_tensor_list=return_tensor_list)


def fused_multi_lora_xw_sb(x, w, *, block_to_lookup_table, block_to_alpha, max_r, total_r, s_ptrs_list=None,
                           b_ptrs_list=None, raw_s_list=None, raw_b_list=None, bias=None, init_zeros: bool = False,
                           block_size_m=None, config=None, **kwargs):
    """``y = x w^T + alpha_i * s_i b_i^T`` per adapter segment (fused_multi_lora_xw_sb.py:221-339).

    ``raw_s_list[i]`` is ``[padded_rows_i, r_i]``, ``raw_b_list[i]`` ``[N, r_i]``.  Rows of a padded
    block beyond its valid count get the base product only (the reference leaves them unwritten).
    """
    if x.shape[1] != w.shape[1]:
        raise ValueError(f"Incompatible dimensions: {x.shape[1]} != {w.shape[1]}. x: {x.shape}, w: {w.shape}")
    bs = _block_size(block_size_m, config)
    s_list, b_list = _lists(s_ptrs_list, b_ptrs_list, raw_s_list, raw_b_list, "raw_s_list and raw_b_list")
    rank_list = [int(b.shape[1]) for b in b_list]
    routing, _ = _routing(s_list, rank_list, block_to_lookup_table, block_to_alpha, None, x.shape[0], bs)
    s_full = _pack_rows(s_list, x.shape[0], routing.R, x.dtype, x.device)
    return hip_ops.fused_multi_lora_xw_sb(x, w, s_full, [b.contiguous() for b in b_list], routing, bias)


def fused_multi_lora_dys_dyb(dy, block_to_lookup_table, block_to_alpha, max_r, total_r, s_ptrs_list=None,
                             b_ptrs_list=None, raw_s_list=None, raw_b_list=None, *, block_size_m=None, config=None,
                             **kwargs):
    """``db_i = alpha_i dy_i^T s_i``, ``ds_i = alpha_i dy_i b_i`` (fused_multi_lora_dys_dyb.py:188-321).
    Returns ``(db_list, ds_list)`` with ``ds_i`` of shape ``[padded_rows_i, r_i]``."""
    bs = _block_size(block_size_m, config)
    s_list, b_list = _lists(s_ptrs_list, b_ptrs_list, raw_s_list, raw_b_list, "raw_s_list and raw_b_list")
    rank_list = [int(b.shape[1]) for b in b_list]
    routing, padded = _routing(s_list, rank_list, block_to_lookup_table, block_to_alpha, None, dy.shape[0], bs)
    s_full = _pack_rows(s_list, dy.shape[0], routing.R, dy.dtype, dy.device)
    db_list, ds = hip_ops.fused_multi_lora_dys_dyb(dy, s_full, [b.contiguous() for b in b_list], routing)
    ds_list, cur = [], 0
    for n, r in zip(padded, rank_list):
        ds_list.append(ds[cur:cur + n, :r].contiguous())
        cur += n
    return db_list, ds_list


def fused_multi_lora_dyw_dsa(dy, w, *, raw_ds_list, raw_a_list, block_to_dropout_p, block_to_lookup_table, max_r,
                             init_zeros: bool = False, enable_dropout: bool = False, dropout_mask=None,
                             block_size_m=None, config=None, **kwargs):
    """``dx = dy w + where(mask, ds_i a_i / (1 - p_i), 0)`` (fused_multi_lora_dyw_dsa.py:188-305)."""
    bs = _block_size(block_size_m, config)
    if enable_dropout and dropout_mask is None:
        raise ValueError("dropout_mask must be provided if enable_dropout is True")
    rank_list = [int(a.shape[0]) for a in raw_a_list]
    p = block_to_dropout_p.to(torch.float32) if enable_dropout else None
    routing, _ = _routing(raw_ds_list, rank_list, block_to_lookup_table, None, p, dy.shape[0], bs)
    ds_full = _pack_rows(raw_ds_list, dy.shape[0], routing.R, dy.dtype, dy.device)
    mask = dropout_mask if enable_dropout else None
    return hip_ops.fused_multi_lora_dyw_dsa(dy, w, ds_full, [a.contiguous() for a in raw_a_list], routing, mask)
