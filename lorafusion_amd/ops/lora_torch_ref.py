"""Unfused PyTorch LoRA linear, single and segmented multi adapter.

The ``use_fused=False`` path of the patch layer; same signatures and semantics as
lorafusion/ops/lora_torch_ref.py:6-120 (dropout through ``torch.nn.functional.dropout`` while
grad is enabled; multi: one segment per adapter, cursor advancing by the padded length).
"""

from __future__ import annotations

import torch
import torch.nn.functional as F


def _lora_branch(x, lora_a, lora_b, alpha, dropout_p):
    if dropout_p > 0.0 and torch.is_grad_enabled():
        x = F.dropout(x, p=dropout_p)
    return (x @ lora_a.T @ lora_b.T) * alpha


def torch_ref_linear_lora(x, linear_w, lora_a, lora_b, alpha, dropout_p: float = 0.0, linear_bias=None):
    """``x @ W.T (+bias) + (dropout(x) @ A.T @ B.T) * alpha``."""
    base = F.linear(x, linear_w, linear_bias)
    return base + _lora_branch(x, lora_a, lora_b, alpha, dropout_p)


def torch_ref_linear_multi_lora(padded_x, linear_w, *, lora_a_list, lora_b_list, seq_len_list,
                                padded_seq_len_list, alpha_list, dropout_p_list, linear_bias=None):
    """Base linear on every row; adapter i's branch added on rows ``[cur, cur + seq_len_i)``."""
    result = F.linear(padded_x, linear_w, linear_bias)
    squeeze = result.ndim == 3
    flat = result.reshape(-1, result.shape[-1]) if squeeze else result
    xflat = padded_x.reshape(-1, padded_x.shape[-1]) if squeeze else padded_x
    cur = 0
    updates = []
    for n, padded, a, b, alpha, p in zip(seq_len_list, padded_seq_len_list, lora_a_list, lora_b_list,
                                         alpha_list, dropout_p_list, strict=True):
        updates.append((cur, n, _lora_branch(xflat[cur : cur + n], a, b, alpha, p)))
        cur += padded
    pieces, pos = [], 0
    for cur, n, upd in updates:
        if cur > pos:
            pieces.append(flat[pos:cur])
        pieces.append(flat[cur : cur + n] + upd)
        pos = cur + n
    if pos < flat.shape[0]:
        pieces.append(flat[pos:])
    out = torch.cat(pieces, dim=0)
    return out.reshape(result.shape) if squeeze else out
