"""Unfused LoRA-linear oracle with an explicit dropout keep-mask (test infrastructure).

Restates /root/reference/lorafusion/ops/lora_torch_ref.py:6-48 (single adapter)
and :51-120 (segmented multi adapter).  The reference draws its dropout mask
inside ``torch.nn.functional.dropout``; here the keep-mask is an argument and
dropout is ``where(mask, x / (1 - p), 0)`` as in
lorafusion/ops/triton_ops/fused_dropout_matmul.py:82-86.

Gradient closed forms follow the docstring of
lorafusion/ops/lora_v1.py:241-247 and the torch refs in
lorafusion/ops/triton_ops/fused_lora_dys_dyb.py:59-67 and
fused_lora_dyw_dsa.py:56-65.

Two precisions:

* ``*_fp32`` -- inputs (bf16 tensors) are widened and every product is
  accumulated in ``acc_dtype`` (fp32 by default, fp64 on request) with no
  intermediate rounding.  This is the pass/fail comparand.
* ``*_bf16_opbyop`` -- the reference's literal arithmetic: every op rounds to
  the tensor dtype.  Used for the CPU timing baseline and reported alongside.
"""

from __future__ import annotations

import torch


def keep_scale(p: float) -> float:
    """1/(1-p), the scale applied to kept elements."""
    return 1.0 / (1.0 - p) if p > 0.0 else 1.0


def dropout_explicit(x: torch.Tensor, mask: torch.Tensor | None, p: float) -> torch.Tensor:
    """``where(mask, x/(1-p), 0)``; identity when ``p == 0`` or ``mask is None``."""
    if p <= 0.0 or mask is None:
        return x
    return torch.where(mask, x * keep_scale(p), torch.zeros((), dtype=x.dtype))


# --------------------------------------------------------------------------- single


def linear_lora_fwd_fp32(x, w, a, b, scale, mask=None, p=0.0, bias=None, acc_dtype=torch.float32):
    """Y = X Wt (+bias) + scale * (drop(X) At) Bt, accumulated in ``acc_dtype``.

    lora_torch_ref.py:32-48.  x [M,K], w [N,K], a [r,K], b [N,r], mask bool [M,K].
    Returns (y [M,N], s [M,r]) in ``acc_dtype``; ``s`` is the unscaled drop(X) At.
    """
    xf, wf, af, bf = (t.to(acc_dtype) for t in (x, w, a, b))
    y = xf @ wf.T
    if bias is not None:
        y = y + bias.to(acc_dtype)
    s = dropout_explicit(xf, mask, p) @ af.T
    y = y + (s @ bf.T) * scale
    return y, s


def linear_lora_bwd_fp32(dy, x, w, a, b, scale, mask=None, p=0.0, acc_dtype=torch.float32):
    """Closed-form gradients (lora_v1.py:241-247).

    db = scale * dYt S, ds = scale * dY B, da = dSt X~, dx = dY W + mask * (dS A)/(1-p).
    Returns (dx [M,K], da [r,K], db [N,r], ds [M,r]) in ``acc_dtype``.  With ``w=None`` the
    M x N x K product is skipped and dx is None (full-size layer shapes, where dx is checked
    on a sample of rows by a second call on those rows: dx is row-wise independent).
    """
    dyf, xf, af, bf = (t.to(acc_dtype) for t in (dy, x, a, b))
    xt = dropout_explicit(xf, mask, p)
    s = xt @ af.T
    db = (dyf.T @ s) * scale
    ds = (dyf @ bf) * scale
    da = ds.T @ xt
    dx = None if w is None else dyf @ w.to(acc_dtype) + dropout_explicit(ds @ af, mask, p)
    return dx, da, db, ds


def linear_lora_bf16_opbyop(x, w, a, b, scale, mask=None, p=0.0, bias=None):
    """The reference's literal op-by-op arithmetic in the tensors' own dtype.

    lora_torch_ref.py:32-48 with F.dropout replaced by the explicit mask.  Stays in the
    autograd graph so ``.backward()`` gives the reference's unfused backward.
    """
    result = x @ w.T
    if bias is not None:
        result = result + bias
    x_for_lora = dropout_explicit(x, mask, p)
    lora_output = (x_for_lora @ a.T @ b.T) * scale
    return result + lora_output


# --------------------------------------------------------------------------- multi


def _segments(seq_len_list, padded_seq_len_list):
    cur = 0
    for seq_len, padded in zip(seq_len_list, padded_seq_len_list, strict=True):
        yield cur, seq_len
        cur += padded


def linear_multi_lora_fwd_fp32(
    padded_x, w, a_list, b_list, seq_len_list, padded_seq_len_list, scale_list, p_list,
    mask=None, bias=None, acc_dtype=torch.float32,
):
    """Segmented forward (lora_torch_ref.py:82-120).

    The base GEMM covers every row; adapter i's LoRA term is added to rows
    ``[cur, cur+seq_len_i)`` only and the cursor advances by the *padded* length, so
    padding rows carry the base GEMM (+bias) alone.
    Returns (y [Mp,N], s_list) with s_i [seq_len_i, r_i] unscaled.
    """
    xf, wf = padded_x.to(acc_dtype), w.to(acc_dtype)
    y = xf @ wf.T
    if bias is not None:
        y = y + bias.to(acc_dtype)
    s_list = []
    for (cur, n), a, b, scale, p in zip(
        _segments(seq_len_list, padded_seq_len_list), a_list, b_list, scale_list, p_list, strict=True
    ):
        seg = xf[cur : cur + n]
        seg_mask = mask[cur : cur + n] if mask is not None else None
        s = dropout_explicit(seg, seg_mask, p) @ a.to(acc_dtype).T
        y[cur : cur + n] += (s @ b.to(acc_dtype).T) * scale
        s_list.append(s)
    return y, s_list


def linear_multi_lora_bwd_fp32(
    dy, padded_x, w, a_list, b_list, seq_len_list, padded_seq_len_list, scale_list, p_list,
    mask=None, acc_dtype=torch.float32,
):
    """Segmented closed-form gradients: the single-adapter formulas on each segment.

    Returns (dx [Mp,K], da_list, db_list, ds_list).  Padding rows of dx get dY W only.
    """
    dyf, xf, wf = dy.to(acc_dtype), padded_x.to(acc_dtype), w.to(acc_dtype)
    dx = dyf @ wf
    da_list, db_list, ds_list = [], [], []
    for (cur, n), a, b, scale, p in zip(
        _segments(seq_len_list, padded_seq_len_list), a_list, b_list, scale_list, p_list, strict=True
    ):
        af, bf = a.to(acc_dtype), b.to(acc_dtype)
        seg_mask = mask[cur : cur + n] if mask is not None else None
        xt = dropout_explicit(xf[cur : cur + n], seg_mask, p)
        dyseg = dyf[cur : cur + n]
        s = xt @ af.T
        ds = (dyseg @ bf) * scale
        db_list.append((dyseg.T @ s) * scale)
        da_list.append(ds.T @ xt)
        ds_list.append(ds)
        dx[cur : cur + n] += dropout_explicit(ds @ af, seg_mask, p)
    return dx, da_list, db_list, ds_list


def linear_multi_lora_bf16_opbyop(
    padded_x, w, a_list, b_list, seq_len_list, padded_seq_len_list, scale_list, p_list,
    mask=None, bias=None,
):
    """Literal lora_torch_ref.py:82-120 arithmetic in the tensors' dtype (autograd-capable)."""
    result = padded_x @ w.T
    if bias is not None:
        result = result + bias
    pieces = []
    for (cur, n), a, b, scale, p in zip(
        _segments(seq_len_list, padded_seq_len_list), a_list, b_list, scale_list, p_list, strict=True
    ):
        seg = padded_x[cur : cur + n]
        seg_mask = mask[cur : cur + n] if mask is not None else None
        pieces.append((cur, n, (dropout_explicit(seg, seg_mask, p) @ a.T @ b.T) * scale))
    # out-of-place accumulation keeps autograd happy; same values as the in-place "+=".
    add = torch.zeros_like(result)
    for cur, n, lo in pieces:
        add = add.index_add(0, torch.arange(cur, cur + n), lo)
    return result + add


# --------------------------------------------------------------------------- tolerance


def bf16_quantum(expected: torch.Tensor) -> float:
    """Empirical bf16 rounding quantum of a tensor's scale.

    lorafusion/utils/testing.py:160-161: ``2.5 * max|((e + 0.3) - 0.3) - e|`` evaluated
    in bf16.
    """
    e = expected.to(torch.bfloat16)
    return 2.5 * float((((e + 0.3) - 0.3) - e).abs().max())


def check_close(actual: torch.Tensor, expected: torch.Tensor, rtol: float = 1e-2, atol: float | None = None):
    """|a - e| <= atol + rtol*|e| elementwise; atol defaults to 1e-2 * rms(e).

    Returns (ok, max_abs_err / max|e|, worst elementwise excess).
    """
    a, e = actual.detach().double(), expected.detach().double()
    if atol is None:
        atol = 1e-2 * float(e.pow(2).mean().sqrt())
    err = (a - e).abs()
    bound = atol + rtol * e.abs()
    denom = float(e.abs().max())
    rel = float(err.max()) / denom if denom > 0 else float(err.max())
    return bool((err <= bound).all()), rel, float((err - bound).max())
