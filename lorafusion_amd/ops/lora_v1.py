"""Single-adapter fused LoRA linear: ``fused_linear_lora`` / ``FusedLinearLoRA``.

Same call signature and gradient contract as lorafusion/ops/lora_v1.py:173-297; the work is two
C calls (forward: ``lf_lora_fwd``, backward: ``lf_lora_bwd``) into the HIP library.

Differences from the reference, all deliberate:
 * the dropped input ``where(mask, x/(1-p), 0)`` is never stored: backward rebuilds it from
   ``x`` and the 1-byte keep-mask inside the kernels (saves an [M,K] tensor per layer);
 * 2-D ``x`` works (the reference only handles 3-D, lora_v1.py:207-232);
 * ``dropout_mask`` (keyword, optional) supplies the keep-mask explicitly; with ``None`` it is
   drawn from ``seed`` (random when ``seed`` is None, as at lora_v1.py:201-202);
 * the dropout scale is fp32 ``1/(1-p)`` in both directions (the reference rounds it to bf16
   in forward, dropout.py:58-63).
"""

from __future__ import annotations

import random

import torch

from lorafusion_amd import _lib as L
from lorafusion_amd.ops import hip_ops


def _validate(x2d, linear_w, lora_a, lora_b, linear_bias, dropout_p):
    L.require_gpu(linear_w, "linear_w")
    return _validate_shapes(x2d, tuple(linear_w.shape), linear_w.dtype, lora_a, lora_b, linear_bias, dropout_p)


def _validate_shapes(x2d, w_shape, w_dtype, lora_a, lora_b, linear_bias, dropout_p):
    """Shape / dtype checks of one LoRA linear; the base weight is given by shape and (dequantised) dtype."""
    for name, t in (("x", x2d), ("lora_a", lora_a), ("lora_b", lora_b)):
        L.require_gpu(t, name)
        if t.dtype != x2d.dtype:
            raise ValueError(f"{name} must have dtype {x2d.dtype}, but got {t.dtype}.")
    if w_dtype != x2d.dtype:
        raise ValueError(f"linear_w must have dtype {x2d.dtype}, but got {w_dtype}.")
    L.dtype_id(x2d.dtype)
    M, K = x2d.shape
    if len(w_shape) != 2 or w_shape[1] != K:
        raise ValueError(f"linear_w must have shape [N, {K}], but got {tuple(w_shape)}.")
    N = w_shape[0]
    if lora_a.ndim != 2 or lora_a.shape[1] != K:
        raise ValueError(f"lora_a must have shape [r, {K}], but got {tuple(lora_a.shape)}.")
    r = lora_a.shape[0]
    if tuple(lora_b.shape) != (N, r):
        raise ValueError(f"lora_b must have shape [{N}, {r}], but got {tuple(lora_b.shape)}.")
    if linear_bias is not None and (tuple(linear_bias.shape) != (N,) or linear_bias.dtype != x2d.dtype):
        raise ValueError(f"linear_bias must have shape [{N}] and dtype {x2d.dtype}.")
    hip_ops._check_dims(M, N, K)
    hip_ops._check_rank(r)
    hip_ops._check_p(dropout_p)
    return M, N, K, r


class FusedLinearLoRA(torch.autograd.Function):
    """``y = x W^T + alpha * (drop(x) A^T) B^T + bias`` with the LoRA term fused into the GEMMs."""

    @staticmethod
    def forward(ctx, x, linear_w, lora_a, lora_b, alpha, dropout_p, seed=None, linear_bias=None, dropout_mask=None):
        if x.ndim == 3:
            lead = x.shape[:2]
            x2d = x.reshape(lead[0] * lead[1], -1)
        elif x.ndim == 2:
            lead = None
            x2d = x
        else:
            raise ValueError(f"Expected x to have 2 or 3 dimensions, got {x.ndim}.")
        x2d = x2d.contiguous()
        linear_w, lora_a, lora_b = linear_w.contiguous(), lora_a.contiguous(), lora_b.contiguous()
        M, N, K, r = _validate(x2d, linear_w, lora_a, lora_b, linear_bias, dropout_p)

        R = L.round_rank(r)
        bias = linear_bias.contiguous() if linear_bias is not None else None
        mask = None
        if dropout_p > 0 and dropout_mask is None:
            # the reference's default path: the keep-mask is drawn while X streams through the rank-r pass
            if seed is None:
                seed = random.randrange(int(1e6))  # noqa: S311
            routing = L.single_routing(r, alpha, dropout_p)
            y, s, mask = hip_ops.lora_forward_seeded(x2d, linear_w, [lora_a], [lora_b], routing, R, seed, bias)
        else:
            if dropout_p > 0:
                mask = hip_ops._check_mask(dropout_mask.reshape(M, -1), (M, K))
                if not hip_ops.is_packed_mask(mask, K):
                    mask = hip_ops.pack_mask(mask)   # read three times (rank-r forward, dA, dX): an eighth of the bytes each
            routing = L.single_routing(r, alpha, dropout_p if mask is not None else 0.0)
            y, s = hip_ops.lora_forward(x2d, linear_w, [lora_a], [lora_b], routing, R, mask, bias)

        ctx.save_for_backward(x2d, linear_w, lora_a, lora_b, mask, s)
        ctx.alpha = alpha
        ctx.dropout_p = dropout_p if mask is not None else 0.0
        ctx.seed = seed
        ctx.lead = lead
        return y if lead is None else y.reshape(*lead, N)

    @staticmethod
    def backward(ctx, dy):
        x2d, linear_w, lora_a, lora_b, mask, s = ctx.saved_tensors
        if dy.ndim == 3:
            dy2d = dy.reshape(dy.shape[0] * dy.shape[1], -1)
        elif dy.ndim == 2:
            dy2d = dy
        else:
            raise ValueError(f"Expected dy to have 2 or 3 dimensions, got {dy.ndim}.")
        dy2d = dy2d.contiguous()
        r = lora_a.shape[0]
        routing = L.single_routing(r, ctx.alpha, ctx.dropout_p)
        dx, da_list, db_list = hip_ops.lora_backward(
            dy2d, x2d, linear_w, [lora_a], [lora_b], s, routing, L.round_rank(r), mask, [r],
            requires_dx=ctx.needs_input_grad[0],
        )
        if dx is not None and ctx.lead is not None:
            dx = dx.reshape(*ctx.lead, -1)
        da = da_list[0] if ctx.needs_input_grad[2] else None
        db = db_list[0] if ctx.needs_input_grad[3] else None
        return dx, None, da, db, None, None, None, None, None


def fused_linear_lora(
    x: torch.Tensor,
    linear_w: torch.Tensor,
    lora_a: torch.Tensor,
    lora_b: torch.Tensor,
    alpha: float,
    seed: int | None = None,
    dropout_p: float = 0.0,
    linear_bias: torch.Tensor | None = None,
    dropout_mask: torch.Tensor | None = None,
) -> torch.Tensor:
    """Fused linear + LoRA (lorafusion/ops/lora_v1.py:284-297).

    ``alpha`` is the multiplier applied to the LoRA branch (PEFT's ``scaling``).
    """
    return FusedLinearLoRA.apply(x, linear_w, lora_a, lora_b, alpha, dropout_p, seed, linear_bias, dropout_mask)
