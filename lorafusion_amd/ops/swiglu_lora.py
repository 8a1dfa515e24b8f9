"""The down projection of a SwiGLU MLP with the activation as the prologue of its LoRA linear.

``down_proj(silu(gate) * up)`` is what liger-kernel's ``LigerSwiGLUMLP`` computes (the reference switches it in with
``apply_liger_kernel``, lorafusion/utils/module.py:41-71) and the reference's patched ``down_proj`` then runs
``fused_linear_lora`` / ``fused_linear_multi_lora`` on the product (lorafusion/patch/patch_lora.py:46-160).  Here the
first kernel of that linear -- the rank-r pass ``S = drop(X) A^T`` -- computes ``X = silu(gate) * up`` itself while it
streams the gate/up tensor, writes ``X`` once (the base GEMM and the backward read it), and the separate activation
pass and the pass's own read of ``X`` disappear.  Results are bit-identical to ``silu_mul_merged`` followed by the
fused LoRA linear with the same mask or seed.
"""

from __future__ import annotations

import ctypes
import random

import torch

from lorafusion_amd import _lib as L
from lorafusion_amd.ops import hip_ops
from lorafusion_amd.ops.hip_ops import MultiRouting
from lorafusion_amd.ops.norm_act import _silu_bwd


def _swiglu_lora_forward(gate, up, ld, w, a_list, b_list, routing_c, R, mask, draw_seed, bias):
    """One C call.  gate, up [M, K] views with unit column stride, rows ``ld`` elements apart.  Returns (x, y, s, mask)."""
    M, K = gate.shape
    N = w.shape[0]
    x = torch.empty((M, K), dtype=gate.dtype, device=gate.device)
    y = torch.empty((M, N), dtype=gate.dtype, device=gate.device)
    s = torch.empty((M, R), dtype=gate.dtype, device=gate.device)
    mask_out = None
    if draw_seed is not None:
        mask_out = torch.empty((M, K // 8), dtype=torch.uint8, device=gate.device)   # drawn masks are kept bit-packed
    ws, nbytes = hip_ops._ws(L.LF_OP_FWD, M, N, K, R, routing_c, gate.device)
    rc = L.lib().lf_swiglu_lora_fwd(
        gate.data_ptr(), up.data_ptr(), ld, x.data_ptr(), L.ptr(w), L.ptr(bias), L.ptr(mask), L.ptr(mask_out),
        ctypes.c_uint64(int(draw_seed or 0) & 0xFFFFFFFFFFFFFFFF), L.ptr_array(a_list), L.ptr_array(b_list), y.data_ptr(),
        s.data_ptr(), L.ptr(ws), nbytes, M, N, K, R, routing_c,
        hip_ops._dt(gate, mask_out if mask_out is not None else mask, K), L.stream_of(gate))
    L.check(rc, "lf_swiglu_lora_fwd")
    return x, y, s, (mask_out if mask_out is not None else mask)


def _rows2d(t: torch.Tensor) -> torch.Tensor:
    t2 = t.reshape(-1, t.shape[-1])
    ok = t2.stride(1) == 1 and t2.stride(0) % 8 == 0 and t2.stride(0) >= t2.shape[1] and t2.data_ptr() % 16 == 0
    return t2 if ok else t2.contiguous()


class FusedSwiGLULinearLoRA(torch.autograd.Function):
    """``y = X W^T + scale_i (drop(X) A_i^T) B_i^T + bias`` with ``X = silu(gate) * up`` taken from a merged
    ``[.., 2K]`` gate/up tensor or from two ``[.., K]`` tensors.  ``routing`` is a ``MultiRouting`` (packed
    multi-adapter batch) or ``None`` (one adapter: ``alpha`` and ``dropout_p`` apply to all rows)."""

    @staticmethod
    def forward(ctx, gate, up, linear_w, linear_bias, dropout_mask, seed, routing, alpha, dropout_p, n_adapters, *ab):
        # up is None: `gate` is the merged [.., 2K] tensor (gate half first)
        merged = up is None
        if merged:
            if gate.shape[-1] % 256 != 0:
                raise ValueError(f"the merged gate/up width must be a multiple of 256, got {gate.shape[-1]}.")
            lead = gate.shape[:-1]
            g2 = gate.reshape(-1, gate.shape[-1])
            g2 = g2 if g2.is_contiguous() else g2.contiguous()
            K = g2.shape[1] // 2
            gv, uv, ld = g2[:, :K], g2[:, K:], 2 * K
            saved_in = (g2,)
        else:
            if gate.shape != up.shape or gate.dtype != up.dtype:
                raise ValueError(f"gate and up differ: {tuple(gate.shape)} {gate.dtype} vs {tuple(up.shape)} {up.dtype}.")
            lead = gate.shape[:-1]
            gv, uv = _rows2d(gate), _rows2d(up)
            if gv.stride(0) != uv.stride(0):
                gv, uv = gv.contiguous(), uv.contiguous()
            K, ld = gv.shape[1], gv.stride(0) if gv.shape[0] > 1 else gv.shape[1]
            saved_in = (gv, uv)
        linear_w = linear_w.contiguous()
        a_list = [t.contiguous() for t in ab[:n_adapters]]
        b_list = [t.contiguous() for t in ab[n_adapters:]]
        M = gv.shape[0]
        N = linear_w.shape[0]
        L.require_gpu(gv, "gate")
        L.dtype_id(gv.dtype)
        hip_ops._check_dims(M, N, K)
        if tuple(linear_w.shape) != (N, K) or linear_w.dtype != gv.dtype:
            raise ValueError(f"linear_w must have shape [N, {K}] and dtype {gv.dtype}.")
        bias = linear_bias.contiguous() if linear_bias is not None else None
        if bias is not None and (tuple(bias.shape) != (N,) or bias.dtype != gv.dtype):
            raise ValueError(f"linear_bias must have shape [{N}] and dtype {gv.dtype}.")
        if routing is not None:
            if M != routing.M:
                raise ValueError(f"the activations have {M} rows but the batch info covers {routing.M}.")
            hip_ops._check_adapters(a_list, b_list, routing, K, N, gv.dtype)
            dropout = routing.enable_dropout
            R, rank_list = routing.R, routing.rank_list
        else:
            r = a_list[0].shape[0]
            if n_adapters != 1 or tuple(a_list[0].shape) != (r, K) or tuple(b_list[0].shape) != (N, r):
                raise ValueError(f"one adapter with lora_a [r, {K}] and lora_b [{N}, r] is expected.")
            hip_ops._check_rank(r)
            hip_ops._check_p(dropout_p)
            dropout = dropout_p > 0
            R, rank_list = L.round_rank(r), [r]
        mask, draw = None, None
        if dropout and dropout_mask is None:
            draw = seed if seed is not None else random.randrange(int(1e6))  # noqa: S311
        elif dropout:
            mask = hip_ops._check_mask(dropout_mask.reshape(M, -1), (M, K))
            if not hip_ops.is_packed_mask(mask, K):
                mask = hip_ops.pack_mask(mask)   # read three times (rank-r forward, dA, dX): an eighth of the bytes each
        p_used = dropout_p if dropout else 0.0
        routing_c = routing.c if routing is not None else L.single_routing(rank_list[0], alpha, p_used)
        x, y, s, mask = _swiglu_lora_forward(gv, uv, ld, linear_w, a_list, b_list, routing_c, R, mask, draw, bias)
        ctx.save_for_backward(x, linear_w, mask, s, *saved_in, *a_list, *b_list)
        ctx.routing, ctx.alpha, ctx.p_used = routing, alpha, p_used
        ctx.R, ctx.rank_list, ctx.n_adapters, ctx.lead, ctx.merged = R, rank_list, n_adapters, lead, merged
        return y.reshape(*lead, N)

    @staticmethod
    def backward(ctx, dy):
        x, linear_w, mask, s, *rest = ctx.saved_tensors
        n_in = 1 if ctx.merged else 2
        inputs, ab = rest[:n_in], rest[n_in:]
        n = ctx.n_adapters
        a_list, b_list = list(ab[:n]), list(ab[n:])
        dy2 = dy.reshape(-1, dy.shape[-1]).contiguous()
        routing_c = ctx.routing.c if ctx.routing is not None else L.single_routing(ctx.rank_list[0], ctx.alpha, ctx.p_used)
        need_dg = ctx.needs_input_grad[0] or (not ctx.merged and ctx.needs_input_grad[1])
        dx, da_list, db_list = hip_ops.lora_backward(dy2, x, linear_w, a_list, b_list, s, routing_c, ctx.R, mask,
                                                     ctx.rank_list, requires_dx=need_dg)
        dg, du = None, None
        if need_dg:
            M, K = x.shape
            if ctx.merged:
                (g2,) = inputs
                dg = torch.empty_like(g2)
                _silu_bwd(dx, K, g2[:, :K], 2 * K, g2[:, K:], 2 * K, dg[:, :K], 2 * K, dg[:, K:], 2 * K)
                dg = dg.reshape(*ctx.lead, 2 * K)
            else:
                gv, uv = inputs
                dg = torch.empty((M, K), dtype=x.dtype, device=x.device)
                du = torch.empty((M, K), dtype=x.dtype, device=x.device)
                _silu_bwd(dx, K, gv, gv.stride(0) if M > 1 else K, uv, uv.stride(0) if M > 1 else K, dg, K, du, K)
                dg, du = dg.reshape(*ctx.lead, K), du.reshape(*ctx.lead, K)
        return (dg, du, None, None, None, None, None, None, None, None, *da_list, *db_list)


def fused_swiglu_linear_lora(gate_up, linear_w, lora_a, lora_b, alpha: float, seed: int | None = None,
                             dropout_p: float = 0.0, linear_bias=None, dropout_mask=None, *, up=None) -> torch.Tensor:
    """``fused_linear_lora(silu(gate) * up, ...)`` (lorafusion/ops/lora_v1.py:284-297).  ``gate_up`` is the merged
    ``[.., 2K]`` tensor, or the gate tensor ``[.., K]`` when ``up`` is given separately."""
    return FusedSwiGLULinearLoRA.apply(gate_up, up, linear_w, linear_bias, dropout_mask, seed, None, alpha, dropout_p, 1,
                                       lora_a, lora_b)


def fused_swiglu_linear_multi_lora(gate_up, linear_w, lora_a_list, lora_b_list, routing: MultiRouting, *, seed=None,
                                   linear_bias=None, dropout_mask=None, up=None) -> torch.Tensor:
    """``fused_linear_multi_lora(silu(gate) * up, ...)`` (lorafusion/ops/multi_lora.py:762-830); ``gate_up`` is the
    merged ``[.., 2K]`` tensor, or the gate tensor when ``up`` is given separately; ``routing`` is the micro-batch's
    ``MultiLoRABatchInfo.routing(...)``."""
    if len(lora_a_list) != len(lora_b_list) or not lora_a_list:
        raise ValueError("lora_a_list and lora_b_list must have the same, non-zero length")
    return FusedSwiGLULinearLoRA.apply(gate_up, up, linear_w, linear_bias, dropout_mask, seed, routing, 0.0, 0.0,
                                       len(lora_a_list), *lora_a_list, *lora_b_list)
