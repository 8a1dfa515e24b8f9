"""RMSNorm and SiLU-multiply on the HIP kernels: the steps either side of a decoder layer's LoRA linears.

The reference swaps HF's RMSNorm and SwiGLU MLP for the liger-kernel package's
(``apply_liger_kernel``, lorafusion/utils/module.py:41-71); the names below follow that package's
(``LigerRMSNormFunction`` / ``LigerRMSNorm``, ``LigerSiLUMulFunction`` / ``LigerSwiGLUMLP``), the arithmetic its
"llama" casting mode.  ``silu_mul_merged`` is an addition for merged gate/up projections: it reads the two halves
of one ``[M, 2I]`` tensor in place and its backward writes the gradient of that tensor directly (no split / cat
copies around the activation).
"""

from __future__ import annotations

import torch
from torch import nn

from lorafusion_amd import _lib as L


def _rows(t: torch.Tensor) -> torch.Tensor:
    t2 = t.reshape(-1, t.shape[-1])
    return t2 if t2.is_contiguous() else t2.contiguous()


class RMSNormFunction(torch.autograd.Function):
    """y = round16(round16(x * rstd) * w), rstd = 1/sqrt(mean(x^2) + eps) in fp32 (HF LlamaRMSNorm's arithmetic)."""

    @staticmethod
    def forward(ctx, x: torch.Tensor, w: torch.Tensor, eps: float):
        L.require_gpu(x, "x")
        L.require_gpu(w, "weight")
        if w.dtype != x.dtype:
            raise ValueError(f"RMSNorm weight dtype {w.dtype} differs from the input's {x.dtype}.")
        H = x.shape[-1]
        if w.shape != (H,):
            raise ValueError(f"RMSNorm weight shape {tuple(w.shape)} does not match the hidden size {H}.")
        x2 = _rows(x)
        wc = w.contiguous()
        M = x2.shape[0]
        y = torch.empty_like(x2)
        rstd = torch.empty(M, dtype=torch.float32, device=x.device)
        if M > 0:
            L.check(L.lib().lf_rmsnorm_fwd(x2.data_ptr(), wc.data_ptr(), y.data_ptr(), rstd.data_ptr(), M, H, float(eps),
                                           L.dtype_id(x.dtype), L.stream_of(x)), "lf_rmsnorm_fwd")
        ctx.save_for_backward(x2, wc, rstd)
        ctx.x_shape = x.shape
        return y.reshape(x.shape)

    @staticmethod
    def backward(ctx, dy: torch.Tensor):
        x2, w, rstd = ctx.saved_tensors
        M, H = x2.shape
        dy2 = _rows(dy)
        need_dw = ctx.needs_input_grad[1]
        dx = torch.empty_like(x2)
        dw = torch.empty_like(w) if need_dw else None
        if M > 0:
            lib = L.lib()
            nbytes = lib.lf_rmsnorm_bwd_workspace(M, H) if need_dw else 0
            ws = L.workspace(nbytes, x2.device)
            L.check(lib.lf_rmsnorm_bwd(dy2.data_ptr(), x2.data_ptr(), w.data_ptr(), rstd.data_ptr(), dx.data_ptr(),
                                       L.ptr(dw), M, H, L.dtype_id(x2.dtype), L.ptr(ws), nbytes, L.stream_of(x2)),
                    "lf_rmsnorm_bwd")
        elif need_dw:
            dw.zero_()
        return dx.reshape(ctx.x_shape), dw, None


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    return RMSNormFunction.apply(x, weight, eps)


class RMSNorm(nn.Module):
    """Drop-in for HF ``LlamaRMSNorm`` / liger's ``LigerRMSNorm`` (offset 0, "llama" casting)."""

    def __init__(self, hidden_size: int, eps: float = 1e-6, device=None, dtype=None) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size, device=device, dtype=dtype))
        self.variance_epsilon = eps

    def forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
        return rms_norm(hidden_states, self.weight, self.variance_epsilon)

    def extra_repr(self) -> str:
        return f"{tuple(self.weight.shape)}, eps={self.variance_epsilon}"


def _view2d(t: torch.Tensor, what: str):
    """(tensor, row stride) of ``t`` seen as [M, I] rows with unit column stride; copies only if it must."""
    t2 = t.reshape(-1, t.shape[-1]) if t.dim() != 2 else t
    if t2.stride(1) != 1 or t2.stride(0) % 8 != 0 or t2.data_ptr() % 16 != 0 or (t2.shape[0] > 1 and t2.stride(0) < t2.shape[1]):
        t2 = t2.contiguous()
    return t2, (t2.stride(0) if t2.shape[0] > 1 else max(t2.stride(0), t2.shape[1]))


def _silu_fwd(a2, lda, b2, ldb, out):
    M, I = a2.shape
    if M > 0:
        L.check(L.lib().lf_silu_mul_fwd(a2.data_ptr(), b2.data_ptr(), out.data_ptr(), M, I, lda, ldb, I,
                                        L.dtype_id(a2.dtype), L.stream_of(a2)), "lf_silu_mul_fwd")


def _silu_bwd(dc2, lddc, a2, lda, b2, ldb, da, ldda, db, lddb):
    M, I = a2.shape
    if M > 0:
        L.check(L.lib().lf_silu_mul_bwd(dc2.data_ptr(), a2.data_ptr(), b2.data_ptr(), da.data_ptr(), db.data_ptr(), M, I,
                                        lddc, lda, ldb, ldda, lddb, L.dtype_id(a2.dtype), L.stream_of(a2)),
                "lf_silu_mul_bwd")


class SiLUMulFunction(torch.autograd.Function):
    """c = silu(a) * b with a, b separate tensors (or views: row strides are honoured)."""

    @staticmethod
    def forward(ctx, a: torch.Tensor, b: torch.Tensor):
        L.require_gpu(a, "a")
        if a.shape != b.shape or a.dtype != b.dtype:
            raise ValueError(f"silu_mul operands differ: {tuple(a.shape)} {a.dtype} vs {tuple(b.shape)} {b.dtype}.")
        if a.shape[-1] % 8 != 0:
            raise ValueError(f"the last dimension must be a multiple of 8, got {a.shape[-1]}.")
        a2, lda = _view2d(a, "a")
        b2, ldb = _view2d(b, "b")
        c = torch.empty(a2.shape, dtype=a.dtype, device=a.device)
        _silu_fwd(a2, lda, b2, ldb, c)
        ctx.save_for_backward(a2, b2)
        ctx.lds = (lda, ldb)
        ctx.shape = a.shape
        return c.reshape(a.shape)

    @staticmethod
    def backward(ctx, dc: torch.Tensor):
        a2, b2 = ctx.saved_tensors
        lda, ldb = ctx.lds
        M, I = a2.shape
        dc2, lddc = _view2d(dc, "dc")
        da = torch.empty((M, I), dtype=a2.dtype, device=a2.device)
        db = torch.empty((M, I), dtype=a2.dtype, device=a2.device)
        _silu_bwd(dc2, lddc, a2, lda, b2, ldb, da, I, db, I)
        return da.reshape(ctx.shape), db.reshape(ctx.shape)


class SiLUMulMergedFunction(torch.autograd.Function):
    """c = silu(gu[..., :I]) * gu[..., I:] for a merged gate/up tensor ``gu`` [.., 2I]; the backward writes d(gu)."""

    @staticmethod
    def forward(ctx, gu: torch.Tensor):
        L.require_gpu(gu, "gate_up")
        if gu.shape[-1] % 16 != 0:
            raise ValueError(f"the merged width must be a multiple of 16, got {gu.shape[-1]}.")
        g2 = _rows(gu)
        M, I2 = g2.shape
        I = I2 // 2
        c = torch.empty((M, I), dtype=gu.dtype, device=gu.device)
        _silu_fwd(g2[:, :I], I2, g2[:, I:], I2, c)
        ctx.save_for_backward(g2)
        ctx.shape = gu.shape
        return c.reshape(*gu.shape[:-1], I)

    @staticmethod
    def backward(ctx, dc: torch.Tensor):
        (g2,) = ctx.saved_tensors
        M, I2 = g2.shape
        I = I2 // 2
        dc2, lddc = _view2d(dc, "dc")
        dg = torch.empty_like(g2)
        _silu_bwd(dc2, lddc, g2[:, :I], I2, g2[:, I:], I2, dg[:, :I], I2, dg[:, I:], I2)
        return dg.reshape(ctx.shape)


def silu_mul(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    return SiLUMulFunction.apply(a, b)


def silu_mul_merged(gate_up: torch.Tensor) -> torch.Tensor:
    return SiLUMulMergedFunction.apply(gate_up)


def swiglu_mlp_forward(mlp: nn.Module, x: torch.Tensor) -> torch.Tensor:
    """``down_proj(silu(gate_proj(x)) * up_proj(x))`` of an HF Llama / Qwen2 MLP (what liger's ``LigerSwiGLUMLP``
    computes), through whatever the three projections are.  A ``down_proj`` that is a LoRA linear on the fused ops
    (a PEFT layer under ``apply_lora``, or ``LoRALinear``) takes the activation as the prologue of its first kernel."""
    from lorafusion_amd.patch import patch_lora

    gate, up = mlp.gate_proj(x), mlp.up_proj(x)
    down = mlp.down_proj
    fused = getattr(down, "use_fused", None)
    if fused is None:
        fused = getattr(type(down), "_lorafusion_use_fused", None)
    if fused and patch_lora._is_lora_linear(down) and gate.shape[-1] % 128 == 0:
        return patch_lora.swiglu_lora_forward(down, gate, up, use_fused=True)
    return down(silu_mul(gate, up))
