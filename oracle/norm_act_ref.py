"""RMSNorm and SiLU-multiply oracle (test infrastructure; the product never imports this).

The reference does not hold these algorithms: ``apply_liger_kernel`` (lorafusion/utils/module.py:41-71) swaps the
RMSNorm and the SwiGLU MLP of Llama / Qwen2 / Mixtral models for the kernels of the third-party package
``liger-kernel`` (pinned ``liger-kernel==0.5.6`` in the reference's requirements.txt:20; absent from the reference
tree and not installed here).  This file restates that package's published algorithm:

* RMSNorm, "llama" casting mode, offset 0 (``liger_kernel/ops/rms_norm.py``): per row, in fp32,
  ``rstd = 1/sqrt(mean(x^2) + eps)``; ``y = round16(round16(x * rstd) * w)`` (only the inverse RMS is taken in fp32, the
  normalised row is rounded to the 16-bit dtype before the weight multiplies it -- what HF's ``LlamaRMSNorm`` does
  too).  Backward: with ``m = dy * w``, ``dx = rstd * (m - x * rstd^2 * mean(m * x))``,
  ``dw = sum_rows dy * round16(x * rstd)`` accumulated in fp32.
* SiLU-multiply (``liger_kernel/ops/swiglu.py``): ``c = round16(round16(silu(a)) * b)`` with ``silu`` in fp32;
  backward ``db = dc * silu(a)``, ``da = dc * (silu(a) * (1 - sig(a)) + sig(a)) * b`` in fp32.

Two forms of each: ``*_exact`` accumulates in fp64 with no intermediate rounding (the pass/fail comparand for
gradients, whose rounding points the package does not fix), and the forward functions that round where the
algorithm rounds (the comparand for outputs).  Pinned in tests/test_oracle_norm_act.py against HF transformers'
``LlamaRMSNorm`` and ``torch.nn.functional.silu`` (library routines of the same definition) and against
``torch.autograd`` of an independently written fp64 forward.
"""

from __future__ import annotations

import torch


def rms_norm_fwd(x: torch.Tensor, w: torch.Tensor, eps: float):
    """x [M,H] and w [H] of one 16-bit dtype -> (y [M,H] of that dtype, rstd [M] fp32), rounding where the
    algorithm rounds."""
    xf = x.float()
    rstd = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    xn = (xf * rstd).to(x.dtype)
    return (xn * w).to(x.dtype), rstd.reshape(-1)


def rms_norm_fwd_exact(x: torch.Tensor, w: torch.Tensor, eps: float):
    """The same in fp64 without intermediate rounding: (y fp64, rstd fp64)."""
    xd, wd = x.double(), w.double()
    rstd = 1.0 / torch.sqrt(xd.pow(2).mean(-1, keepdim=True) + eps)
    return xd * rstd * wd, rstd.reshape(-1)


def rms_norm_bwd_exact(dy: torch.Tensor, x: torch.Tensor, w: torch.Tensor, eps: float):
    """(dx [M,H], dw [H]) in fp64.  ``dw`` sums dy times the *16-bit-rounded* normalised row, as the algorithm
    defines it; pass ``round_xn=False`` to ``rms_norm_dw_exact`` for the unrounded sum."""
    dyd, xd, wd = dy.double(), x.double(), w.double()
    rstd = 1.0 / torch.sqrt(xd.pow(2).mean(-1, keepdim=True) + eps)
    m = dyd * wd
    dx = rstd * (m - xd * rstd.pow(2) * (m * xd).mean(-1, keepdim=True))
    return dx, rms_norm_dw_exact(dy, x, eps, round_xn=True)


def rms_norm_dw_exact(dy: torch.Tensor, x: torch.Tensor, eps: float, *, round_xn: bool):
    xd = x.double()
    rstd = 1.0 / torch.sqrt(xd.pow(2).mean(-1, keepdim=True) + eps)
    xn = xd * rstd
    if round_xn:
        xn = (x.float() * rstd.float()).to(x.dtype).double()
    return (dy.double() * xn).sum(0)


def silu_mul_fwd(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """c = round16(round16(silu(a)) * b); a, b of one 16-bit dtype."""
    af = a.float()
    s = (af * torch.sigmoid(af)).to(b.dtype)
    return (s * b).to(b.dtype)


def silu_mul_fwd_exact(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    ad = a.double()
    return ad / (1.0 + torch.exp(-ad)) * b.double()


def silu_mul_bwd_exact(dc: torch.Tensor, a: torch.Tensor, b: torch.Tensor):
    """(da, db) in fp64."""
    ad, bd, dcd = a.double(), b.double(), dc.double()
    sig = 1.0 / (1.0 + torch.exp(-ad))
    silu = ad * sig
    return dcd * (silu * (1.0 - sig) + sig) * bd, dcd * silu


def ulp16_err(actual: torch.Tensor, expected: torch.Tensor) -> float:
    """Largest |actual - expected| in units of the 16-bit dtype's spacing at ``expected`` (``actual`` is a 16-bit
    tensor, ``expected`` any float tensor)."""
    bits = 8 if actual.dtype == torch.bfloat16 else 11
    e = expected.double()
    mag = e.abs().clamp_min(torch.finfo(actual.dtype).tiny)
    spacing = torch.exp2(torch.floor(torch.log2(mag)) - (bits - 1))
    return float(((actual.detach().double() - e).abs() / spacing).max())
