"""Pins of the RMSNorm / SiLU-multiply oracle (CPU).

The algorithm is liger-kernel's (absent here); what pins the restatement: HF transformers' ``LlamaRMSNorm`` and
``torch.nn.functional.silu`` (library routines of the same definition, bit for bit on 16-bit inputs),
``torch.autograd`` through independently written fp64 forwards, closed forms (constant rows), and the invariants
the mathematics fixes (dx orthogonal to x when eps = 0; finite differences).  Also the host-side argument checks of
the C entry points, which return before anything is launched.
"""

import ctypes
import math

import pytest
import torch

from oracle import norm_act_ref as R


def _rand(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(7, 64), (33, 1000), (4, 4096)])
def test_rms_norm_forward_is_hf_llama_rmsnorm(dtype, shape):
    from transformers.models.llama.modeling_llama import LlamaRMSNorm

    x = _rand(shape, dtype, 1, scale=3.0)
    w = (1.0 + 0.1 * _rand((shape[1],), torch.float32, 2)).to(dtype)
    hf = LlamaRMSNorm(shape[1], eps=1e-5).to(dtype)
    with torch.no_grad():
        hf.weight.copy_(w)
        exp = hf(x)
    y, rstd = R.rms_norm_fwd(x, w, 1e-5)
    assert y.dtype == dtype and torch.equal(y, exp)
    ye, rstde = R.rms_norm_fwd_exact(x, w, 1e-5)
    assert torch.allclose(rstd.double(), rstde, rtol=1e-6, atol=0)
    assert R.ulp16_err(y, ye) <= 1.51  # two roundings of an exact value


def test_rms_norm_closed_forms():
    # a constant row c: y = w * c / sqrt(c^2 + eps); a row of +-c alternates sign
    H, c, eps = 256, 0.75, 1e-3
    x = torch.full((2, H), c, dtype=torch.float64)
    x[1, ::2] = -c
    w = torch.linspace(0.5, 1.5, H, dtype=torch.float64)
    y, rstd = R.rms_norm_fwd_exact(x, w, eps)
    assert torch.allclose(rstd, torch.full((2,), 1 / math.sqrt(c * c + eps), dtype=torch.float64), rtol=1e-14)
    assert torch.allclose(y[0], w * c / math.sqrt(c * c + eps), rtol=1e-14)
    assert torch.allclose(y[1], y[0] * torch.sign(x[1]), rtol=1e-14)
    # eps = 0: the output does not change when the row is rescaled
    x = torch.randn(3, H, dtype=torch.float64, generator=torch.Generator().manual_seed(0))
    a, _ = R.rms_norm_fwd_exact(x, w, 0.0)
    b, _ = R.rms_norm_fwd_exact(x * 7.5, w, 0.0)
    assert torch.allclose(a, b, rtol=1e-13)


@pytest.mark.parametrize("eps", [0.0, 1e-6, 1e-2])
def test_rms_norm_backward_against_autograd(eps):
    from transformers.models.llama.modeling_llama import LlamaRMSNorm

    M, H = 9, 96
    g = torch.Generator().manual_seed(3)
    x = torch.randn(M, H, dtype=torch.float64, generator=g)
    w = 1.0 + 0.2 * torch.randn(H, dtype=torch.float64, generator=g)
    dy = torch.randn(M, H, dtype=torch.float64, generator=g)
    # an independent way to write the forward: x w sqrt(H) / sqrt(|x|^2 + H eps)
    xa, wa = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    y = xa * wa * math.sqrt(H) / torch.sqrt((xa * xa).sum(-1, keepdim=True) + H * eps)
    y.backward(dy)
    dx, _ = R.rms_norm_bwd_exact(dy, x, w, eps)
    assert torch.allclose(dx, xa.grad, rtol=1e-11, atol=1e-13)
    assert torch.allclose(R.rms_norm_dw_exact(dy, x, eps, round_xn=False), wa.grad, rtol=1e-11, atol=1e-13)
    # and through HF's module (which computes the normalisation in fp32 whatever the input: fp32 tolerance)
    hf = LlamaRMSNorm(H, eps=eps).double()
    with torch.no_grad():
        hf.weight.copy_(w)
    xb = x.clone().requires_grad_(True)
    hf(xb).backward(dy)
    assert torch.allclose(dx, xb.grad, rtol=1e-4, atol=1e-5)
    assert torch.allclose(R.rms_norm_dw_exact(dy, x, eps, round_xn=False), hf.weight.grad, rtol=1e-4, atol=1e-5)
    if eps == 0.0:
        # the output ignores the row's scale, so the gradient has no component along the row
        assert float((dx * x).sum(-1).abs().max()) < 1e-12


def test_rms_norm_dw_rounding_point():
    """dw sums dy times the 16-bit-rounded normalised row: close to, and not identical with, the unrounded sum."""
    x, dy = _rand((512, 128), torch.bfloat16, 5), _rand((512, 128), torch.bfloat16, 6)
    w = torch.ones(128, dtype=torch.bfloat16)
    _, dw = R.rms_norm_bwd_exact(dy, x, w, 1e-6)
    plain = R.rms_norm_dw_exact(dy, x, 1e-6, round_xn=False)
    assert not torch.equal(dw, plain)
    assert float((dw - plain).abs().max()) < 2.0 ** -8 * float((dy.double().abs() * 4).sum(0).max())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_silu_mul_forward_is_hf_mlp_activation(dtype):
    a, b = _rand((37, 264), dtype, 7, scale=4.0), _rand((37, 264), dtype, 8)
    exp = torch.nn.functional.silu(a) * b          # LlamaMLP.forward: act_fn(gate) * up
    got = R.silu_mul_fwd(a, b)
    assert got.dtype == dtype
    if dtype == torch.bfloat16:
        assert torch.equal(got, exp)
    else:
        # torch's half silu divides (x / (1 + exp(-x))) where the algorithm multiplies by the sigmoid: the fp32
        # values differ in the last place and a few of them round to the neighbouring half
        assert float((got != exp).float().mean()) < 5e-3 and R.ulp16_err(got, exp.double()) <= 3.0  # a neighbouring intermediate: two spacings of the result, and a rounding each
    exact = R.silu_mul_fwd_exact(a, b)
    assert torch.allclose(exact, torch.nn.functional.silu(a.double()) * b.double(), rtol=1e-14, atol=1e-300)
    assert R.ulp16_err(got, exact) <= 1.51


def test_silu_mul_backward_against_autograd_and_differences():
    g = torch.Generator().manual_seed(9)
    a = (torch.randn(11, 40, dtype=torch.float64, generator=g) * 3).requires_grad_(True)
    b = torch.randn(11, 40, dtype=torch.float64, generator=g).requires_grad_(True)
    dc = torch.randn(11, 40, dtype=torch.float64, generator=g)
    (torch.nn.functional.silu(a) * b).backward(dc)
    da, db = R.silu_mul_bwd_exact(dc, a.detach(), b.detach())
    assert torch.allclose(da, a.grad, rtol=1e-12, atol=1e-14) and torch.allclose(db, b.grad, rtol=1e-12, atol=1e-14)
    h = 1e-6
    fd = (R.silu_mul_fwd_exact(a.detach() + h, b.detach()) - R.silu_mul_fwd_exact(a.detach() - h, b.detach())) / (2 * h)
    assert torch.allclose(da, dc * fd, rtol=1e-6, atol=1e-8)
    # known points: silu'(0) = 1/2, silu(0) = 0
    z = torch.zeros(1, 8, dtype=torch.float64)
    da0, db0 = R.silu_mul_bwd_exact(torch.ones_like(z), z, torch.full_like(z, 3.0))
    assert torch.equal(da0, torch.full_like(z, 1.5)) and torch.equal(db0, z)


def test_norm_act_argument_checks_without_gpu():
    from lorafusion_amd import _lib

    lib = _lib.lib()
    p = ctypes.c_void_p(4096)
    assert lib.lf_rmsnorm_fwd(None, p, p, p, 4, 64, 1e-6, 0, None) == _lib.LF_EINVAL
    assert lib.lf_rmsnorm_fwd(p, p, p, p, 4, 60, 1e-6, 0, None) == _lib.LF_ESHAPE          # H % 8
    assert lib.lf_rmsnorm_fwd(ctypes.c_void_p(4100), p, p, p, 4, 64, 1e-6, 0, None) == _lib.LF_ESHAPE   # alignment
    assert lib.lf_rmsnorm_fwd(p, p, p, p, 4, 8200, 1e-6, 0, None) == _lib.LF_ELIMIT
    assert lib.lf_rmsnorm_fwd(p, p, p, p, 4, 64, 1e-6, 5, None) == _lib.LF_EINVAL          # dtype
    assert lib.lf_rmsnorm_bwd(p, p, p, p, p, p, 4, 64, 0, None, 0, None) == _lib.LF_EWORKSPACE
    assert lib.lf_rmsnorm_bwd(p, p, p, p, p, p, 4, 8200, 0, None, 0, None) == _lib.LF_ELIMIT
    # one fp32 row per workgroup of the persistent kernel, never more workgroups than four-row groups
    assert lib.lf_rmsnorm_bwd_workspace(8, 4096) == 2 * 4096 * 4
    big = lib.lf_rmsnorm_bwd_workspace(1 << 20, 4096)
    assert 0 < big <= 4 * 4096 * 4 * 1024 and big % (4096 * 4) == 0
    assert lib.lf_rmsnorm_bwd_workspace(8, 8200) == 0
    assert lib.lf_silu_mul_fwd(p, p, None, 4, 64, 64, 64, 64, 0, None) == _lib.LF_EINVAL
    assert lib.lf_silu_mul_fwd(p, p, p, 4, 64, 56, 64, 64, 0, None) == _lib.LF_ESHAPE       # ld < I
    assert lib.lf_silu_mul_fwd(p, p, p, 4, 60, 64, 64, 64, 0, None) == _lib.LF_ESHAPE       # I % 8
    assert lib.lf_silu_mul_bwd(p, p, p, p, p, 4, 64, 64, 64, 64, 68, 64, 0, None) == _lib.LF_ESHAPE  # ld % 8
    assert lib.lf_silu_mul_bwd(p, p, p, p, p, 4, 64, 64, 64, 64, 64, 64, 9, None) == _lib.LF_EINVAL


def test_ops_refuse_cpu_tensors_and_bad_levels():
    from lorafusion_amd.ops import norm_act
    from lorafusion_amd.utils.module import LigerKernelLevel, apply_liger_kernel, restore_liger_kernel

    with pytest.raises(ValueError, match="GPU"):
        norm_act.rms_norm(torch.zeros(2, 64, dtype=torch.bfloat16), torch.ones(64, dtype=torch.bfloat16))
    with pytest.raises(ValueError, match="GPU"):
        norm_act.silu_mul(torch.zeros(2, 64, dtype=torch.bfloat16), torch.zeros(2, 64, dtype=torch.bfloat16))
    with pytest.raises(ValueError, match="Invalid Liger kernel level"):
        apply_liger_kernel("everything")
    from transformers.models.llama import modeling_llama as ml

    before = (ml.LlamaRMSNorm.forward, ml.LlamaMLP.forward)
    apply_liger_kernel(LigerKernelLevel.DISABLE)
    assert (ml.LlamaRMSNorm.forward, ml.LlamaMLP.forward) == before
    apply_liger_kernel(LigerKernelLevel.NO_RMS_NORM)
    assert ml.LlamaRMSNorm.forward is before[0] and ml.LlamaMLP.forward is not before[1]
    apply_liger_kernel("all")
    assert ml.LlamaRMSNorm.forward is not before[0]
    # fp32 / CPU activations keep HF's arithmetic under the patch
    n = ml.LlamaRMSNorm(64)
    x = torch.randn(3, 64)
    patched = n(x)

    # a subclass inherits the patched forward; its fallback is found along the MRO
    class MyNorm(ml.LlamaRMSNorm):
        pass

    class MyMLP(ml.LlamaMLP):
        pass

    sub = MyNorm(64)
    sub_patched = sub(x)
    cfg = ml.LlamaConfig(hidden_size=64, intermediate_size=96, hidden_act="silu")
    mlp = MyMLP(cfg)
    mlp_patched = mlp(x)
    restore_liger_kernel()
    assert (ml.LlamaRMSNorm.forward, ml.LlamaMLP.forward) == before
    assert torch.equal(patched, n(x))
    assert torch.equal(sub_patched, sub(x)) and torch.equal(mlp_patched, mlp(x))
