"""RMSNorm and SiLU-multiply HIP kernels against the oracle (GPU), through the C ABI and the autograd layer.

Tolerances.  Forward outputs are two roundings of an exact value: the first is at most half a spacing of the
intermediate, i.e. at most one spacing of the result in relative terms, the second half a spacing more -- at most 1.51
spacings from the fp64 value, which is asserted.  Against the oracle that rounds where the algorithm rounds the outputs
are equal except where the kernel's fp32 ``rstd`` / sigmoid differs from the CPU's in the last place and the
intermediate rounds to the neighbouring value (under 0.2 % of the elements, asserted): one spacing of the intermediate
is at most two of the result, and each side then rounds once more -- at most 3 spacings apart.
Gradients are compared with the fp64 closed forms: |err| <= 1e-2 |e| + 1e-2 rms(e), the bar of the LoRA kernels, and
those of SiLU-multiply, single roundings of fp32 values, to 0.51 spacings (plus the fp32 error where silu' cancels).
"""

from __future__ import annotations

import ctypes

import pytest
import torch

from oracle import lora_ref
from oracle import norm_act_ref as R

pytestmark = pytest.mark.gpu

DTYPES = [torch.bfloat16, torch.float16]


def _rand(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def _close(got, exp, name, rtol=1e-2):
    ok, rel, excess = lora_ref.check_close(got.detach().float().cpu(), exp, rtol=rtol)
    assert ok, f"{name}: max|err|/max|e| = {rel:.3e}, worst excess over bound {excess:.3e}"


def _spacing(e, dtype):
    bits = 8 if dtype == torch.bfloat16 else 11
    mag = e.abs().clamp_min(torch.finfo(dtype).tiny)
    return torch.exp2(torch.floor(torch.log2(mag)) - (bits - 1))


def _lib():
    from lorafusion_amd import _lib as L

    return L


def _rms_fwd_abi(x, w, eps):
    L = _lib()
    M, H = x.shape
    y = torch.empty_like(x)
    rstd = torch.empty(M, dtype=torch.float32, device=x.device)
    L.check(L.lib().lf_rmsnorm_fwd(x.data_ptr(), w.data_ptr(), y.data_ptr(), rstd.data_ptr(), M, H, eps,
                                   L.dtype_id(x.dtype), L.stream_of(x)), "lf_rmsnorm_fwd")
    return y, rstd


def _rms_bwd_abi(dy, x, w, rstd, with_dw=True, dx=None):
    L = _lib()
    M, H = x.shape
    dx = torch.empty_like(x) if dx is None else dx
    dw = torch.empty_like(w) if with_dw else None
    n = L.lib().lf_rmsnorm_bwd_workspace(M, H) if with_dw else 0
    ws = torch.empty(max(n, 16), dtype=torch.uint8, device=x.device)
    L.check(L.lib().lf_rmsnorm_bwd(dy.data_ptr(), x.data_ptr(), w.data_ptr(), rstd.data_ptr(), dx.data_ptr(), L.ptr(dw),
                                   M, H, L.dtype_id(x.dtype), ws.data_ptr() if with_dw else None, n, L.stream_of(x)),
            "lf_rmsnorm_bwd")
    return dx, dw


# rows x width: one row, fewer rows than a workgroup's waves, ragged widths below each register tiling (64..8192
# elements per row in steps of 8), the exact-fit widths, and more rows than the persistent grid has waves
RMS_SHAPES = [(1, 64), (3, 8), (5, 1000), (130, 1024), (67, 1536), (257, 2048), (96, 3584), (300, 4096), (33, 5120),
              (41, 8192), (5000, 512)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", RMS_SHAPES)
def test_rmsnorm_forward_backward(shape, dtype):
    M, H = shape
    eps = 1e-5
    x = _rand(shape, dtype, 10 + H, scale=2.0)
    w = (1.0 + 0.2 * _rand((H,), torch.float32, 11)).to(dtype)
    dy = _rand(shape, dtype, 12 + M)
    print(f"rmsnorm {shape} {dtype}", flush=True)
    y, rstd = _rms_fwd_abi(x.cuda(), w.cuda(), eps)
    torch.cuda.synchronize()
    yo, rstdo = R.rms_norm_fwd(x, w, eps)
    ye, rstde = R.rms_norm_fwd_exact(x, w, eps)
    assert torch.allclose(rstd.cpu().double(), rstde, rtol=2e-6, atol=0)
    assert R.ulp16_err(y.cpu(), yo.double()) <= 3.0 and float((y.cpu() != yo).float().mean()) < 2e-3
    assert R.ulp16_err(y.cpu(), ye) <= 1.51
    dx, dw = _rms_bwd_abi(dy.cuda(), x.cuda(), w.cuda(), rstd)
    torch.cuda.synchronize()
    dxe, dwe = R.rms_norm_bwd_exact(dy, x, w, eps)
    _close(dx, dxe, "dx")
    _close(dw, dwe, "dw")
    # without the weight gradient: the same dx, bit for bit; and in place over dy
    dx2, none = _rms_bwd_abi(dy.cuda(), x.cuda(), w.cuda(), rstd, with_dw=False)
    assert none is None and torch.equal(dx2, dx)
    buf = dy.cuda().clone()
    dx3, dw3 = _rms_bwd_abi(buf, x.cuda(), w.cuda(), rstd, dx=buf)
    torch.cuda.synchronize()
    assert torch.equal(dx3, dx) and torch.equal(dw3, dw)


def test_rmsnorm_layer_size_and_scale_invariance():
    """16512 x 4096 (the rows of the 8B-layer workload): sampled rows against the oracle, dw in full, and with
    eps = 0 the output must not change by one bit when the input is doubled (every step scales by a power of two)."""
    M, H = 16512, 4096
    x, dy = _rand((M, H), torch.bfloat16, 1, scale=1.5), _rand((M, H), torch.bfloat16, 2)
    w = (1.0 + 0.1 * _rand((H,), torch.float32, 3)).to(torch.bfloat16)
    xd, wd, dyd = x.cuda(), w.cuda(), dy.cuda()
    y, rstd = _rms_fwd_abi(xd, wd, 1e-6)
    rows = torch.arange(0, M, 397)
    yo, _ = R.rms_norm_fwd(x[rows], w, 1e-6)
    assert R.ulp16_err(y[rows.cuda()].cpu(), yo.double()) <= 3.0
    dx, dw = _rms_bwd_abi(dyd, xd, wd, rstd)
    dxe, _ = R.rms_norm_bwd_exact(dy[rows], x[rows], w, 1e-6)
    _close(dx[rows.cuda()], dxe, "dx")
    _, dwe = R.rms_norm_bwd_exact(dy, x, w, 1e-6)
    _close(dw, dwe, "dw")
    y0, r0 = _rms_fwd_abi(xd, wd, 0.0)
    y2, r2 = _rms_fwd_abi(xd * 2, wd, 0.0)
    assert torch.equal(y0, y2) and torch.equal(r0, r2 * 2)
    # dw does not depend on which workgroup took which rows: two runs agree bit for bit
    _, dw_again = _rms_bwd_abi(dyd, xd, wd, rstd)
    assert torch.equal(dw, dw_again)


def _silu_fwd_abi(a, b, I):
    L = _lib()
    M = a.shape[0]
    c = torch.empty((M, I), dtype=a.dtype, device=a.device)
    L.check(L.lib().lf_silu_mul_fwd(a.data_ptr(), b.data_ptr(), c.data_ptr(), M, I, a.stride(0), b.stride(0), I,
                                    L.dtype_id(a.dtype), L.stream_of(a)), "lf_silu_mul_fwd")
    return c


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(1, 8), (7, 264), (130, 2048), (1, 14336), (515, 1032)])
@pytest.mark.parametrize("merged", [False, True])
def test_silu_mul_forward_backward(shape, dtype, merged):
    M, I = shape
    a, b, dc = _rand(shape, dtype, 20, scale=3.0), _rand(shape, dtype, 21), _rand(shape, dtype, 22)
    print(f"silu_mul {shape} {dtype} merged={merged}", flush=True)
    L = _lib()
    if merged:
        gu = torch.cat([a, b], dim=1).cuda()
        ad, bd = gu[:, :I], gu[:, I:]
    else:
        ad, bd = a.cuda(), b.cuda()
    c = _silu_fwd_abi(ad, bd, I)
    torch.cuda.synchronize()
    co = R.silu_mul_fwd(a, b)
    assert R.ulp16_err(c.cpu(), co.double()) <= 3.0 and float((c.cpu() != co).float().mean()) < 2e-3
    assert R.ulp16_err(c.cpu(), R.silu_mul_fwd_exact(a, b)) <= 1.51
    dg = torch.empty((M, 2 * I), dtype=dtype, device="cuda")
    da, db = (dg[:, :I], dg[:, I:]) if merged else (torch.empty_like(ad), torch.empty_like(bd))
    dcd = dc.cuda()
    L.check(L.lib().lf_silu_mul_bwd(dcd.data_ptr(), ad.data_ptr(), bd.data_ptr(), da.data_ptr(), db.data_ptr(), M, I, I,
                                    ad.stride(0), bd.stride(0), da.stride(0), db.stride(0), L.dtype_id(dtype),
                                    L.stream_of(ad)), "lf_silu_mul_bwd")
    torch.cuda.synchronize()
    dae, dbe = R.silu_mul_bwd_exact(dc, a, b)
    assert R.ulp16_err(db.cpu(), dbe) <= 0.51
    # silu'(a) = silu (1 - sig) + sig cancels near its root (a ~ -1.28): there the fp32 error of the bracket, 1e-6 of
    # |dc b|, is what remains next to the half spacing of the final rounding
    fp32_term = 1e-6 * (dc.double() * b.double()).abs()
    assert bool(((da.cpu().double() - dae).abs() <= 0.51 * _spacing(dae, dtype) + fp32_term).all())
    _close(da, dae, "da")
    _close(db, dbe, "db")
    # in place, as liger stores the gradients over its inputs
    a2, b2 = ad.clone(), bd.clone()
    L.check(L.lib().lf_silu_mul_bwd(dcd.data_ptr(), a2.data_ptr(), b2.data_ptr(), a2.data_ptr(), b2.data_ptr(), M, I, I,
                                    a2.stride(0), b2.stride(0), a2.stride(0), b2.stride(0), L.dtype_id(dtype),
                                    L.stream_of(ad)), "lf_silu_mul_bwd")
    torch.cuda.synchronize()
    assert torch.equal(a2, da) and torch.equal(b2, db)


def test_silu_mul_layer_size_is_linear_in_up():
    """16512 x 14336 halves of a merged [16512, 28672] tensor: sampled rows against the oracle; doubling ``up``
    doubles the output bit for bit."""
    M, I = 16512, 14336
    g = torch.Generator(device="cuda").manual_seed(5)
    gu = (torch.randn(M, 2 * I, device="cuda", generator=g) * 2).to(torch.bfloat16)
    c = _silu_fwd_abi(gu[:, :I], gu[:, I:], I)
    rows = torch.arange(0, M, 1031, device="cuda")
    co = R.silu_mul_fwd(gu[rows, :I].cpu(), gu[rows, I:].cpu())
    assert R.ulp16_err(c[rows].cpu(), co.double()) <= 3.0
    gu2 = gu.clone()
    gu2[:, I:] *= 2
    c2 = _silu_fwd_abi(gu2[:, :I], gu2[:, I:], I)
    assert torch.equal(c2, c * 2)


def test_autograd_layer_and_hf_patch():
    """The autograd Functions, the merged variant against the two-tensor one, and HF's Llama classes under
    ``apply_liger_kernel`` against the oracle."""
    from transformers.models.llama import modeling_llama as ml
    from transformers.models.llama.configuration_llama import LlamaConfig

    from lorafusion_amd.ops import norm_act
    from lorafusion_amd.utils.module import apply_liger_kernel, restore_liger_kernel

    M, H, I = 200, 512, 1024
    x = _rand((2, M // 2, H), torch.bfloat16, 30, scale=2.0)
    dy = _rand((2, M // 2, H), torch.bfloat16, 31)
    norm = norm_act.RMSNorm(H, eps=1e-5, device="cuda", dtype=torch.bfloat16)
    with torch.no_grad():
        norm.weight.copy_((1.0 + 0.2 * _rand((H,), torch.float32, 32)).cuda())
    xd = x.cuda().requires_grad_(True)
    y = norm(xd)
    y.backward(dy.cuda())
    w = norm.weight.detach().cpu()
    yo, _ = R.rms_norm_fwd(x.reshape(M, H), w, 1e-5)
    dxe, dwe = R.rms_norm_bwd_exact(dy.reshape(M, H), x.reshape(M, H), w, 1e-5)
    assert y.shape == x.shape and R.ulp16_err(y.reshape(M, H).cpu(), yo.double()) <= 3.0
    _close(xd.grad.reshape(M, H), dxe, "dx")
    _close(norm.weight.grad, dwe, "dw")
    # frozen weight: no dw is computed, dx is the same
    norm.weight.requires_grad_(False)
    xd2 = x.cuda().requires_grad_(True)
    norm(xd2).backward(dy.cuda())
    assert torch.equal(xd2.grad, xd.grad)

    gu = _rand((M, 2 * I), torch.bfloat16, 33, scale=2.0).cuda()
    dc = _rand((M, I), torch.bfloat16, 34).cuda()
    g1 = gu.clone().requires_grad_(True)
    c1 = norm_act.silu_mul_merged(g1)
    c1.backward(dc)
    g2 = gu.clone().requires_grad_(True)
    a, b = torch.split(g2, [I, I], dim=-1)
    c2 = norm_act.silu_mul(a, b)
    c2.backward(dc)
    assert torch.equal(c1, c2) and torch.equal(g1.grad, g2.grad)
    dae, dbe = R.silu_mul_bwd_exact(dc.cpu(), gu[:, :I].cpu(), gu[:, I:].cpu())
    _close(g1.grad[:, :I], dae, "da")
    _close(g1.grad[:, I:], dbe, "db")

    cfg = LlamaConfig(hidden_size=H, intermediate_size=I, num_hidden_layers=1, num_attention_heads=4,
                      num_key_value_heads=4, vocab_size=32)
    torch.manual_seed(0)
    mlp = ml.LlamaMLP(cfg).to("cuda", torch.bfloat16)
    hn = ml.LlamaRMSNorm(H, eps=1e-5).to("cuda", torch.bfloat16)
    xm = x.reshape(M, H).cuda()
    ref_out = mlp(hn(xm))
    apply_liger_kernel("all")
    try:
        assert ml.LlamaMLP.forward is not None
        xr = xm.clone().requires_grad_(True)
        out = mlp(hn(xr))
        out.float().square().mean().backward()
    finally:
        restore_liger_kernel()
    # the patched modules compute what HF's compute (same roundings; the GEMMs are torch's in both)
    _close(out, ref_out.detach().float().cpu(), "patched mlp(norm(x))")
    assert xr.grad is not None and torch.isfinite(xr.grad.float()).all()
    # and the activation inside is the oracle's
    gate, up = mlp.gate_proj(hn(xm)), mlp.up_proj(hn(xm))
    co = R.silu_mul_fwd(gate.detach().cpu(), up.detach().cpu())
    assert R.ulp16_err(norm_act.silu_mul(gate, up).detach().cpu(), co.double()) <= 3.0


def test_rejected_shapes_enqueue_nothing():
    L = _lib()
    x = torch.zeros(4, 8200, dtype=torch.bfloat16, device="cuda")
    w = torch.ones(8200, dtype=torch.bfloat16, device="cuda")
    y = torch.full_like(x, 7.0)
    rstd = torch.empty(4, dtype=torch.float32, device="cuda")
    rc = L.lib().lf_rmsnorm_fwd(x.data_ptr(), w.data_ptr(), y.data_ptr(), rstd.data_ptr(), 4, 8200, 1e-6, 0, None)
    torch.cuda.synchronize()
    assert rc == L.LF_ELIMIT and bool((y == 7.0).all())
    from lorafusion_amd.ops import norm_act

    with pytest.raises(RuntimeError, match="lf_rmsnorm_fwd failed"):
        norm_act.rms_norm(x, w)
    with pytest.raises(ValueError, match="dtype"):
        norm_act.rms_norm(x[:, :64].contiguous(), w[:64].float())
    assert ctypes.sizeof(ctypes.c_void_p) == 8


def test_empty_three_dimensional_and_strided_inputs():
    from lorafusion_amd.ops import norm_act

    w = torch.ones(64, dtype=torch.bfloat16, device="cuda", requires_grad=True)
    # no rows: nothing is launched, shapes and gradients are still right
    x0 = torch.empty(0, 64, dtype=torch.bfloat16, device="cuda", requires_grad=True)
    y0 = norm_act.rms_norm(x0, w, 1e-6)
    y0.sum().backward()
    assert y0.shape == (0, 64) and x0.grad.shape == (0, 64) and torch.count_nonzero(w.grad) == 0
    g0 = torch.empty(2, 0, 128, dtype=torch.bfloat16, device="cuda", requires_grad=True)
    c0 = norm_act.silu_mul_merged(g0)
    c0.sum().backward()
    assert c0.shape == (2, 0, 64) and g0.grad.shape == g0.shape
    # [batch, seq, hidden] with a transposed (non-contiguous) batch/seq layout, and column slices as operands
    x = _rand((5, 7, 64), torch.bfloat16, 40, scale=2.0)
    xt = x.cuda().transpose(0, 1)                     # [7, 5, 64], strides (64, 448, 1)
    y = norm_act.rms_norm(xt, w.detach(), 1e-5)
    yo, _ = R.rms_norm_fwd(x.transpose(0, 1).reshape(35, 64), torch.ones(64, dtype=torch.bfloat16), 1e-5)
    assert y.shape == (7, 5, 64) and R.ulp16_err(y.reshape(35, 64).cpu(), yo.double()) <= 3.0
    big = _rand((33, 400), torch.bfloat16, 41, scale=2.0).cuda()
    a, b = big[:, 8:136], big[:, 200:328]               # 128 columns each, row stride 400, 16-byte aligned starts
    c = norm_act.silu_mul(a, b)
    co = R.silu_mul_fwd(a.cpu(), b.cpu())
    assert R.ulp16_err(c.cpu(), co.double()) <= 3.0
    a2, b2 = big[:, 4:132], big[:, 204:332]             # starts that are not 16-byte aligned: copied, same result rule
    c2 = norm_act.silu_mul(a2, b2)
    assert R.ulp16_err(c2.cpu(), R.silu_mul_fwd(a2.cpu(), b2.cpu()).double()) <= 3.0
