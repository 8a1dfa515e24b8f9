"""SiLU-multiply as the prologue of the down projection's LoRA linear (GPU).

``lf_lora_xa_silu_mul`` must write exactly what ``lf_silu_mul_fwd`` writes and produce exactly the ``S`` that
``lf_lora_xa`` / ``lf_lora_xa_seeded`` produce on it (bit for bit: the same arithmetic, the same summation order), and
the autograd layer on top must match the oracle -- ``silu_mul_fwd`` (rounded where the algorithm rounds), then the
LoRA-linear oracle on the product, its ``dX`` through the fp64 SiLU-multiply gradient; |err| <= 1e-2 |e| + 1e-2 rms(e) --
and, bit for bit, the unfused composition of the same HIP ops.
"""

from __future__ import annotations

import ctypes

import pytest
import torch

from oracle import lora_ref
from oracle import norm_act_ref as R
from tests.util import multi_inputs, single_inputs

pytestmark = pytest.mark.gpu


def _close(got, exp, name):
    ok, rel, excess = lora_ref.check_close(got.detach().float().cpu(), exp, rtol=1e-2)
    assert ok, f"{name}: max|err|/max|e| = {rel:.3e}, worst excess over bound {excess:.3e}"


def _gate_up(M, K, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(M, 2 * K, generator=g) * 1.5).to(dtype)


def _xa_silu_abi(gu, a_list, routing_c, R_cols, mask=None, seed=None):
    from lorafusion_amd import _lib as L

    M, K = gu.shape[0], gu.shape[1] // 2
    x = torch.empty((M, K), dtype=gu.dtype, device=gu.device)
    s = torch.empty((M, R_cols), dtype=gu.dtype, device=gu.device)
    mask_out = torch.empty((M, K), dtype=torch.bool, device=gu.device) if seed is not None else None
    rc = L.lib().lf_lora_xa_silu_mul(gu.data_ptr(), gu[:, K:].data_ptr(), 2 * K, x.data_ptr(), L.ptr(mask), L.ptr(mask_out),
                                     ctypes.c_uint64(seed or 0), L.ptr_array(a_list), s.data_ptr(), M, K, R_cols, routing_c,
                                     L.dtype_id(gu.dtype), L.stream_of(gu))
    L.check(rc, "lf_lora_xa_silu_mul")
    return x, s, mask_out


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rank", [16, 24, 64, 128])
@pytest.mark.parametrize("mode", ["none", "mask", "seed"])
def test_prologue_equals_activation_then_xa_single(rank, mode, dtype):
    from lorafusion_amd import _lib as L
    from lorafusion_amd.ops import hip_ops, norm_act

    M, K, p = 203, 512, 0.1       # a row count that is no multiple of the 16-row blocks
    print(f"xa_silu single r={rank} {mode} {dtype}", flush=True)
    gu = _gate_up(M, K, dtype, 1).cuda()
    a = ((torch.rand(rank, K, generator=torch.Generator().manual_seed(2)) * 2 - 1) / K ** 0.5).to(dtype).cuda()
    Rc = L.round_rank(rank)
    use_p = p if mode != "none" else 0.0
    routing = L.single_routing(rank, 2.0, use_p)
    mask = (torch.rand(M, K, generator=torch.Generator().manual_seed(3)) >= p).cuda() if mode == "mask" else None
    x, s, mask_out = _xa_silu_abi(gu, [a], routing, Rc, mask=mask, seed=77 if mode == "seed" else None)
    c = norm_act.silu_mul_merged(gu)
    assert torch.equal(x, c)
    if mode == "seed":
        exp_mask = hip_ops.make_dropout_mask((M, K), p, 77, "cuda")
        assert torch.equal(mask_out, exp_mask)
        mask = exp_mask
    s_ref = hip_ops._xa(c, mask, [a], routing, M, K, Rc)
    assert torch.equal(s, s_ref)
    # and against the oracle: S = drop(c) A^T (1/(1-p) applied), c the rounded activation
    co = R.silu_mul_fwd(gu[:, :K].cpu(), gu[:, K:].cpu())
    assert R.ulp16_err(x.cpu(), co.double()) <= 3.0
    _, s_exp = lora_ref.linear_lora_fwd_fp32(x.cpu(), torch.zeros(8, K), a.cpu(), torch.zeros(8, rank), 1.0,
                                             mask.cpu() if mask is not None else None, use_p)
    _close(s[:, :rank], s_exp, "S")


@pytest.mark.parametrize("ranks", [[16, 16, 16], [8, 64, 32], [48, 16]])
@pytest.mark.parametrize("seeded", [False, True])
def test_fused_layer_against_oracle_and_unfused_ops_multi(ranks, seeded):
    from lorafusion_amd.ops import multi_lora as ml
    from lorafusion_amd.ops import norm_act
    from lorafusion_amd.ops.swiglu_lora import fused_swiglu_linear_multi_lora

    seq = [200, 129, 300][: len(ranks)]
    p_list, scales = [0.1, 0.0, 0.05][: len(ranks)], [2.0, 1.0, 0.5][: len(ranks)]
    K, N = 1024, 384
    print(f"swiglu multi ranks={ranks} seeded={seeded}", flush=True)
    d = multi_inputs(seq, K, N, ranks, p_list, seed=5)
    Mp = sum(d["padded"])
    gu = _gate_up(Mp, K, torch.bfloat16, 6)
    info = ml.prepare_multi_lora_batch_info(seq, list(range(len(seq))), ranks, p_list, scales, 128)
    routing = info.routing(enable_dropout=True)
    w = d["w"].cuda()

    def run(fused):
        g = gu.cuda().requires_grad_(True)
        a = [t.cuda().requires_grad_(True) for t in d["a_list"]]
        b = [t.cuda().requires_grad_(True) for t in d["b_list"]]
        kw = dict(seed=1234) if seeded else dict(dropout_mask=d["mask"].cuda())
        if fused:
            y = fused_swiglu_linear_multi_lora(g, w, a, b, routing, **kw)
        else:
            c = norm_act.silu_mul_merged(g)
            y = ml.fused_linear_multi_lora(
                c, w, lora_a_list=a, lora_b_list=b, seq_len_list=seq, padded_seq_len_list=info.padded_seq_len_list,
                block_to_lookup_table=info.block_to_lookup_table, block_to_dropout_p=info.block_to_dropout_p,
                block_to_alpha=info.block_to_alpha, enable_dropout=True, same_dropout_p_value=None, max_r=max(ranks),
                routing=routing, **kw)
        y.backward(d["dy"].cuda())
        torch.cuda.synchronize()
        return y.detach(), g.grad, [t.grad for t in a], [t.grad for t in b]

    y, dg, da, db = run(True)
    y0, dg0, da0, db0 = run(False)
    assert torch.equal(y, y0) and torch.equal(dg, dg0)
    for i in range(len(ranks)):
        assert torch.equal(da[i], da0[i]) and torch.equal(db[i], db0[i])
    if not seeded:
        c = R.silu_mul_fwd(gu[:, :K], gu[:, K:])
        ye, _ = lora_ref.linear_multi_lora_fwd_fp32(c, d["w"], d["a_list"], d["b_list"], seq, d["padded"], scales, p_list, d["mask"])
        dce, dae, dbe, _ = lora_ref.linear_multi_lora_bwd_fp32(d["dy"], c, d["w"], d["a_list"], d["b_list"], seq, d["padded"],
                                                               scales, p_list, d["mask"])
        dge_a, dge_b = R.silu_mul_bwd_exact(dce, gu[:, :K], gu[:, K:])
        _close(y, ye, "y")
        _close(dg[:, :K], dge_a, "d gate")
        _close(dg[:, K:], dge_b, "d up")
        for i in range(len(ranks)):
            _close(da[i], dae[i], f"da{i}")
            _close(db[i], dbe[i], f"db{i}")


@pytest.mark.parametrize("p", [0.0, 0.1])
def test_fused_layer_single_adapter_with_bias(p):
    from lorafusion_amd.ops.swiglu_lora import fused_swiglu_linear_lora

    M, K, N, r = 333, 768, 256, 16
    d = single_inputs(M, K, N, r, p=p, seed=9, bias=True)
    gu = _gate_up(M, K, torch.bfloat16, 10)
    g = gu.cuda().reshape(1, M, 2 * K).requires_grad_(True)
    a, b = d["a"].cuda().requires_grad_(True), d["b"].cuda().requires_grad_(True)
    mask = d["mask"].cuda() if p > 0 else None
    y = fused_swiglu_linear_lora(g, d["w"].cuda(), a, b, 0.5, dropout_p=p, linear_bias=d["bias"].cuda(), dropout_mask=mask)
    assert y.shape == (1, M, N)
    y.backward(d["dy"].cuda().reshape(1, M, N))
    torch.cuda.synchronize()
    c = R.silu_mul_fwd(gu[:, :K], gu[:, K:])
    ye, _ = lora_ref.linear_lora_fwd_fp32(c, d["w"], d["a"], d["b"], 0.5, d["mask"], p, d["bias"])
    dce, dae, dbe, _ = lora_ref.linear_lora_bwd_fp32(d["dy"], c, d["w"], d["a"], d["b"], 0.5, d["mask"], p)
    dga, dgb = R.silu_mul_bwd_exact(dce, gu[:, :K], gu[:, K:])
    _close(y[0], ye, "y")
    _close(g.grad[0][:, :K], dga, "d gate")
    _close(g.grad[0][:, K:], dgb, "d up")
    _close(a.grad, dae, "da")
    _close(b.grad, dbe, "db")


def test_layer_harness_takes_the_prologue_path(monkeypatch):
    """``DecoderLayerLoRAProjections`` without a caller-supplied activation runs the down projection through
    ``lf_swiglu_lora_fwd`` and gives what the activation kernel followed by the plain LoRA linear gives."""
    from lorafusion_amd import _lib as L
    from lorafusion_amd.ops import norm_act
    from lorafusion_amd.patch.patch_transformers import DecoderLayerLoRAProjections

    layer = DecoderLayerLoRAProjections.from_shapes(512, 128, 1024, {"default": (16, 32.0, 0.0)}, seed=5)
    for lin in layer.linears().values():
        torch.nn.init.normal_(lin.lora_B["default"].weight, std=0.01)
    x = torch.randn(256, 512, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16).cuda()
    calls = []
    real_lib = L.lib()

    def counting(*args):
        calls.append(1)
        return real_lib.lf_swiglu_lora_fwd(*args)

    class _Lib:
        def __getattr__(self, name):
            return counting if name == "lf_swiglu_lora_fwd" else getattr(real_lib, name)

    monkeypatch.setattr(L, "lib", lambda: _Lib())
    out = layer(x)
    assert len(calls) == 1
    monkeypatch.undo()
    out2 = layer(x, activation=lambda g, u: norm_act.silu_mul(g, u))
    assert torch.equal(out, out2)


def test_argument_errors():
    from lorafusion_amd import _lib as L

    gu = torch.zeros(128, 512, dtype=torch.bfloat16, device="cuda")
    a = torch.zeros(16, 256, dtype=torch.bfloat16, device="cuda")
    x = torch.full((128, 256), 3.0, dtype=torch.bfloat16, device="cuda")
    s = torch.zeros(128, 16, dtype=torch.bfloat16, device="cuda")
    m = torch.ones(128, 256, dtype=torch.bool, device="cuda")
    r = L.single_routing(16, 1.0, 0.1)
    lib = L.lib()
    args = lambda ld, mask, mask_out: (gu.data_ptr(), gu[:, 256:].data_ptr(), ld, x.data_ptr(), mask, mask_out, ctypes.c_uint64(1),
                                       L.ptr_array([a]), s.data_ptr(), 128, 256, 16, r, 0, None)
    assert lib.lf_lora_xa_silu_mul(*args(512, m.data_ptr(), m.data_ptr())) == L.LF_EINVAL   # both kinds of mask
    assert lib.lf_lora_xa_silu_mul(*args(248, None, None)) == L.LF_ESHAPE                     # rows closer than K
    assert lib.lf_lora_xa_silu_mul(*args(516, None, None)) == L.LF_ESHAPE                     # stride not a multiple of 8
    torch.cuda.synchronize()
    assert bool((x == 3.0).all())
    from lorafusion_amd.ops.swiglu_lora import fused_swiglu_linear_lora

    with pytest.raises(ValueError, match="multiple of 256"):
        fused_swiglu_linear_lora(gu[:, :384].contiguous(), torch.zeros(128, 192, dtype=torch.bfloat16, device="cuda"), a[:, :192], 
                                 torch.zeros(128, 16, dtype=torch.bfloat16, device="cuda"), 1.0)


def test_separate_gate_and_up_tensors_and_the_patched_hf_mlp():
    """gate and up as two tensors (what HF's ``LlamaMLP`` produces): the same results as the merged layout, bit for
    bit; and an HF ``LlamaMLP`` whose ``down_proj`` is a LoRA linear takes the prologue path under
    ``apply_liger_kernel`` and matches the unpatched module."""
    from transformers.models.llama import modeling_llama as mlm
    from transformers.models.llama.configuration_llama import LlamaConfig

    from lorafusion_amd import _lib as L
    from lorafusion_amd.ops.swiglu_lora import fused_swiglu_linear_lora
    from lorafusion_amd.patch.patch_transformers import LoRALinear
    from lorafusion_amd.utils.module import apply_liger_kernel, restore_liger_kernel

    M, K, N, r = 260, 512, 384, 32
    d = single_inputs(M, K, N, r, p=0.1, seed=3)
    gu = _gate_up(M, K, torch.bfloat16, 4).cuda()

    def run(separate):
        a, b = d["a"].cuda().requires_grad_(True), d["b"].cuda().requires_grad_(True)
        if separate:
            g, u = gu[:, :K].contiguous().requires_grad_(True), gu[:, K:].contiguous().requires_grad_(True)
            y = fused_swiglu_linear_lora(g, d["w"].cuda(), a, b, 2.0, dropout_p=0.1, dropout_mask=d["mask"].cuda(), up=u)
        else:
            g = gu.clone().requires_grad_(True)
            y = fused_swiglu_linear_lora(g, d["w"].cuda(), a, b, 2.0, dropout_p=0.1, dropout_mask=d["mask"].cuda())
        y.backward(d["dy"].cuda())
        dg = torch.cat([g.grad, u.grad], dim=1) if separate else g.grad
        return y.detach(), dg, a.grad, b.grad

    for got, exp in zip(run(True), run(False)):
        assert torch.equal(got, exp)

    H, I = 256, 512
    cfg = LlamaConfig(hidden_size=H, intermediate_size=I, num_hidden_layers=1, num_attention_heads=4,
                      num_key_value_heads=4, vocab_size=32)
    torch.manual_seed(0)
    mlp = mlm.LlamaMLP(cfg).to("cuda", torch.bfloat16)
    mlp.down_proj = LoRALinear(mlp.down_proj, {"default": (16, 32.0, 0.0)})
    torch.nn.init.normal_(mlp.down_proj.lora_B["default"].weight, std=0.02)
    x = torch.randn(200, H, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16).cuda()
    ref = mlp(x)
    calls = []
    real_lib = L.lib()

    class _Lib:
        def __getattr__(self, name):
            if name == "lf_swiglu_lora_fwd":
                calls.append(1)
            return getattr(real_lib, name)

    apply_liger_kernel("all")
    try:
        import unittest.mock as mock

        with mock.patch.object(L, "lib", lambda: _Lib()):
            xr = x.clone().requires_grad_(True)
            out = mlp(xr)
            out.float().square().mean().backward()
    finally:
        restore_liger_kernel()
    assert len(calls) == 1
    _close(out, ref.detach().float().cpu(), "patched MLP with a LoRA down projection")
    assert torch.isfinite(xr.grad.float()).all() and mlp.down_proj.lora_A["default"].weight.grad is not None
