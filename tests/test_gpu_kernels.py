"""GPU parity of the kernel-level wrappers (one per reference Triton wrapper) and of the plain GEMM
in every tile configuration, against fp32 CPU expressions built from the oracle's formulas."""

import pytest
import torch

from oracle import lora_ref
from tests.util import single_inputs

pytestmark = pytest.mark.gpu


def _close(actual, expected, what, rtol=1e-2):
    ok, rel, excess = lora_ref.check_close(actual.detach().float().cpu(), expected, rtol=rtol)
    assert ok, f"{what}: max|err|/max|e| = {rel:.3e}, worst excess {excess:.3e}"


@pytest.mark.parametrize("cfg", [0, 1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("trans_b", [True, False])
@pytest.mark.parametrize("M,N,K", [(256, 256, 128), (520, 640, 384), (1024, 1280, 1024), (77, 136, 64), (130, 72, 704),
                                   (256, 264, 64), (300, 256, 192), (2100, 4360, 320)])
def test_gemm_all_tiles(cfg, trans_b, M, N, K):
    from lorafusion_amd.ops import hip_ops

    if cfg == 7 and (M < 256 or N < 256 or K < 128):
        pytest.skip("the persistent 256x256 kernel shifts edge tiles inwards (M, N >= 256) and pipelines two K steps (K >= 128)")
    if cfg == 8 and (M < 128 or N < 256 or K < 256):
        pytest.skip("the persistent 128x256 kernel shifts edge tiles inwards (M >= 128, N >= 256) and pipelines three K steps (K >= 256)")

    g = torch.Generator().manual_seed(M + N + K)
    a = torch.randn(M, K, generator=g).bfloat16()
    b = (torch.randn(N, K, generator=g) if trans_b else torch.randn(K, N, generator=g)).bfloat16()
    c = hip_ops.gemm(a.cuda(), b.cuda(), trans_b=trans_b, tile_cfg=cfg)
    e = a.float() @ (b.float().T if trans_b else b.float())
    _close(c, e, f"gemm cfg={cfg} trans_b={trans_b}")


@pytest.mark.parametrize("trans_b", [True, False])
@pytest.mark.parametrize("M,N", [(4352, 4096), (8448, 4096), (2304, 8192), (4100, 4096)])
def test_gemm_row_split_plan(trans_b, M, N):
    """Automatic tile choice: row counts just above whole rounds of 256x256 tiles run as two launches
    (whole rounds + a short tail with small tiles); every row must still be the product.  (Tiles of
    different shapes start their K loop at different offsets, so the plans agree to rounding, not bitwise.)"""
    from lorafusion_amd.ops import hip_ops

    K = 128
    g = torch.Generator().manual_seed(M + N)
    a = torch.randn(M, K, generator=g).bfloat16().cuda()
    b = (torch.randn(N, K, generator=g) if trans_b else torch.randn(K, N, generator=g)).bfloat16().cuda()
    auto = hip_ops.gemm(a, b, trans_b=trans_b)
    e = a.float().cpu() @ (b.float().cpu().T if trans_b else b.float().cpu())
    _close(auto, e, f"gemm auto plan M={M} N={N} trans_b={trans_b}")


@pytest.mark.parametrize("trans_b", [True, False])
def test_gemm_row_operand_above_2_gib(trans_b):
    """A row operand of 2.46 GB (300000 x 4096): the tile loads address one 256-row panel at a time, so only the
    panel has to fit 32-bit offsets.  Checked on the first, last and some middle rows against fp32 torch."""
    from lorafusion_amd.ops import hip_ops

    M, K, N = 300_000, 4096, 128
    g = torch.Generator(device="cuda").manual_seed(3)
    a = torch.randn(M, K, generator=g, device="cuda").bfloat16()
    b = (torch.randn(N, K, generator=g, device="cuda") if trans_b else torch.randn(K, N, generator=g, device="cuda")).bfloat16()
    c = hip_ops.gemm(a, b, trans_b=trans_b)
    rows = torch.tensor([0, 1, 255, 256, 131_071, 131_072, 262_143, 262_144, 262_145, M - 257, M - 2, M - 1], device="cuda")
    e = a[rows].float() @ (b.float().T if trans_b else b.float())
    _close(c[rows], e.cpu(), f"gemm rows of a 2.46 GB operand, trans_b={trans_b}")
    del a, c


def test_gemm_identity_exact():
    """A @ I^T reproduces A bit for bit in every layout (catches operand / index transpositions)."""
    from lorafusion_amd.ops import hip_ops

    g = torch.Generator().manual_seed(0)
    a = torch.randn(300, 256, generator=g).bfloat16().cuda()
    eye = torch.eye(256).bfloat16().cuda()
    for trans_b in (True, False):
        for cfg in range(7):
            assert torch.equal(hip_ops.gemm(a, eye, trans_b=trans_b, tile_cfg=cfg), a)
    # a permutation matrix tells B from B^T
    perm = torch.randperm(256, generator=g)
    pm = torch.zeros(256, 256)
    pm[torch.arange(256), perm] = 1.0   # pm[i, perm[i]] = 1
    pmb = pm.bfloat16().cuda()
    assert torch.equal(hip_ops.gemm(a, pmb, trans_b=False), a[:, torch.argsort(perm).cuda()])   # a @ pm
    assert torch.equal(hip_ops.gemm(a, pmb, trans_b=True), a[:, perm.cuda()])                   # a @ pm.T


def test_tier2_wrappers():
    from lorafusion_amd.ops import triton_ops as T

    M, K, N, r, p, alpha = 384, 512, 640, 16, 0.1, 2.0
    d = single_inputs(M, K, N, r, p=p, seed=4, bias=True)
    x, w, a, b, dy, mask, bias = (d[k].cuda() for k in ("x", "w", "a", "b", "dy", "mask", "bias"))
    xt = lora_ref.dropout_explicit(d["x"].float(), d["mask"], p)

    s, m_out, xs = T.fused_dropout_matmul(x, a, p, dropout_mask=mask, store_mask=True, store_masked_scaled_x=True)
    s_e = xt @ d["a"].float().T
    _close(s[:, :r], s_e, "fused_dropout_matmul s")
    assert torch.equal(m_out, mask)
    _close(xs, xt, "masked_scaled_x", rtol=1e-2)

    y = T.fused_lora_xw_sb(x, w, s, b, alpha, bias)
    y_e = d["x"].float() @ d["w"].float().T + (s[:, :r].float().cpu() @ d["b"].float().T) * alpha + d["bias"].float()
    _close(y, y_e, "fused_lora_xw_sb")

    db, ds = T.fused_lora_dys_dyb(dy, b, s, alpha)
    _close(db, (d["dy"].float().T @ s[:, :r].float().cpu()) * alpha, "db")
    _close(ds[:, :r], (d["dy"].float() @ d["b"].float()) * alpha, "ds")

    da = T.fused_lora_da(x, ds, r, p, mask)
    _close(da, ds[:, :r].float().cpu().T @ xt, "da")

    dx = T.fused_lora_dyw_dsa(dy, w, ds, a, p, mask)
    dx_e = d["dy"].float() @ d["w"].float() + lora_ref.dropout_explicit(ds[:, :r].float().cpu() @ d["a"].float(), d["mask"], p)
    _close(dx, dx_e, "dx")

    with pytest.raises(ValueError):
        T.fused_lora_xw_sb(x, w, s[:-1].contiguous(), b, alpha)
    with pytest.raises(ValueError):
        T.fused_lora_dyw_dsa(dy, w.t(), ds, a, p, mask)
    # dropout asked for but no mask given: an error, as in the reference (fused_lora_dyw_dsa.py:234-236)
    with pytest.raises(ValueError, match="dropout_mask must be provided"):
        T.fused_lora_dyw_dsa(dy, w, ds, a, p, None)
    with pytest.raises(ValueError, match="dropout_mask must be provided"):
        T.fused_lora_da(x, ds, r, p, None)


def test_null_mask_means_no_dropout_at_the_c_abi():
    """At the C ABI a NULL keep-mask switches dropout off for the call: p of the routing is ignored and
    nothing is rescaled by 1/(1-p) (xa, da, dyw_dsa), single routing and block tables alike."""
    from lorafusion_amd import _lib as L
    from lorafusion_amd.ops import hip_ops
    from lorafusion_amd.ops.multi_lora import prepare_multi_lora_batch_info

    M, K, N, r = 256, 512, 384, 16
    d = single_inputs(M, K, N, r, p=0.0, seed=6)
    x, w, a, b, dy = (d[k].cuda() for k in ("x", "w", "a", "b", "dy"))
    lib = L.lib()
    info = prepare_multi_lora_batch_info([M], [0], [r], [0.25], [2.0], 128)
    multi = hip_ops.MultiRouting(info.padded_seq_len_list, [r], info.block_to_lookup_table, info.block_to_alpha,
                                 info.block_to_dropout_p)
    for what, rt in (("single", L.single_routing(r, 1.0, 0.25)), ("table", multi.c)):
        s = torch.empty((M, 16), dtype=x.dtype, device="cuda")
        rc = lib.lf_lora_xa(L.ptr(x), None, L.ptr_array([a]), L.ptr(s), None, 0, M, K, 16, rt, L.LF_BF16, L.stream_of(x))
        assert rc == 0
        _close(s, d["x"].float() @ d["a"].float().T, f"{what}: S without a mask")
        ds = (torch.randn(M, 16) * 0.1).to(torch.bfloat16).cuda()
        da = torch.empty((r, K), dtype=x.dtype, device="cuda")
        need = lib.lf_workspace_bytes(L.LF_OP_DA, M, 0, K, 16, rt)
        ws = torch.empty(max(need, 256), dtype=torch.uint8, device="cuda")
        rc = lib.lf_lora_da(L.ptr(x), None, L.ptr(ds), L.ptr_array([da]), L.ptr(ws), need, M, K, 16, rt, L.LF_BF16,
                            L.stream_of(x))
        assert rc == 0
        _close(da, ds.float().cpu().T @ d["x"].float(), f"{what}: dA without a mask")
        dx = torch.empty((M, K), dtype=x.dtype, device="cuda")
        rc = lib.lf_lora_dyw_dsa(L.ptr(dy), L.ptr(w), L.ptr(ds), L.ptr_array([a]), None, L.ptr(dx), M, N, K, 16, rt,
                                 L.LF_BF16, L.stream_of(x))
        assert rc == 0
        _close(dx, d["dy"].float() @ d["w"].float() + ds.float().cpu() @ d["a"].float(), f"{what}: dX without a mask")


def test_seeded_mask_statistics_and_reproducibility():
    """Seeded path (no explicit mask): same seed -> same output; keep rate ~ 1-p."""
    from lorafusion_amd.ops import hip_ops
    from lorafusion_amd.ops.lora_v1 import fused_linear_lora

    d = single_inputs(512, 512, 256, 16, p=0.0, seed=8)
    x, w, a, b = (d[k].cuda() for k in ("x", "w", "a", "b"))
    y1 = fused_linear_lora(x, w, a, b, 2.0, seed=123, dropout_p=0.3)
    y2 = fused_linear_lora(x, w, a, b, 2.0, seed=123, dropout_p=0.3)
    y3 = fused_linear_lora(x, w, a, b, 2.0, seed=124, dropout_p=0.3)
    assert torch.equal(y1, y2) and not torch.equal(y1, y3)
    m = hip_ops.make_dropout_mask((512, 512), 0.3, 123, "cuda")
    assert abs(float(m.float().mean()) - 0.7) < 0.01
