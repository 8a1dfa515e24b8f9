"""GPU parity of the bit-packed keep-mask format (element k of a row = bit k & 7 of byte k >> 3) against the
one-byte-per-element format of the reference (lorafusion/ops/triton_ops/dropout.py:79): conversion both ways against
numpy, and every kernel that reads or writes a mask -- the rank-r forward (read and drawn), dA, the dX product in its
small tiles and in the persistent kernel -- with the same mask in both formats.  Where both formats run the same
arithmetic in the same order the results must be identical bit for bit; the dX product of large shapes takes a
different kernel per format, so there both are held to the oracle's bound."""

import ctypes

import numpy as np
import pytest
import torch

from oracle import dropout as od
from oracle import lora_ref
from tests.util import multi_inputs, single_inputs

pytestmark = pytest.mark.gpu


def _close(actual, expected, what, rtol=1e-2):
    ok, rel, excess = lora_ref.check_close(actual.detach().float().cpu(), expected, rtol=rtol)
    assert ok, f"{what}: max|err|/max|e| = {rel:.3e}, worst excess {excess:.3e}"


@pytest.mark.parametrize("M,K", [(1, 128), (130, 256), (257, 1024), (64, 4096)])
def test_pack_and_unpack_against_numpy(M, K):
    from lorafusion_amd.ops import hip_ops

    rng = np.random.default_rng(M + K)
    m = rng.random((M, K)) >= 0.3
    bits = hip_ops.pack_mask(torch.from_numpy(m).cuda())
    assert bits.dtype == torch.uint8 and tuple(bits.shape) == (M, K // 8)
    assert np.array_equal(bits.cpu().numpy(), np.packbits(m, axis=1, bitorder="little"))
    assert np.array_equal(hip_ops.unpack_mask(bits).cpu().numpy(), m)
    # any non-zero byte keeps
    u8 = torch.from_numpy((m * rng.integers(1, 256, (M, K))).astype(np.uint8)).cuda()
    assert torch.equal(hip_ops.pack_mask(u8), bits)
    with pytest.raises(ValueError):
        hip_ops.pack_mask(torch.zeros(4, 64, dtype=torch.bool, device="cuda"))


@pytest.mark.parametrize("r", [8, 16, 32, 64, 128])
def test_rank_r_passes_same_result_in_both_formats(r):
    """xa and da read the mask: same S, same dA, bit for bit."""
    from lorafusion_amd.ops import hip_ops

    M, K, N, p = 300, 512, 384, 0.2
    d = single_inputs(M, K, N, r, p=p, seed=r)
    x, a, mask = d["x"].cuda(), d["a"].cuda(), d["mask"].cuda()
    bits = hip_ops.pack_mask(mask)
    s_bytes, _, _ = hip_ops.fused_dropout_matmul(x, a, p, dropout_mask=mask)
    s_bits, _, _ = hip_ops.fused_dropout_matmul(x, a, p, dropout_mask=bits)
    assert torch.equal(s_bytes, s_bits)
    ds = (torch.randn(M, r, generator=torch.Generator().manual_seed(1)) * 0.1).bfloat16().cuda()
    da_bytes = hip_ops.fused_lora_da(x, ds, r, p, mask)
    da_bits = hip_ops.fused_lora_da(x, ds, r, p, bits)
    assert torch.equal(da_bytes, da_bits)
    xd = torch.where(d["mask"], d["x"].float() / (1 - p), torch.zeros(()))
    _close(da_bits, ds.float().cpu().T @ xd, f"da r={r}")


@pytest.mark.parametrize("seq,ranks,p_list", [([100, 300, 64, 257], [16, 16, 16, 16], [0.0, 0.05, 0.1, 0.3]),
                                              ([200, 130], [64, 8], [0.25, 0.1])])
def test_multi_rank_r_passes_and_drawn_masks_in_both_formats(seq, ranks, p_list):
    from lorafusion_amd import _lib as L
    from lorafusion_amd.ops import hip_ops
    from lorafusion_amd.ops.multi_lora import prepare_multi_lora_batch_info

    K, N, seed = 512, 384, 4242
    scales = [1.0, 2.0, 2.0, 4.0][: len(seq)]
    d = multi_inputs(seq, K, N, ranks, p_list, seed=3)
    info = prepare_multi_lora_batch_info(seq, list(range(len(seq))), ranks, p_list, scales, 128, output_dtype=torch.float32)
    routing = hip_ops.MultiRouting(info.padded_seq_len_list, ranks, info.block_to_lookup_table, info.block_to_alpha,
                                   info.block_to_dropout_p)
    x, mask = d["x"].cuda(), d["mask"].cuda()
    a_list = [t.cuda() for t in d["a_list"]]
    bits = hip_ops.pack_mask(mask)
    assert torch.equal(hip_ops.fused_multi_lora_xa(x, a_list, routing, mask), hip_ops.fused_multi_lora_xa(x, a_list, routing, bits))
    M = x.shape[0]
    ds = (torch.randn(M, routing.R, generator=torch.Generator().manual_seed(5)) * 0.1).bfloat16().cuda()
    for g1, g2 in zip(hip_ops.fused_multi_lora_da(x, ds, routing, mask), hip_ops.fused_multi_lora_da(x, ds, routing, bits)):
        assert torch.equal(g1, g2)
    # the mask drawn inside the rank-r pass: same draws in both formats, same S
    expect = od.keep_mask(M, K, np.repeat(info.block_to_dropout_p.float().cpu().numpy(), 128), seed)
    outs = {}
    for packed in (False, True):
        s = torch.empty((M, routing.R), dtype=x.dtype, device="cuda")
        m = torch.zeros((M, K // 8) if packed else (M, K), dtype=torch.uint8, device="cuda")
        rc = L.lib().lf_lora_xa_seeded(L.ptr(x), L.ptr(m), L.ptr_array(a_list), L.ptr(s), M, K, routing.R, routing.c,
                                       ctypes.c_uint64(seed), L.dtype_id(x.dtype) | (L.LF_MASK_BITS if packed else 0), L.stream_of(x))
        assert rc == 0
        outs[packed] = (s, m)
    assert np.array_equal(outs[False][1].cpu().numpy(), expect)
    assert np.array_equal(outs[True][1].cpu().numpy(), np.packbits(expect, axis=1, bitorder="little"))
    assert torch.equal(outs[False][0], outs[True][0])


@pytest.mark.parametrize("M,K,N,r,p,cfg", [(300, 256, 384, 16, 0.2, -1), (256, 512, 256, 8, 0.1, 5), (520, 384, 640, 32, 0.3, 3),
                                           (384, 256, 512, 64, 0.1, 1), (640, 768, 512, 16, 0.25, 7), (512, 1024, 256, 32, 0.1, 7),
                                           (300, 384, 640, 8, 0.5, 7), (640, 768, 512, 16, 0.25, 8), (200, 384, 640, 32, 0.5, 8)])
def test_dx_product_in_both_formats(M, K, N, r, p, cfg):
    """dx = dy w + mask (ds a) / (1 - p).  cfg pins the tile; 7, 8 = the persistent kernel, which takes bits only (bytes then
    run on a small tile): both against the fp32 expression; the small tiles agree bit for bit between formats."""
    from lorafusion_amd import _lib as L
    from lorafusion_amd.ops import hip_ops

    d = single_inputs(M, K, N, r, p=p, seed=M + r)
    dy, w, a, mask = d["dy"].cuda(), d["w"].cuda(), d["a"].cuda(), d["mask"].cuda()
    ds = (torch.randn(M, r, generator=torch.Generator().manual_seed(2)) * 0.1).bfloat16()
    bits = hip_ops.pack_mask(mask)
    assert L.lib().lf_set_tile_cfg(cfg) == 0
    try:
        dx_bytes = hip_ops.fused_lora_dyw_dsa(dy, w, ds.cuda(), a, p, mask)
        dx_bits = hip_ops.fused_lora_dyw_dsa(dy, w, ds.cuda(), a, p, bits)
    finally:
        assert L.lib().lf_set_tile_cfg(-1) == 0
    e = d["dy"].float() @ d["w"].float() + torch.where(d["mask"], (ds.float() @ d["a"].float()) / (1 - p), torch.zeros(()))
    _close(dx_bytes, e, f"dx bytes cfg={cfg}")
    _close(dx_bits, e, f"dx bits cfg={cfg}")
    if cfg not in (7, 8):
        assert torch.equal(dx_bytes, dx_bits)


def test_whole_op_with_a_packed_mask_equals_the_bool_mask():
    """fused_linear_lora takes the mask in either format (it packs a bool mask once, up front)."""
    from lorafusion_amd.ops import hip_ops
    from lorafusion_amd.ops.lora_v1 import fused_linear_lora

    M, K, N, r, p = 520, 512, 640, 16, 0.1
    d = single_inputs(M, K, N, r, p=p, seed=11)
    res = []
    for fmt in ("bool", "bits"):
        x = d["x"].cuda().requires_grad_(True)
        a, b = d["a"].cuda().requires_grad_(True), d["b"].cuda().requires_grad_(True)
        m = d["mask"].cuda() if fmt == "bool" else hip_ops.pack_mask(d["mask"].cuda())
        y = fused_linear_lora(x, d["w"].cuda(), a, b, 2.0, dropout_p=p, dropout_mask=m)
        y.backward(d["dy"].cuda())
        res.append((y.detach(), x.grad, a.grad, b.grad))
    for t1, t2 in zip(*res):
        assert torch.equal(t1, t2)
