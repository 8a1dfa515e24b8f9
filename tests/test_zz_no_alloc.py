"""GPU test of lf_lora_bwd_static, the backward entry point that allocates nothing.

It is called through the C ABI and compared with lf_lora_bwd (caller-provided workspace) on the
same inputs: the two run the same kernels in the same order, so every output must be bit-identical
(torch.equal).  Two calls in a row share the library's static scratch buffer; the second is a
smaller batch, so stale partial sums of the first call lie beyond (and inside) what it uses.
A call whose partial sums do not fit the buffer must return LF_ESTATIC and leave the outputs alone.
"""

import ctypes

import pytest
import torch

from tests.util import multi_inputs, single_inputs

pytestmark = pytest.mark.gpu


def _outputs(M, N, K, ranks, dev, dtype):
    dx = torch.full((M, K), float("nan"), dtype=dtype, device=dev)
    da = [torch.full((r, K), float("nan"), dtype=dtype, device=dev) for r in ranks]
    db = [torch.full((N, r), float("nan"), dtype=dtype, device=dev) for r in ranks]
    ds = torch.full((M, (max(ranks) + 15) // 16 * 16), float("nan"), dtype=dtype, device=dev)
    return dx, da, db, ds


def _both(dy, x, w, mask, a_list, b_list, routing_c, R, ranks):
    """Run lf_lora_bwd (with a torch workspace) and lf_lora_bwd_static; return both output sets."""
    from lorafusion_amd import _lib as L
    from lorafusion_amd.ops import hip_ops

    M, N = dy.shape
    K = x.shape[1]
    dev, dtype = dy.device, dy.dtype
    y, s = hip_ops.lora_forward(x, w, a_list, b_list, routing_c, R, mask, None)
    lib = L.lib()
    need = lib.lf_workspace_bytes(L.LF_OP_BWD, M, N, K, R, routing_c)
    assert 0 < need <= L.LF_STATIC_SCRATCH_BYTES
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    ref = _outputs(M, N, K, ranks, dev, dtype)
    rc = lib.lf_lora_bwd(L.ptr(dy), L.ptr(x), L.ptr(w), L.ptr(mask), L.ptr(s), L.ptr_array(a_list), L.ptr_array(b_list),
                         L.ptr(ref[0]), L.ptr_array(ref[1]), L.ptr_array(ref[2]), L.ptr(ref[3]), L.ptr(ws), need,
                         M, N, K, R, routing_c, L.dtype_id(dtype), L.stream_of(dy))
    assert rc == 0, lib.lf_strerror(rc)
    got = _outputs(M, N, K, ranks, dev, dtype)
    rc = lib.lf_lora_bwd_static(L.ptr(dy), L.ptr(x), L.ptr(w), L.ptr(mask), L.ptr(s), L.ptr_array(a_list),
                                L.ptr_array(b_list), L.ptr(got[0]), L.ptr_array(got[1]), L.ptr_array(got[2]),
                                L.ptr(got[3]), M, N, K, R, routing_c, L.dtype_id(dtype), L.stream_of(dy))
    assert rc == 0, lib.lf_strerror(rc)
    torch.cuda.synchronize()
    return ref, got


def _assert_same(ref, got, what):
    assert torch.equal(ref[0], got[0]), f"{what}: dX differs"
    for i, (r, g) in enumerate(zip(ref[1], got[1])):
        assert torch.equal(r, g), f"{what}: dA[{i}] differs"
    for i, (r, g) in enumerate(zip(ref[2], got[2])):
        assert torch.equal(r, g), f"{what}: dB[{i}] differs"
    assert torch.equal(ref[3], got[3]), f"{what}: dS differs"
    assert not torch.isnan(got[0].float()).any() and not torch.isnan(got[3].float()).any()


def test_static_scratch_backward_matches_workspace_backward():
    from lorafusion_amd import _lib as L
    from lorafusion_amd.ops import hip_ops
    from lorafusion_amd.ops.multi_lora import prepare_multi_lora_batch_info

    dev = "cuda"
    # first call: a packed batch of four adapters, 1664 rows
    seq, ranks, p_list, scales = [300, 520, 129, 600], [16, 32, 16, 8], [0.0, 0.05, 0.1, 0.1], [1.0, 2.0, 2.0, 4.0]
    K, N = 1024, 768
    d = multi_inputs(seq, K, N, ranks, p_list, seed=3)
    info = prepare_multi_lora_batch_info(seq, list(range(len(seq))), ranks, p_list, scales, 128)
    routing = hip_ops.MultiRouting(info.padded_seq_len_list, ranks, info.block_to_lookup_table, info.block_to_alpha,
                                   info.block_to_dropout_p, enable_dropout=info.enable_dropout)
    a_list = [a.to(dev) for a in d["a_list"]]
    b_list = [b.to(dev) for b in d["b_list"]]
    ref, got = _both(d["dy"].to(dev), d["x"].to(dev), d["w"].to(dev), d["mask"].to(dev), a_list, b_list, routing.c,
                     routing.R, ranks)
    _assert_same(ref, got, "multi-LoRA batch")

    # second call, smaller: one adapter, 200 rows (not a multiple of the row block), the same process
    # and the same scratch buffer, which still holds the first call's partial sums
    M2, K2, N2, r2 = 200, 512, 384, 16
    e = single_inputs(M2, K2, N2, r2, p=0.1, seed=5)
    rs = L.single_routing(r2, 2.0, 0.1)
    ref2, got2 = _both(e["dy"].to(dev), e["x"].to(dev), e["w"].to(dev), e["mask"].to(dev), [e["a"].to(dev)],
                       [e["b"].to(dev)], rs, 16, [r2])
    _assert_same(ref2, got2, "single adapter, smaller call")


def test_static_scratch_rejects_oversized_call():
    from lorafusion_amd import _lib as L

    dev = "cuda"
    lib = L.lib()
    # rank 64 at N = 28672: the dB partial sums alone exceed the static buffer; nothing may be launched,
    # so the (tiny, wrong-sized) buffers passed here are never touched
    M, N, K, R = 8192, 28672, 8192, 64
    rs = L.single_routing(64, 1.0, 0.0)
    assert lib.lf_workspace_bytes(L.LF_OP_BWD, M, N, K, R, rs) > L.LF_STATIC_SCRATCH_BYTES
    t = torch.zeros(16, dtype=torch.bfloat16, device=dev)
    arr = L.ptr_array([t])
    rc = lib.lf_lora_bwd_static(L.ptr(t), L.ptr(t), L.ptr(t), None, L.ptr(t), arr, arr, L.ptr(t), arr, arr, L.ptr(t),
                                M, N, K, R, rs, L.LF_BF16, L.stream_of(t))
    assert rc == L.LF_ESTATIC
    assert b"static" in lib.lf_strerror(rc)
    torch.cuda.synchronize()
    assert float(t.float().abs().sum()) == 0.0
    # shapes the rank-r passes do not tile are refused before anything is planned or launched
    for n, k, r in ((64, 256, 16), (256, 32, 16), (256, 256, 24)):
        rc = lib.lf_lora_bwd_static(L.ptr(t), L.ptr(t), L.ptr(t), None, L.ptr(t), arr, arr, L.ptr(t), arr, arr, L.ptr(t),
                                    256, n, k, r, L.single_routing(16, 1.0, 0.0), L.LF_BF16, L.stream_of(t))
        assert rc == L.LF_ESHAPE, (n, k, r, rc)
    torch.cuda.synchronize()
    assert float(t.float().abs().sum()) == 0.0
