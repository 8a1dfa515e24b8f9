"""GPU parity of the split contraction: launches with few tiles and a long reduction (left-over rows of a packed
batch, short batches) cut K into slices, keep fp32 partial tiles in the caller's workspace and add them in a
second kernel.  Checked against the CPU oracle with the tolerance of test_gpu_lora_single.py, and against the same
product through the entry points without a workspace, which never split (fp32 sums in another order: equal to
within one 16-bit step of the result's magnitude).
"""

import pytest
import torch

from oracle import lora_ref
from tests.util import multi_inputs, single_inputs

pytestmark = pytest.mark.gpu

RTOL = 1e-2


def _close(actual, expected, what):
    ok, rel, excess = lora_ref.check_close(actual.detach().float().cpu(), expected, rtol=RTOL)
    assert ok, f"{what}: max|err|/max|e| = {rel:.3e}, worst excess over bound {excess:.3e}"


def _split_bytes(op, M, N, K, R, routing):
    from lorafusion_amd import _lib as L

    return L.lib().lf_workspace_bytes(op, M, N, K, R, routing)


@pytest.mark.parametrize("M,K,N,r,p,dtype,bias,sized", [
    (128, 8192, 256, 16, 0.1, torch.bfloat16, False, "fwd"),     # Y over K = 8192 in five slices of 128x64 tiles
    (128, 4096, 8192, 16, 0.1, torch.bfloat16, False, "bwd"),    # dX [128, 4096] over N = 8192 in four
    (200, 6144, 2048, 32, 0.1, torch.bfloat16, True, "fwd"),     # ragged rows, bias added by the second kernel
    (64, 8192, 384, 16, 0.0, torch.float16, True, "fwd"),        # fp16, no dropout
    (300, 12288, 512, 64, 0.2, torch.bfloat16, False, "fwd"),    # more than 256 rows: eight-wave 256x256 tiles, rank 64
    (384, 512, 12288, 16, 0.1, torch.bfloat16, False, None),     # the same for dX (its slices fit the rank-r passes' bytes)
    (1, 8192, 128, 16, 0.1, torch.bfloat16, False, "fwd"),       # a single token
])
def test_single_adapter_split(M, K, N, r, p, dtype, bias, sized):
    from lorafusion_amd import _lib as L
    from lorafusion_amd.ops import hip_ops
    from lorafusion_amd.ops.lora_v1 import fused_linear_lora

    routing = L.single_routing(r, 2.0, p)
    R = L.round_rank(r)
    # the size query shows the split where its partial tiles are the largest use of the workspace
    if sized == "fwd":
        assert _split_bytes(L.LF_OP_FWD, M, N, K, R, routing) > _split_bytes(L.LF_OP_XA, M, N, K, R, routing)
    if sized == "bwd":
        rank_r = max(_split_bytes(L.LF_OP_DYS_DYB, M, N, K, R, routing), _split_bytes(L.LF_OP_DA, M, N, K, R, routing))
        assert _split_bytes(L.LF_OP_BWD, M, N, K, R, routing) > rank_r
    d = single_inputs(M, K, N, r, p=p, seed=3, dtype=dtype, bias=bias)
    dev = "cuda"
    x = d["x"].to(dev).requires_grad_(True)
    a = d["a"].to(dev).requires_grad_(True)
    b = d["b"].to(dev).requires_grad_(True)
    w = d["w"].to(dev)
    mask = d["mask"].to(dev) if d["mask"] is not None else None
    bias_t = d["bias"].to(dev) if bias else None
    y = fused_linear_lora(x, w, a, b, 2.0, dropout_p=p, linear_bias=bias_t, dropout_mask=mask)
    y.backward(d["dy"].to(dev))
    torch.cuda.synchronize()
    ye, se = lora_ref.linear_lora_fwd_fp32(d["x"], d["w"], d["a"], d["b"], 2.0, d["mask"], p, d["bias"])
    dxe, dae, dbe, _ = lora_ref.linear_lora_bwd_fp32(d["dy"], d["x"], d["w"], d["a"], d["b"], 2.0, d["mask"], p)
    _close(y, ye, "y")
    _close(x.grad, dxe, "dx")
    _close(a.grad, dae, "da")
    _close(b.grad, dbe, "db")

    # the same forward product through the entry point without a workspace (one launch, no split)
    s, _, _ = hip_ops.fused_dropout_matmul(x.detach(), a.detach(), dropout_p=p, dropout_mask=mask) if p > 0 else \
        hip_ops.fused_dropout_matmul(x.detach(), a.detach(), dropout_p=0.0)
    y1 = hip_ops.fused_lora_xw_sb(x.detach(), w, s, b.detach(), 2.0, bias=bias_t)
    step = float(y1.float().abs().max()) * 2.0 ** (-7 if dtype == torch.bfloat16 else -10)
    assert float((y.detach().float() - y1.float()).abs().max()) <= step


def test_left_over_rows_of_a_packed_batch():
    """Two adapters, 256 + 128 padded rows: the 128 left-over rows are a launch of their own with a split contraction
    (K = 4096 forward, N = 4096 backward)."""
    from lorafusion_amd.ops.multi_lora import fused_linear_multi_lora, prepare_multi_lora_batch_info

    seq, ranks, p_list, scales = [250, 100], [16, 32], [0.1, 0.05], [2.0, 0.5]
    K, N = 4096, 4096
    d = multi_inputs(seq, K, N, ranks, p_list, seed=5)
    info = prepare_multi_lora_batch_info(seq, [0, 1], ranks, p_list, scales, 128, output_dtype=torch.float32)
    dev = "cuda"
    x = d["x"].to(dev).requires_grad_(True)
    a_list = [a.to(dev).requires_grad_(True) for a in d["a_list"]]
    b_list = [b.to(dev).requires_grad_(True) for b in d["b_list"]]
    y = fused_linear_multi_lora(
        x.unsqueeze(0), d["w"].to(dev), lora_a_list=a_list, lora_b_list=b_list, seq_len_list=seq,
        padded_seq_len_list=info.padded_seq_len_list, block_to_lookup_table=info.block_to_lookup_table,
        block_to_dropout_p=info.block_to_dropout_p, block_to_alpha=info.block_to_alpha,
        enable_dropout=info.enable_dropout, same_dropout_p_value=info.same_dropout_p_value, max_r=info.max_r,
        dropout_mask=d["mask"].to(dev),
    )
    y.backward(d["dy"].to(dev).unsqueeze(0))
    torch.cuda.synchronize()
    ye, _ = lora_ref.linear_multi_lora_fwd_fp32(d["x"], d["w"], d["a_list"], d["b_list"], seq, d["padded"], scales, p_list,
                                                d["mask"], None)
    dxe, dae, dbe, _ = lora_ref.linear_multi_lora_bwd_fp32(d["dy"], d["x"], d["w"], d["a_list"], d["b_list"], seq,
                                                           d["padded"], scales, p_list, d["mask"])
    _close(y[0], ye, "y")
    _close(x.grad, dxe, "dx")
    for i in range(2):
        _close(a_list[i].grad, dae[i], f"da[{i}]")
        _close(b_list[i].grad, dbe[i], f"db[{i}]")
