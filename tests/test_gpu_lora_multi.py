"""GPU parity: packed multi-adapter LoRA linear vs the CPU oracle; routing is bit-exact.

Floating-point tolerance as in test_gpu_lora_single.py (rtol 1e-2, atol 1e-2*rms, fp32-accumulated
oracle).  Integer checks: the device routing table equals the oracle's table and the rows that
receive a LoRA term are exactly the table's valid rows.
"""

import numpy as np
import pytest
import torch

from oracle import lora_ref, routing
from tests.util import lognormal_segments, multi_inputs

pytestmark = pytest.mark.gpu

RTOL = 1e-2


def _close(actual, expected, what):
    ok, rel, excess = lora_ref.check_close(actual.detach().float().cpu(), expected, rtol=RTOL)
    assert ok, f"{what}: max|err|/max|e| = {rel:.3e}, worst excess over bound {excess:.3e}"


def _run(seq_len_list, K, N, ranks, p_list, scale_list, seed=0, bias=False, explicit_dtype=torch.float32):
    from lorafusion_amd.ops.multi_lora import fused_linear_multi_lora, prepare_multi_lora_batch_info

    d = multi_inputs(seq_len_list, K, N, ranks, p_list, seed=seed, bias=bias)
    info = prepare_multi_lora_batch_info(seq_len_list, list(range(len(seq_len_list))), ranks, p_list, scale_list,
                                         128, output_dtype=explicit_dtype)
    exp_padded, exp_lookup, *_ = routing.block_tables(seq_len_list, ranks, p_list, scale_list, 128)
    assert info.padded_seq_len_list == exp_padded == d["padded"]
    assert np.array_equal(info.block_to_lookup_table.cpu().numpy(), exp_lookup)

    dev = "cuda"
    x = d["x"].to(dev).requires_grad_(True)
    a_list = [a.to(dev).requires_grad_(True) for a in d["a_list"]]
    b_list = [b.to(dev).requires_grad_(True) for b in d["b_list"]]
    mask = d["mask"].to(dev) if d["mask"] is not None else None
    bias_t = d["bias"].to(dev) if bias else None
    y = fused_linear_multi_lora(
        x.unsqueeze(0), d["w"].to(dev), lora_a_list=a_list, lora_b_list=b_list, seq_len_list=seq_len_list,
        padded_seq_len_list=info.padded_seq_len_list, block_to_lookup_table=info.block_to_lookup_table,
        block_to_dropout_p=info.block_to_dropout_p, block_to_alpha=info.block_to_alpha,
        enable_dropout=info.enable_dropout, same_dropout_p_value=info.same_dropout_p_value, max_r=info.max_r,
        linear_bias=bias_t, dropout_mask=mask,
    )
    assert y.shape == (1, sum(exp_padded), N)
    y.backward(d["dy"].to(dev).unsqueeze(0))
    torch.cuda.synchronize()

    ye, _ = lora_ref.linear_multi_lora_fwd_fp32(d["x"], d["w"], d["a_list"], d["b_list"], seq_len_list, exp_padded,
                                                scale_list, p_list, d["mask"], d["bias"])
    dxe, dae, dbe, _ = lora_ref.linear_multi_lora_bwd_fp32(d["dy"], d["x"], d["w"], d["a_list"], d["b_list"],
                                                           seq_len_list, exp_padded, scale_list, p_list, d["mask"])
    _close(y[0], ye, "y")
    _close(x.grad, dxe, "dx")
    for i in range(len(ranks)):
        _close(a_list[i].grad, dae[i], f"da[{i}]")
        _close(b_list[i].grad, dbe[i], f"db[{i}]")
    return d, info, y


@pytest.mark.parametrize(
    "seq,ranks,p_list,scales",
    [
        ([256, 128], [16, 16], [0.1, 0.1], [2.0, 2.0]),
        ([129, 130, 128], [16, 16, 16], [0.1, 0.1, 0.1], [1.0, 2.0, 4.0]),          # the reference's worked example
        ([100, 300, 64, 257], [16, 16, 16, 16], [0.0, 0.05, 0.1, 0.1], [1.0, 2.0, 2.0, 4.0]),  # heterogeneous p
        ([200, 50], [16, 64], [0.0, 0.0], [2.0, 0.5]),                               # mixed ranks, no dropout
        ([1, 127, 128, 129, 5, 300, 77, 64], [16, 32, 16, 8, 64, 16, 16, 32], [0.1] * 8, [1.0] * 8),  # 8 adapters
        ([640], [16], [0.1], [2.0]),                                                 # one segment through the multi path
        ([200, 130, 300], [16, 48, 8], [0.1, 0.0, 0.25], [1.0, 2.0, 0.5]),          # S/dS of 48 columns: not a power of two
        ([150, 260], [96, 40], [0.1, 0.1], [0.5, 2.0]),                              # 96 columns; rank 40 inside them
    ],
)
def test_multi_parity(seq, ranks, p_list, scales):
    _run(seq, 512, 384, ranks, p_list, scales)


def test_multi_bias_and_bf16_tables():
    """bias; per-block alpha / p handed over as bf16 tensors (exactly representable values)."""
    _run([256, 130, 384], 384, 512, [16, 16, 32], [0.125, 0.0, 0.25], [2.0, 1.0, 0.5], bias=True,
         explicit_dtype=torch.bfloat16)


def test_multi_config1_shape():
    """The headline multi-adapter configuration: 4 adapters r=16, scales {16,32,32,64}/16, p {0,.05,.1,.1}, lognormal
    segments packed to 8192 tokens, K=N=4096."""
    seq = lognormal_segments(8192, 4, seed=0)
    assert sum(seq) == 8192
    _run(seq, 4096, 4096, [16] * 4, [0.0, 0.05, 0.1, 0.1], [1.0, 2.0, 2.0, 4.0])


def test_rows_written_exact():
    """The rows whose output differs from the base GEMM are exactly the valid rows of the table;
    padded rows equal the base GEMM bit for bit."""
    from lorafusion_amd.ops import hip_ops
    from lorafusion_amd.ops.multi_lora import fused_linear_multi_lora, prepare_multi_lora_batch_info

    seq, ranks, p_list, scales = [100, 300, 64], [16, 16, 16], [0.0, 0.0, 0.0], [2.0, 2.0, 2.0]
    d = multi_inputs(seq, 256, 256, ranks, p_list, seed=7)
    # large B so every valid row moves by far more than a rounding step
    b_list = [(torch.ones_like(b) * 0.5).cuda() for b in d["b_list"]]
    info = prepare_multi_lora_batch_info(seq, [0, 1, 2], ranks, p_list, scales, 128)
    x, w = d["x"].cuda(), d["w"].cuda()
    y = fused_linear_multi_lora(
        x.unsqueeze(0), w, lora_a_list=[a.cuda() for a in d["a_list"]], lora_b_list=b_list, seq_len_list=seq,
        padded_seq_len_list=info.padded_seq_len_list, block_to_lookup_table=info.block_to_lookup_table,
        block_to_dropout_p=info.block_to_dropout_p, block_to_alpha=info.block_to_alpha, enable_dropout=False,
        same_dropout_p_value=None, max_r=16)[0]
    base = hip_ops.gemm(x, w)
    changed = (y != base).any(dim=1).cpu().numpy()
    expect = np.zeros(sum(info.padded_seq_len_list), dtype=bool)
    expect[routing.rows_written(info.block_to_lookup_table.cpu().numpy(), 128)] = True
    assert np.array_equal(changed, expect)


def test_one_adapter_equals_single_path():
    from lorafusion_amd.ops.lora_v1 import fused_linear_lora
    from lorafusion_amd.ops.multi_lora import fused_linear_multi_lora, prepare_multi_lora_batch_info

    seq = [384]
    d = multi_inputs(seq, 256, 256, [16], [0.1], seed=11)
    # fp32 tables: with the default bf16 storage p = 0.1 becomes 0.10009765625 and 1/(1-p) differs in the last bits
    info = prepare_multi_lora_batch_info(seq, [0], [16], [0.1], [2.0], 128, output_dtype=torch.float32)
    x, w, a, b, mask = d["x"].cuda(), d["w"].cuda(), d["a_list"][0].cuda(), d["b_list"][0].cuda(), d["mask"].cuda()
    ym = fused_linear_multi_lora(
        x.unsqueeze(0), w, lora_a_list=[a], lora_b_list=[b], seq_len_list=seq,
        padded_seq_len_list=info.padded_seq_len_list, block_to_lookup_table=info.block_to_lookup_table,
        block_to_dropout_p=info.block_to_dropout_p, block_to_alpha=info.block_to_alpha, enable_dropout=True,
        same_dropout_p_value=0.1, max_r=16, dropout_mask=mask)[0]
    ys = fused_linear_lora(x, w, a, b, 2.0, dropout_p=0.1, dropout_mask=mask)
    assert torch.equal(ym, ys)


def test_adapter_in_two_segments_accumulates_through_autograd():
    """The C ABI writes one dA / dB per segment.  At the autograd layer an adapter whose tokens sit in two separate
    row ranges is passed once per range: each occurrence gets its segment's gradient and autograd adds them, which
    is the gradient of the adapter over both ranges (oracle: the two segments' gradients summed)."""
    from lorafusion_amd.ops.multi_lora import fused_linear_multi_lora, prepare_multi_lora_batch_info

    seq, ranks, p_list, scales = [200, 150, 90], [16, 16, 16], [0.1, 0.0, 0.1], [2.0, 0.5, 2.0]
    d = multi_inputs(seq, 256, 384, ranks, p_list, seed=11)
    d["a_list"][2], d["b_list"][2] = d["a_list"][0], d["b_list"][0]      # segment 2 belongs to adapter 0 again
    info = prepare_multi_lora_batch_info(seq, [0, 1, 0], ranks, p_list, scales, 128, output_dtype=torch.float32)
    dev = "cuda"
    x = d["x"].to(dev).requires_grad_(True)
    a0, a1 = (d["a_list"][i].to(dev).requires_grad_(True) for i in (0, 1))
    b0, b1 = (d["b_list"][i].to(dev).requires_grad_(True) for i in (0, 1))
    y = fused_linear_multi_lora(
        x.unsqueeze(0), d["w"].to(dev), lora_a_list=[a0, a1, a0], lora_b_list=[b0, b1, b0], seq_len_list=seq,
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
    _close(a0.grad, dae[0] + dae[2], "da of the adapter with two segments")
    _close(b0.grad, dbe[0] + dbe[2], "db of the adapter with two segments")
    _close(a1.grad, dae[1], "da[1]")
    _close(b1.grad, dbe[1], "db[1]")


def test_multi_errors():
    from lorafusion_amd.ops.multi_lora import fused_linear_multi_lora, prepare_multi_lora_batch_info

    seq = [128, 128]
    d = multi_inputs(seq, 256, 256, [16, 16], [0.0, 0.0])
    info = prepare_multi_lora_batch_info(seq, [0, 1], [16, 16], [0.0, 0.0], [1.0, 1.0], 128)
    kw = dict(seq_len_list=seq, padded_seq_len_list=info.padded_seq_len_list,
              block_to_lookup_table=info.block_to_lookup_table, block_to_dropout_p=info.block_to_dropout_p,
              block_to_alpha=info.block_to_alpha, enable_dropout=False, same_dropout_p_value=0.0, max_r=16)
    a = [t.cuda() for t in d["a_list"]]
    b = [t.cuda() for t in d["b_list"]]
    with pytest.raises(ValueError):
        fused_linear_multi_lora(d["x"].cuda().unsqueeze(0), d["w"].cuda(), lora_a_list=[], lora_b_list=[], **kw)
    with pytest.raises(ValueError):
        fused_linear_multi_lora(d["x"].cuda().unsqueeze(0), d["w"].cuda(), lora_a_list=a, lora_b_list=b[:1], **kw)
    with pytest.raises(ValueError):  # batch size must be 1
        fused_linear_multi_lora(d["x"].cuda().reshape(2, 128, 256), d["w"].cuda(), lora_a_list=a, lora_b_list=b, **kw)
    with pytest.raises(ValueError):  # rows do not match the tables
        fused_linear_multi_lora(d["x"].cuda()[:128].unsqueeze(0), d["w"].cuda(), lora_a_list=a, lora_b_list=b, **kw)
