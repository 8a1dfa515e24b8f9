"""GPU parity: the seeded keep-mask kernel against the CPU oracle, bit for bit."""

import ctypes

import numpy as np
import pytest
import torch

from oracle import dropout as od

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("M,K,p,seed", [
    (1, 16, 0.5, 0),
    (7, 48, 0.1, 1),
    (130, 256, 0.3, 123456),
    (512, 4096, 0.05, 2**40 + 17),       # seed above 32 bits: both key words
    (33, 1040, 0.999, 5),
    (64, 128, 0.0, 9),
])
def test_mask_bit_exact(M, K, p, seed):
    from lorafusion_amd.ops import hip_ops

    m = hip_ops.make_dropout_mask((M, K), p, seed, "cuda")
    assert m.dtype == torch.bool and m.shape == (M, K)
    assert np.array_equal(m.cpu().numpy().astype(np.uint8), od.keep_mask(M, K, p, seed))


def test_mask_counter_beyond_32_bits():
    """Element indices above 2^32 (64-bit index arithmetic in the kernel): a tall mask checked on its last rows."""
    from lorafusion_amd.ops import hip_ops

    M, K, p, seed = 270_000, 16_384, 0.25, 77     # 4.4e9 elements, 4.4 GB of mask
    m = hip_ops.make_dropout_mask((M, K), p, seed, "cuda")
    rows = [0, 1, 262_143, 262_144, 262_145, M - 1]  # element 2^32 starts row 262144
    got = m[torch.tensor(rows, device="cuda")].cpu().numpy().astype(np.uint8)
    thr = od.keep_threshold(p)
    for r, g in zip(rows, got):
        e0 = r * K
        exp = np.empty(K, dtype=np.uint8)
        for c in range(K // 8):
            ctr = (e0 >> 3) + c
            w = od.philox4x32_10([ctr & 0xFFFFFFFF, ctr >> 32, 0, 0], [seed & 0xFFFFFFFF, seed >> 32])
            draws = np.stack([w & 0xFFFF, w >> 16], axis=1).reshape(-1)    # low half first
            exp[8 * c:8 * c + 8] = draws >= thr
        assert np.array_equal(g, exp), f"row {r}"
    del m


def test_mask_per_block_p_matches_routing():
    """Packed multi-adapter batch: every 128-row block uses its own p (heterogeneous dropout)."""
    from lorafusion_amd.ops import hip_ops
    from lorafusion_amd.ops.multi_lora import prepare_multi_lora_batch_info

    seq, p_list = [100, 300, 64, 257], [0.0, 0.05, 0.1, 0.3]
    info = prepare_multi_lora_batch_info(seq, [0, 1, 2, 3], [16] * 4, p_list, [1.0] * 4, 128, output_dtype=torch.float32)
    routing = hip_ops.MultiRouting(info.padded_seq_len_list, [16] * 4, info.block_to_lookup_table, info.block_to_alpha,
                                   info.block_to_dropout_p)
    M, K, seed = sum(info.padded_seq_len_list), 512, 4242
    m = hip_ops.make_dropout_mask((M, K), None, seed, "cuda", routing=routing)
    row_p = np.repeat(info.block_to_dropout_p.float().cpu().numpy(), 128)
    assert np.array_equal(m.cpu().numpy().astype(np.uint8), od.keep_mask(M, K, row_p, seed))


def test_mask_through_the_c_abi_and_errors():
    from lorafusion_amd import _lib as L

    lib = L.lib()
    M, K = 32, 64
    out = torch.empty((M, K), dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    assert lib.lf_dropout_mask(out.data_ptr(), M, K, ctypes.c_float(0.5), None, ctypes.c_uint64(3), st) == 0
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), od.keep_mask(M, K, 0.5, 3))
    assert lib.lf_dropout_mask(out.data_ptr(), M, 72, ctypes.c_float(0.5), None, ctypes.c_uint64(3), st) == L.LF_ESHAPE
    assert lib.lf_dropout_mask(out.data_ptr(), M, K, ctypes.c_float(1.0), None, ctypes.c_uint64(3), st) == L.LF_EINVAL
    assert lib.lf_dropout_mask(None, M, K, ctypes.c_float(0.5), None, ctypes.c_uint64(3), st) == L.LF_EINVAL


def test_fused_ops_draw_their_mask_on_the_device():
    """dropout_p > 0 without an explicit mask: the op's output equals the op run with the oracle's mask."""
    from lorafusion_amd.ops.lora_v1 import fused_linear_lora
    from tests.util import single_inputs

    d = single_inputs(256, 512, 256, 16, p=0.0, seed=3)
    x, w, a, b = (d[k].cuda() for k in ("x", "w", "a", "b"))
    seed, p = 99, 0.2
    y = fused_linear_lora(x, w, a, b, 2.0, seed=seed, dropout_p=p)
    mask = torch.from_numpy(od.keep_mask(256, 512, p, seed)).bool().cuda()
    y_ref = fused_linear_lora(x, w, a, b, 2.0, dropout_p=p, dropout_mask=mask)
    assert torch.equal(y, y_ref)


@pytest.mark.parametrize("ranks", [[16, 16, 16, 16], [8, 64, 32, 128], [64, 48, 16, 64], [32, 8, 24, 32]])
def test_seeded_forward_draws_the_oracle_mask(ranks):
    """The rank-r forward kernel that draws its own mask writes exactly the oracle's bytes (per-block p,
    padded rows included) and produces the same S and Y, bit for bit, as the run fed that mask."""
    from lorafusion_amd.ops import hip_ops
    from lorafusion_amd.ops.multi_lora import prepare_multi_lora_batch_info
    from tests.util import multi_inputs

    seq, p_list, scales = [100, 300, 64, 257], [0.0, 0.05, 0.1, 0.3], [1.0, 2.0, 2.0, 4.0]
    K, N, seed = 512, 384, 31337
    d = multi_inputs(seq, K, N, ranks, p_list, seed=5)
    info = prepare_multi_lora_batch_info(seq, [0, 1, 2, 3], ranks, p_list, scales, 128, output_dtype=torch.float32)
    routing = hip_ops.MultiRouting(info.padded_seq_len_list, ranks, info.block_to_lookup_table, info.block_to_alpha,
                                   info.block_to_dropout_p)
    x, w = d["x"].cuda(), d["w"].cuda()
    a_list, b_list = [t.cuda() for t in d["a_list"]], [t.cuda() for t in d["b_list"]]
    y, s, mask = hip_ops.lora_forward_seeded(x, w, a_list, b_list, routing.c, routing.R, seed, None)
    M = x.shape[0]
    row_p = np.repeat(info.block_to_dropout_p.float().cpu().numpy(), 128)
    expect = od.keep_mask(M, K, row_p, seed)
    assert mask.dtype == torch.uint8 and tuple(mask.shape) == (M, K // 8)      # drawn masks come back bit-packed
    assert np.array_equal(mask.cpu().numpy(), np.packbits(expect, axis=1, bitorder="little"))
    assert np.array_equal(hip_ops.unpack_mask(mask).cpu().numpy().astype(np.uint8), expect)
    y1, s1, mask1 = hip_ops.lora_forward_seeded(x, w, a_list, b_list, routing.c, routing.R, seed, None, packed=False)
    assert np.array_equal(mask1.cpu().numpy().astype(np.uint8), expect) and torch.equal(s, s1) and torch.equal(y, y1)
    y2, s2 = hip_ops.lora_forward(x, w, a_list, b_list, routing.c, routing.R, torch.from_numpy(expect).bool().cuda(), None)
    assert torch.equal(s, s2) and torch.equal(y, y2)


def test_seeded_multi_op_backward_uses_the_drawn_mask():
    """fused_linear_multi_lora without an explicit mask: forward and backward agree with the oracle
    evaluated on the mask the kernel drew."""
    from lorafusion_amd.ops.multi_lora import fused_linear_multi_lora, prepare_multi_lora_batch_info
    from oracle import lora_ref
    from tests.util import multi_inputs

    seq, ranks, p_list, scales = [200, 130], [16, 32], [0.1, 0.25], [2.0, 1.0]
    K, N, seed = 256, 384, 77
    d = multi_inputs(seq, K, N, ranks, p_list, seed=2)
    info = prepare_multi_lora_batch_info(seq, [0, 1], ranks, p_list, scales, 128, output_dtype=torch.float32)
    x = d["x"].cuda().requires_grad_(True)
    a = [t.cuda().requires_grad_(True) for t in d["a_list"]]
    b = [t.cuda().requires_grad_(True) for t in d["b_list"]]
    y = fused_linear_multi_lora(
        x.unsqueeze(0), d["w"].cuda(), lora_a_list=a, lora_b_list=b, seq_len_list=seq,
        padded_seq_len_list=info.padded_seq_len_list, block_to_lookup_table=info.block_to_lookup_table,
        block_to_dropout_p=info.block_to_dropout_p, block_to_alpha=info.block_to_alpha, enable_dropout=True,
        same_dropout_p_value=None, max_r=32, seed=seed)
    y.backward(d["dy"].cuda().unsqueeze(0))
    M = x.shape[0]
    mask = torch.from_numpy(od.keep_mask(M, K, np.repeat(info.block_to_dropout_p.float().cpu().numpy(), 128), seed)).bool()
    ye, _ = lora_ref.linear_multi_lora_fwd_fp32(d["x"], d["w"], d["a_list"], d["b_list"], seq, d["padded"], scales, p_list, mask)
    dxe, dae, dbe, _ = lora_ref.linear_multi_lora_bwd_fp32(d["dy"], d["x"], d["w"], d["a_list"], d["b_list"], seq, d["padded"],
                                                           scales, p_list, mask)
    for got, exp, name in [(y[0], ye, "y"), (x.grad, dxe, "dx"), (a[0].grad, dae[0], "da0"), (b[1].grad, dbe[1], "db1")]:
        ok, rel, _ = lora_ref.check_close(got.detach().float().cpu(), exp, rtol=1e-2)
        assert ok, f"{name}: {rel:.3e}"
