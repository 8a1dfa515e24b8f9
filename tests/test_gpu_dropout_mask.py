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
    """Element indices above 2^32 (counter index above 2^30): a tall mask checked on its last rows."""
    from lorafusion_amd.ops import hip_ops

    M, K, p, seed = 270_000, 16_384, 0.25, 77     # 4.4e9 elements, 4.4 GB of mask
    m = hip_ops.make_dropout_mask((M, K), p, seed, "cuda")
    rows = [0, 1, 262_143, 262_144, 262_145, M - 1]  # element 2^32 starts row 262144
    got = m[torch.tensor(rows, device="cuda")].cpu().numpy().astype(np.uint8)
    thr = od.keep_threshold(p)
    for r, g in zip(rows, got):
        e0 = r * K
        exp = np.empty(K, dtype=np.uint8)
        for c in range(K // 4):
            ctr = (e0 >> 2) + c
            w = od.philox4x32_10([ctr & 0xFFFFFFFF, ctr >> 32, 0, 0], [seed & 0xFFFFFFFF, seed >> 32])
            exp[4 * c:4 * c + 4] = w >= thr
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
