"""Pins the routing-table oracle and checks the product's vectorised table builder against it (bit-exact).

Anchors: the worked example in the reference's comments (multi_lora.py:377-379:
seq_len_list [129,130,128] -> padded [256,256,128], valid sizes [128,1,128,2,128]); invariants
(sum valid = sum seq_len, first_block = prefix sum of padded/block, ranks constant per segment);
the C restatement vs the Python one; hypothesis-generated ragged inputs.
"""

import numpy as np
import pytest
import torch
from hypothesis import given, settings, strategies as st

from oracle import nf4 as onf4
from oracle import routing
from tests.util import golden


def test_reference_worked_example():
    ex = golden("routing_worked_example.json")
    n = len(ex["seq_len_list"])
    padded, lookup, bp, ba, max_r, en, same = routing.block_tables(ex["seq_len_list"], [16] * n, [0.1] * n, [2.0] * n,
                                                                   ex["block_size_m"])
    assert padded == ex["padded_seq_len_list"]
    assert lookup[:, 1].tolist() == ex["valid_rows_per_block"]
    assert lookup[:, 2].tolist() == ex["first_block_per_block"]
    assert lookup[:, 0].tolist() == [16] * 5
    assert max_r == 16 and en and same == 0.1
    assert bp.tolist() == [0.1] * 5 and ba.tolist() == [2.0] * 5


@pytest.mark.parametrize("seq,block", [([1], 128), ([128], 128), ([127, 129], 128), ([64, 64, 64], 64),
                                       ([4096, 64, 1000, 1], 128), ([5, 7, 9], 4)])
def test_invariants_and_c_restatement(seq, block):
    ranks = [16 * (1 + i % 3) for i in range(len(seq))]
    ps = [0.05 * i for i in range(len(seq))]
    alphas = [1.0 + i for i in range(len(seq))]
    padded, lookup, bp, ba, max_r, en, same = routing.block_tables(seq, ranks, ps, alphas, block)
    assert all(p % block == 0 and 0 <= p - n < block for p, n in zip(padded, seq))
    assert int(lookup[:, 1].sum()) == sum(seq)
    first = np.concatenate(([0], np.cumsum(np.asarray(padded) // block)[:-1]))
    blk = 0
    for i, p in enumerate(padded):
        nb = p // block
        assert (lookup[blk:blk + nb, 2] == first[i]).all() and (lookup[blk:blk + nb, 0] == ranks[i]).all()
        assert (lookup[blk:blk + nb - 1, 1] == block).all() and lookup[blk + nb - 1, 1] == seq[i] - (nb - 1) * block
        assert (bp[blk:blk + nb] == ps[i]).all() and (ba[blk:blk + nb] == alphas[i]).all()
        blk += nb
    assert blk == lookup.shape[0] and max_r == max(ranks)
    assert np.array_equal(onf4.routing_table_c(seq, ranks, block), lookup)
    rows = routing.rows_written(lookup, block)
    assert len(rows) == sum(seq) and len(set(rows.tolist())) == len(rows)


@settings(max_examples=60, deadline=None)
@given(st.lists(st.integers(min_value=1, max_value=700), min_size=1, max_size=9), st.sampled_from([16, 64, 128, 256]))
def test_product_table_builder_bit_exact(seq, block):
    from lorafusion_amd.ops.multi_lora import build_block_tables, prepare_multi_lora_batch_info

    ranks = [8 * (1 + (n % 4)) for n in seq]
    ps = [(n % 5) * 0.05 for n in seq]
    alphas = [0.5 * (1 + n % 7) for n in seq]
    exp_padded, exp_lookup, exp_p, exp_a, max_r, en, same = routing.block_tables(seq, ranks, ps, alphas, block)
    padded, lookup, bp, ba = build_block_tables(seq, ranks, ps, alphas, block)
    assert padded == exp_padded
    assert lookup.dtype == np.int32 and np.array_equal(lookup, exp_lookup)
    assert np.array_equal(bp, exp_p) and np.array_equal(ba, exp_a)
    info = prepare_multi_lora_batch_info(seq, list(range(len(seq))), ranks, ps, alphas, block, output_dtype=torch.float32)
    assert np.array_equal(info.block_to_lookup_table.cpu().numpy(), exp_lookup)
    assert info.block_to_lookup_table.dtype == torch.int32
    assert info.max_r == max_r and info.enable_dropout == en and info.same_dropout_p_value == same
    assert info.block_to_alpha.dtype == torch.float32
    assert np.array_equal(info.block_to_alpha.cpu().numpy(), exp_a.astype(np.float32))
    # the default storage type is the reference's (multi_lora.py:355)
    info16 = prepare_multi_lora_batch_info(seq, list(range(len(seq))), ranks, ps, alphas, block)
    assert info16.block_to_alpha.dtype == info16.block_to_dropout_p.dtype == torch.bfloat16
    assert torch.equal(info16.block_to_alpha.cpu(), torch.from_numpy(exp_a).to(torch.bfloat16))
    assert info.num_active_adapters == len(seq)


def test_product_table_builder_errors_and_bf16_option():
    from lorafusion_amd.ops.multi_lora import prepare_multi_lora_batch_info

    with pytest.raises(ValueError):
        prepare_multi_lora_batch_info([], [], [], [], [], 128)
    with pytest.raises(ValueError):
        prepare_multi_lora_batch_info([0, 5], [0, 1], [16, 16], [0.0, 0.0], [1.0, 1.0], 128)
    with pytest.raises(ValueError):
        prepare_multi_lora_batch_info([5], [0], [16, 16], [0.0], [1.0], 128)
    info = prepare_multi_lora_batch_info([100, 200], [3, 1], [16, 16], [0.1, 0.05], [2.0, 4.0], 128,
                                         output_dtype=torch.bfloat16)
    # the reference's bf16 storage of p (multi_lora.py:393-394): 0.1 -> 0.10009765625
    assert info.block_to_dropout_p.dtype == torch.bfloat16
    assert float(info.block_to_dropout_p[0]) == 0.10009765625
    assert info.lora_idx_list == [3, 1]


def test_batch_info_from_micro_batch_descriptor():
    """The scheduler's micro-batch descriptor (duck-typed) drives the routing tables:
    lorafusion/train/training_utils.py:1304-1334 restated."""
    from types import SimpleNamespace

    import torch

    from lorafusion_amd.ops.multi_lora import batch_info_from_micro_batch

    tokens = {3: 129, 0: 130, 7: 128}
    mb = SimpleNamespace(
        adapter_group_info=set(tokens), adapter_num_tokens_pairs=tokens,
        padded_adapter_num_tokens_pairs={a: ((n - 1) // 128 + 1) * 128 for a, n in tokens.items()},
        adapter_padding_multiple=128, is_empty_marker=False)
    cfgs = {a: SimpleNamespace(r=16 * (1 + a % 2), lora_dropout=0.05 * (a % 3), lora_alpha=16.0 + a) for a in tokens}
    info = batch_info_from_micro_batch(mb, cfgs, output_dtype=torch.float32)
    assert info.lora_idx_list == [0, 3, 7] and info.seq_len_list == [130, 129, 128]
    padded, lookup, block_p, block_alpha, *_ = routing.block_tables([130, 129, 128], [16, 32, 32], [0.0, 0.0, 0.05],
                                                                    [16.0, 19.0, 23.0], 128)
    assert info.padded_seq_len_list == padded == [256, 256, 128]
    assert np.array_equal(info.block_to_lookup_table.cpu().numpy(), lookup)
    assert np.allclose(info.block_to_dropout_p.cpu().numpy(), block_p) and np.allclose(info.block_to_alpha.cpu().numpy(), block_alpha)
    assert info.micro_batch_info is mb and info.max_r == 32
    # a descriptor padded to another multiple cannot drive 128-row kernels
    mb.adapter_padding_multiple = 64
    with pytest.raises(ValueError):
        batch_info_from_micro_batch(mb, cfgs)
    with pytest.raises(ValueError):
        batch_info_from_micro_batch(SimpleNamespace(is_empty_marker=True), cfgs)
