"""Multi-LoRA per-block routing tables (test infrastructure).

Restates /root/reference/lorafusion/ops/multi_lora.py:369-435: each adapter's token
segment is padded up to a multiple of ``block_size_m``; for every ``block_size_m``-row
block the table holds ``(rank, valid_rows, first_block_of_segment)``.  Plain Python
loops on purpose -- this is the checker for the vectorised product code.
"""

from __future__ import annotations

import numpy as np


def padded_lengths(seq_len_list, block_size_m):
    """multi_lora.py:369-371: round each segment up to a multiple of block_size_m."""
    return [((n - 1) // block_size_m + 1) * block_size_m for n in seq_len_list]


def block_tables(seq_len_list, lora_rank_list, dropout_p_list, alpha_list, block_size_m):
    """multi_lora.py:380-425.

    Returns (padded_seq_len_list, lookup int32 [nb,3], block_p float64 [nb],
    block_alpha float64 [nb], max_r, enable_dropout, same_dropout_p_value).
    The reference stores p / alpha per block in bf16 (multi_lora.py:393-394); the values
    are returned unrounded here and the caller rounds when it wants that behaviour.
    """
    padded = padded_lengths(seq_len_list, block_size_m)
    total_blocks = sum(padded) // block_size_m
    lookup = np.zeros((total_blocks, 3), dtype=np.int32)
    block_p = np.zeros(total_blocks, dtype=np.float64)
    block_alpha = np.zeros(total_blocks, dtype=np.float64)
    block_idx = 0
    for seq_idx, (seq_len, rank, p, alpha) in enumerate(
        zip(seq_len_list, lora_rank_list, dropout_p_list, alpha_list, strict=True)
    ):
        nblk = padded[seq_idx] // block_size_m
        start_m = block_idx
        for i in range(nblk):
            lookup[block_idx, 0] = rank
            lookup[block_idx, 1] = min(block_size_m, seq_len - i * block_size_m)
            lookup[block_idx, 2] = start_m
            block_p[block_idx] = p
            block_alpha[block_idx] = alpha
            block_idx += 1
    if block_idx != total_blocks:
        raise ValueError(f"Expected {total_blocks} blocks, but filled {block_idx}")
    max_r = max(lora_rank_list)
    enable_dropout = any(p > 0 for p in dropout_p_list)
    same = all(p == dropout_p_list[0] for p in dropout_p_list)
    return padded, lookup, block_p, block_alpha, max_r, enable_dropout, (dropout_p_list[0] if same else None)


def rows_written(lookup, block_size_m):
    """Row indices that carry a LoRA term (the per-block walk of
    lorafusion/ops/tests/test_fused_multi_lora_xw_sb.py:206-229)."""
    rows = []
    for blk in range(lookup.shape[0]):
        rows.extend(range(blk * block_size_m, blk * block_size_m + int(lookup[blk, 1])))
    return np.asarray(rows, dtype=np.int64)
