"""The multi-adapter kernel wrappers called the way the reference's own kernel tests call them
(lorafusion/ops/tests/test_fused_multi_lora_xw_sb.py:131-231, ..._dys_dyb.py:155-187, ..._dyw_dsa.py:157-257):
per-adapter tensor lists plus the block tables, compared with the oracle's per-segment arithmetic."""

from __future__ import annotations

import pytest
import torch

from oracle import dropout as odrop
from oracle import lora_ref
from tests.util import multi_inputs

pytestmark = pytest.mark.gpu


def _close(got, exp, name):
    ok, rel, excess = lora_ref.check_close(got.detach().float().cpu(), exp, rtol=1e-2)
    assert ok, f"{name}: rel {rel:.3e} excess {excess:.3e}"


def _setup():
    from lorafusion_amd.ops.multi_lora import prepare_multi_lora_batch_info

    seq, ranks, p_list, scales = [200, 128, 61], [16, 32, 16], [0.1, 0.0, 0.2], [2.0, 0.5, 1.0]
    K, N = 384, 512
    d = multi_inputs(seq, K, N, ranks, p_list, seed=13, bias=True)
    info = prepare_multi_lora_batch_info(seq, [0, 1, 2], ranks, p_list, scales, 128, output_dtype=torch.float32)
    return seq, ranks, p_list, scales, K, N, d, info


def test_xw_sb_dys_dyb_dyw_dsa_with_reference_signatures():
    from lorafusion_amd.ops.triton_ops.fused_multi_lora_dys_dyb import fused_multi_lora_dys_dyb
    from lorafusion_amd.ops.triton_ops.fused_multi_lora_dyw_dsa import fused_multi_lora_dyw_dsa
    from lorafusion_amd.ops.triton_ops.fused_multi_lora_xw_sb import construct_s_and_b_ptrs_list, fused_multi_lora_xw_sb

    seq, ranks, p_list, scales, K, N, d, info = _setup()
    padded = d["padded"]
    x, w, dy, mask = d["x"].cuda(), d["w"].cuda(), d["dy"].cuda(), d["mask"].cuda()
    # oracle pieces per segment
    _, s_or = lora_ref.linear_multi_lora_fwd_fp32(d["x"], d["w"], d["a_list"], d["b_list"], seq, padded, scales, p_list, d["mask"])
    ye, _ = lora_ref.linear_multi_lora_fwd_fp32(d["x"], d["w"], d["a_list"], d["b_list"], seq, padded, scales, p_list,
                                                d["mask"], bias=d["bias"])
    dxe, dae, dbe, dse = lora_ref.linear_multi_lora_bwd_fp32(d["dy"], d["x"], d["w"], d["a_list"], d["b_list"], seq, padded,
                                                             scales, p_list, d["mask"])
    # per-adapter S / dS with padded row counts, as lorafusion/ops/multi_lora.py hands them to the kernels
    raw_s, raw_ds = [], []
    for s_i, ds_i, pl, r in zip(s_or, dse, padded, ranks):
        t = torch.zeros(pl, r)
        t[: s_i.shape[0]] = s_i
        raw_s.append(t.to(torch.bfloat16).cuda())
        t = torch.zeros(pl, r)
        t[: ds_i.shape[0]] = ds_i
        raw_ds.append(t.to(torch.bfloat16).cuda())
    raw_b = [b.cuda() for b in d["b_list"]]
    raw_a = [a.cuda() for a in d["a_list"]]
    kw = dict(block_to_lookup_table=info.block_to_lookup_table, block_to_alpha=info.block_to_alpha, max_r=info.max_r,
              total_r=sum(ranks))

    y = fused_multi_lora_xw_sb(x, w, raw_s_list=raw_s, raw_b_list=raw_b, bias=d["bias"].cuda(), block_size_m=128, **kw)
    _close(y, ye, "y")
    s_ptrs, b_ptrs, _, _ = construct_s_and_b_ptrs_list(raw_s, raw_b, 128)
    y2 = fused_multi_lora_xw_sb(x, w, s_ptrs_list=s_ptrs, b_ptrs_list=b_ptrs, bias=d["bias"].cuda(), **kw)
    assert torch.equal(y, y2)

    db_list, ds_list = fused_multi_lora_dys_dyb(dy, info.block_to_lookup_table, info.block_to_alpha, info.max_r, sum(ranks),
                                                raw_s_list=raw_s, raw_b_list=raw_b)
    for i, (n, pl) in enumerate(zip(seq, padded)):
        assert ds_list[i].shape == (pl, ranks[i])
        _close(ds_list[i][:n], dse[i], f"ds[{i}]")
        assert not ds_list[i][n:].any(), "padded rows of dS must be zero"
        _close(db_list[i], dbe[i], f"db[{i}]")

    dx = fused_multi_lora_dyw_dsa(dy, w, raw_ds_list=raw_ds, raw_a_list=raw_a, block_to_dropout_p=info.block_to_dropout_p,
                                  block_to_lookup_table=info.block_to_lookup_table, max_r=info.max_r, enable_dropout=True,
                                  dropout_mask=mask)
    _close(dx, dxe, "dx")
    with pytest.raises(ValueError):
        fused_multi_lora_dyw_dsa(dy, w, raw_ds_list=raw_ds, raw_a_list=raw_a, block_to_dropout_p=info.block_to_dropout_p,
                                 block_to_lookup_table=info.block_to_lookup_table, max_r=info.max_r, enable_dropout=True)
    with pytest.raises(ValueError):
        fused_multi_lora_xw_sb(x, w, **kw)                                    # neither raw lists nor pointer lists
    with pytest.raises(ValueError):
        fused_multi_lora_xw_sb(x, w, raw_s_list=raw_s, raw_b_list=raw_b, block_size_m=64, **kw)


def test_blocked_seeded_dropout_matches_the_mask_oracle():
    from lorafusion_amd.ops.triton_ops.blocked_dropout import blocked_seeded_dropout

    M, K, bs, seed = 512, 256, 128, 4242
    p_blocks = [0.0, 0.25, 0.5, 0.1]
    g = torch.Generator().manual_seed(1)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    out, mask = blocked_seeded_dropout(x.cuda(), torch.tensor(p_blocks), bs, seed)
    import numpy as np

    want = odrop.keep_mask(M, K, np.repeat(np.asarray(p_blocks, dtype=np.float32), bs), seed)
    assert (mask.cpu().numpy().astype("uint8") == want).all()
    for b, p in enumerate(p_blocks):
        rows = slice(b * bs, (b + 1) * bs)
        exp = torch.where(mask[rows].cpu(), (x[rows].float() * (1.0 / (1.0 - p))).to(torch.bfloat16), torch.zeros((), dtype=torch.bfloat16))
        assert torch.equal(out[rows].cpu(), exp)
    out2, none = blocked_seeded_dropout(x.cuda(), torch.tensor(p_blocks), bs, seed, store_mask=False)
    assert none is None and torch.equal(out2, out)
    with pytest.raises(ValueError):
        blocked_seeded_dropout(x.cuda()[:100], torch.tensor(p_blocks), bs, seed)
