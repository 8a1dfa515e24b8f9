"""Pins the LoRA oracle (oracle/lora_ref.py) without using its own formulas:

* forward vs brute-force Python loops over scalars on tiny inputs;
* closed-form gradients vs torch.autograd on an independently written forward, and vs central
  finite differences in fp64;
* special cases that reduce to a plain linear layer (B = 0, scale = 0, all-dropped mask) or
  to no dropout (p = 0 ignores the mask);
* segmented (multi-adapter) version vs the single-adapter one per segment, per-token brute
  force, permutation invariance across adapters, and padded rows = base GEMM only;
* the reference's tolerance helper quantum (utils/testing.py:160-161).
"""

import itertools

import numpy as np
import pytest
import torch

from oracle import lora_ref


def _rand(shape, g, scale=1.0, dtype=torch.float64):
    return (torch.randn(*shape, generator=g, dtype=torch.float64) * scale).to(dtype)


def _tiny(seed=0, M=5, K=6, N=4, r=3, p=0.25):
    g = torch.Generator().manual_seed(seed)
    x, w, a, b, dy = _rand((M, K), g), _rand((N, K), g), _rand((r, K), g), _rand((N, r), g), _rand((M, N), g)
    bias = _rand((N,), g)
    mask = torch.rand(M, K, generator=g) >= p
    return x, w, a, b, dy, bias, mask


def test_forward_bruteforce_scalar_loops():
    x, w, a, b, dy, bias, mask = _tiny()
    p, scale = 0.25, 1.7
    M, K = x.shape
    N, r = b.shape
    y = np.zeros((M, N))
    for m, n in itertools.product(range(M), range(N)):
        acc = float(bias[n])
        for k in range(K):
            acc += float(x[m, k]) * float(w[n, k])
        lora = 0.0
        for j in range(r):
            sj = 0.0
            for k in range(K):
                if bool(mask[m, k]):
                    sj += float(x[m, k]) / (1.0 - p) * float(a[j, k])
            lora += sj * float(b[n, j])
        y[m, n] = acc + scale * lora
    got, s = lora_ref.linear_lora_fwd_fp32(x, w, a, b, scale, mask, p, bias, acc_dtype=torch.float64)
    assert np.allclose(got.numpy(), y, rtol=1e-12, atol=1e-12)
    assert s.shape == (M, r)


def _independent_forward(x, w, a, b, scale, mask, p, bias=None):
    # written with einsum / masked_fill instead of the oracle's where/@ chain
    keep = mask.to(x.dtype) / (1.0 - p) if p > 0 else torch.ones_like(x)
    base = torch.einsum("mk,nk->mn", x, w)
    if bias is not None:
        base = base + bias[None, :]
    s = torch.einsum("mk,rk->mr", x * keep, a)
    return base + scale * torch.einsum("mr,nr->mn", s, b)


@pytest.mark.parametrize("p", [0.0, 0.25])
def test_backward_vs_autograd_and_finite_differences(p):
    x, w, a, b, dy, bias, mask = _tiny(seed=1, p=max(p, 0.25))
    scale = 0.6
    xg, ag, bg = (t.clone().requires_grad_(True) for t in (x, a, b))
    y = _independent_forward(xg, w, ag, bg, scale, mask, p, bias)
    y.backward(dy)
    dx, da, db, ds = lora_ref.linear_lora_bwd_fp32(dy, x, w, a, b, scale, mask, p, acc_dtype=torch.float64)
    assert torch.allclose(dx, xg.grad, rtol=1e-12, atol=1e-12)
    assert torch.allclose(da, ag.grad, rtol=1e-12, atol=1e-12)
    assert torch.allclose(db, bg.grad, rtol=1e-12, atol=1e-12)
    assert torch.allclose(ds, scale * dy @ b, rtol=1e-12, atol=1e-12)

    # central differences on a few entries of each gradient
    def loss(xx, aa, bb):
        yy, _ = lora_ref.linear_lora_fwd_fp32(xx, w, aa, bb, scale, mask, p, bias, acc_dtype=torch.float64)
        return float((yy * dy).sum())

    eps = 1e-6
    for (t, grad, which) in ((x, dx, 0), (a, da, 1), (b, db, 2)):
        for idx in [(0, 0), (1, 2), (t.shape[0] - 1, t.shape[1] - 1)]:
            tp, tm = t.clone(), t.clone()
            tp[idx] += eps
            tm[idx] -= eps
            args_p = [x, a, b]
            args_m = [x, a, b]
            args_p[which], args_m[which] = tp, tm
            fd = (loss(*args_p) - loss(*args_m)) / (2 * eps)
            assert abs(fd - float(grad[idx])) < 1e-6 * max(1.0, abs(fd))


def test_special_cases():
    x, w, a, b, dy, bias, mask = _tiny(seed=2)
    base = x @ w.T + bias
    y0, _ = lora_ref.linear_lora_fwd_fp32(x, w, a, torch.zeros_like(b), 2.0, mask, 0.25, bias, acc_dtype=torch.float64)
    assert torch.allclose(y0, base, atol=1e-13)                       # B = 0 (PEFT init) -> plain linear
    y1, _ = lora_ref.linear_lora_fwd_fp32(x, w, a, b, 0.0, mask, 0.25, bias, acc_dtype=torch.float64)
    assert torch.allclose(y1, base, atol=1e-13)                       # scale = 0
    none = torch.zeros_like(mask)
    y2, s2 = lora_ref.linear_lora_fwd_fp32(x, w, a, b, 2.0, none, 0.25, bias, acc_dtype=torch.float64)
    assert torch.allclose(y2, base, atol=1e-13) and float(s2.abs().max()) == 0.0   # everything dropped
    y3, _ = lora_ref.linear_lora_fwd_fp32(x, w, a, b, 2.0, mask, 0.0, bias, acc_dtype=torch.float64)
    y4, _ = lora_ref.linear_lora_fwd_fp32(x, w, a, b, 2.0, None, 0.0, bias, acc_dtype=torch.float64)
    assert torch.equal(y3, y4)                                        # p = 0 ignores the mask
    full = torch.ones_like(mask)
    y5, _ = lora_ref.linear_lora_fwd_fp32(x, w, a, b, 2.0, full, 0.5, None, acc_dtype=torch.float64)
    assert torch.allclose(y5, x @ w.T + 2.0 * ((2.0 * x) @ a.T @ b.T), atol=1e-12)  # keep-all scales by 1/(1-p)
    # rank-1 identity-like check: a = e_0, b = e_0 column -> y[:,0] gets scale * x[:,0]
    a1 = torch.zeros(1, x.shape[1], dtype=x.dtype); a1[0, 0] = 1
    b1 = torch.zeros(w.shape[0], 1, dtype=x.dtype); b1[0, 0] = 1
    y6, _ = lora_ref.linear_lora_fwd_fp32(x, torch.zeros_like(w), a1, b1, 3.0, None, 0.0, None, acc_dtype=torch.float64)
    assert torch.allclose(y6[:, 0], 3.0 * x[:, 0]) and float(y6[:, 1:].abs().max()) == 0.0


def _multi_case(seed=3):
    g = torch.Generator().manual_seed(seed)
    seq, block = [3, 5, 2], 4
    padded = [4, 8, 4]
    K, N = 6, 5
    ranks, scales, ps = [2, 3, 1], [0.5, 2.0, 1.5], [0.0, 0.25, 0.5]
    Mp = sum(padded)
    x, w, dy, bias = _rand((Mp, K), g), _rand((N, K), g), _rand((Mp, N), g), _rand((N,), g)
    a_list = [_rand((r, K), g) for r in ranks]
    b_list = [_rand((N, r), g) for r in ranks]
    mask = torch.rand(Mp, K, generator=g) >= 0.3
    return seq, padded, x, w, dy, bias, a_list, b_list, scales, ps, mask


def test_multi_equals_single_per_segment_and_padded_rows_are_base_only():
    seq, padded, x, w, dy, bias, a_list, b_list, scales, ps, mask = _multi_case()
    y, s_list = lora_ref.linear_multi_lora_fwd_fp32(x, w, a_list, b_list, seq, padded, scales, ps, mask, bias,
                                                    acc_dtype=torch.float64)
    dx, da_list, db_list, _ = lora_ref.linear_multi_lora_bwd_fp32(dy, x, w, a_list, b_list, seq, padded, scales, ps,
                                                                  mask, acc_dtype=torch.float64)
    base = x @ w.T + bias
    cur = 0
    for i, (n, pad) in enumerate(zip(seq, padded)):
        sl = slice(cur, cur + n)
        ys, _ = lora_ref.linear_lora_fwd_fp32(x[sl], w, a_list[i], b_list[i], scales[i], mask[sl], ps[i], bias,
                                              acc_dtype=torch.float64)
        dxs, das, dbs, _ = lora_ref.linear_lora_bwd_fp32(dy[sl], x[sl], w, a_list[i], b_list[i], scales[i], mask[sl],
                                                         ps[i], acc_dtype=torch.float64)
        assert torch.allclose(y[sl], ys, atol=1e-12)
        assert torch.allclose(dx[sl], dxs, atol=1e-12)
        assert torch.allclose(da_list[i], das, atol=1e-12) and torch.allclose(db_list[i], dbs, atol=1e-12)
        pad_sl = slice(cur + n, cur + pad)                      # lora_torch_ref.py:116-118: cursor += padded length
        assert torch.equal(y[pad_sl], base[pad_sl])
        assert torch.allclose(dx[pad_sl], dy[pad_sl] @ w, atol=1e-13)
        cur += pad


def test_multi_per_token_bruteforce_and_autograd():
    seq, padded, x, w, dy, bias, a_list, b_list, scales, ps, mask = _multi_case(seed=4)
    y, _ = lora_ref.linear_multi_lora_fwd_fp32(x, w, a_list, b_list, seq, padded, scales, ps, mask, bias,
                                               acc_dtype=torch.float64)
    owner = []
    for i, (n, pad) in enumerate(zip(seq, padded)):
        owner += [i] * n + [-1] * (pad - n)
    for m, i in enumerate(owner):
        row = x[m] @ w.T + bias
        if i >= 0:
            xt = torch.where(mask[m], x[m] / (1 - ps[i]), torch.zeros((), dtype=x.dtype)) if ps[i] > 0 else x[m]
            row = row + scales[i] * (b_list[i] @ (a_list[i] @ xt))
        assert torch.allclose(y[m], row, atol=1e-12)
    # autograd through the op-by-op variant (the CPU timing baseline) agrees with the closed forms
    xg = x.clone().requires_grad_(True)
    ag = [a.clone().requires_grad_(True) for a in a_list]
    bg = [b.clone().requires_grad_(True) for b in b_list]
    yo = lora_ref.linear_multi_lora_bf16_opbyop(xg, w, ag, bg, seq, padded, scales, ps, mask, bias)
    assert torch.allclose(yo, y, atol=1e-12)
    yo.backward(dy)
    dx, da_list, db_list, _ = lora_ref.linear_multi_lora_bwd_fp32(dy, x, w, a_list, b_list, seq, padded, scales, ps,
                                                                  mask, acc_dtype=torch.float64)
    assert torch.allclose(xg.grad, dx, atol=1e-12)
    for i in range(3):
        assert torch.allclose(ag[i].grad, da_list[i], atol=1e-12) and torch.allclose(bg[i].grad, db_list[i], atol=1e-12)


def test_multi_permutation_invariance():
    seq, padded, x, w, dy, bias, a_list, b_list, scales, ps, mask = _multi_case(seed=5)
    y, _ = lora_ref.linear_multi_lora_fwd_fp32(x, w, a_list, b_list, seq, padded, scales, ps, mask, bias,
                                               acc_dtype=torch.float64)
    perm = [2, 0, 1]
    starts = np.concatenate(([0], np.cumsum(padded)[:-1]))
    rows = torch.cat([torch.arange(starts[i], starts[i] + padded[i]) for i in perm])
    y2, _ = lora_ref.linear_multi_lora_fwd_fp32(
        x[rows], w, [a_list[i] for i in perm], [b_list[i] for i in perm], [seq[i] for i in perm],
        [padded[i] for i in perm], [scales[i] for i in perm], [ps[i] for i in perm], mask[rows], bias,
        acc_dtype=torch.float64)
    assert torch.allclose(y2, y[rows], atol=1e-12)


def test_opbyop_single_matches_fp32_within_bf16_error():
    from tests.util import single_inputs

    d = single_inputs(64, 128, 96, 16, p=0.1, seed=0)
    y32, _ = lora_ref.linear_lora_fwd_fp32(d["x"], d["w"], d["a"], d["b"], 2.0, d["mask"], 0.1)
    y16 = lora_ref.linear_lora_bf16_opbyop(d["x"], d["w"], d["a"], d["b"], 2.0, d["mask"], 0.1)
    ok, rel, _ = lora_ref.check_close(y16.float(), y32, rtol=2e-2)
    assert ok, rel


def test_tolerance_helpers():
    e = torch.tensor([1.0, -2.0, 100.0])
    # bf16 spacing near 100 is 0.5: (100 + 0.3) - 0.3 rounds by at most that much
    q = lora_ref.bf16_quantum(e)
    assert 0.0 <= q <= 2.5 * 0.5
    ok, rel, _ = lora_ref.check_close(e * 1.005, e, rtol=1e-2)
    assert ok and abs(rel - 0.005) < 1e-6
    ok, _, _ = lora_ref.check_close(e * 1.05, e, rtol=1e-2, atol=0.0)
    assert not ok
