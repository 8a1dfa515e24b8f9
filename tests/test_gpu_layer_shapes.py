"""GPU parity at the full layer shapes of the benchmark configurations.

The dense M x N x K products are too large to restate on the CPU in a test, and they do not need
to be: Y and dX are row-wise independent, so the oracle is evaluated on a sample of rows of every
adapter segment (plus padded rows, which must carry the base GEMM only), while dA and dB -- sums
over all rows of a segment, but only rank-r wide -- are restated in full.  Tolerance as in
test_gpu_lora_single.py: rtol 1e-2, atol 1e-2*rms against the fp32-accumulated oracle.

Shapes: an 8B-class decoder layer (hidden 4096, kv 1024, MLP 14336; merged qkv N=6144), 16384 packed
tokens, 4 adapters r=16; a 70B-class layer (hidden 8192, kv 1024, MLP 28672), 8192 tokens, 8 adapters
r=64, base weights in NF4; the single NF4 linear 4096 -> 14336 with 4096 tokens.
"""

import math

import numpy as np
import pytest
import torch

from oracle import lora_ref
from oracle import nf4 as onf4
from tests.util import lognormal_segments

pytestmark = pytest.mark.gpu

RTOL = 1e-2
ROWS_PER_SEGMENT = 24


def _close(actual, expected, what):
    ok, rel, excess = lora_ref.check_close(actual.detach().float().cpu(), expected, rtol=RTOL)
    assert ok, f"{what}: max|err|/max|e| = {rel:.3e}, worst excess over bound {excess:.3e}"


def _gpu_randn(shape, seed, std=1.0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.randn(shape, generator=g, device="cuda") * std).to(torch.bfloat16)


def _nf4_weight(w_gpu):
    """Quantise on the GPU (the build's own quantiser), dequantise with the CPU oracle: the
    oracle's weight is the exact bf16 value the device dequant must reproduce."""
    from lorafusion_amd.ops.nf4 import dequantize_nf4_triton, quantize_nf4

    packed, qs = quantize_nf4(w_gpu.float())
    st = onf4.NF4State(
        packed=packed.cpu().numpy().reshape(-1), absmax=qs.absmax.cpu().numpy(), shape=tuple(w_gpu.shape), blocksize=qs.blocksize,
        code2=qs.state2.code.cpu().numpy(), absmax2=qs.state2.absmax.cpu().numpy(),
        offset=qs.offset.cpu().numpy().reshape(1).astype(np.float32),
        blocksize2=qs.state2.blocksize)
    w_oracle = torch.from_numpy(onf4.dequantize(st).view(np.int16)).view(torch.bfloat16).reshape(w_gpu.shape)
    w_dev = dequantize_nf4_triton(packed, qs).reshape(w_gpu.shape)
    assert torch.equal(w_dev.cpu().view(torch.int16), w_oracle.view(torch.int16)), "NF4 dequant is not bit-exact"
    return packed, qs, w_oracle


def _run_multi(tokens, K, N, ranks, p_list, scale_list, nf4=False, seed=0):
    from lorafusion_amd.ops.multi_lora import fused_linear_multi_lora, prepare_multi_lora_batch_info

    n_ad = len(ranks)
    seq = lognormal_segments(tokens, n_ad, seed=seed)
    assert len(seq) == n_ad and sum(seq) == tokens
    info = prepare_multi_lora_batch_info(seq, list(range(n_ad)), ranks, p_list, scale_list, 128, output_dtype=torch.float32)
    padded = info.padded_seq_len_list
    Mp = sum(padded)
    x = _gpu_randn((Mp, K), seed + 1).requires_grad_(True)
    w = _gpu_randn((N, K), seed + 2, 0.02)
    dy = _gpu_randn((Mp, N), seed + 3)
    a_list = [(_gpu_randn((r, K), seed + 10 + i) / math.sqrt(K)).requires_grad_(True) for i, r in enumerate(ranks)]
    b_list = [_gpu_randn((N, r), seed + 30 + i, 0.01).requires_grad_(True) for i, r in enumerate(ranks)]
    gm = torch.Generator(device="cuda").manual_seed(seed + 4)
    row_p = torch.cat([torch.full((pl,), float(p)) for pl, p in zip(padded, p_list)]).cuda()
    mask = torch.rand((Mp, K), generator=gm, device="cuda") >= row_p[:, None]
    qs = None
    if nf4:
        # the op takes the packed codes + quant state and dequantises inside lf_nf4_lora_fwd / _bwd
        w, qs, w_cpu = _nf4_weight(w)
    else:
        w_cpu = w.cpu()

    y = fused_linear_multi_lora(
        x.unsqueeze(0), w, lora_a_list=a_list, lora_b_list=b_list, seq_len_list=seq, padded_seq_len_list=padded,
        block_to_lookup_table=info.block_to_lookup_table, block_to_dropout_p=info.block_to_dropout_p,
        block_to_alpha=info.block_to_alpha, enable_dropout=info.enable_dropout,
        same_dropout_p_value=info.same_dropout_p_value, max_r=info.max_r, dropout_mask=mask, quant_state=qs)
    y.backward(dy.unsqueeze(0))
    torch.cuda.synchronize()
    y, dx = y[0].detach(), x.grad

    rng = np.random.default_rng(seed)
    start = 0
    for i, (n, pl) in enumerate(zip(seq, padded)):
        a, b = a_list[i].detach().cpu(), b_list[i].detach().cpu()
        sl = slice(start, start + n)
        xs, dys, ms = x.detach()[sl].cpu(), dy[sl].cpu(), mask[sl].cpu()
        # rank-r gradients of the whole segment
        _, dae, dbe, _ = lora_ref.linear_lora_bwd_fp32(dys, xs, None, a, b, scale_list[i], ms, p_list[i])
        _close(a_list[i].grad, dae, f"da[{i}]")
        _close(b_list[i].grad, dbe, f"db[{i}]")
        # sampled valid rows: first, last and random ones
        idx = np.unique(np.concatenate([[0, n - 1], rng.integers(0, n, ROWS_PER_SEGMENT)]))
        ti = torch.from_numpy(idx)
        ye, _ = lora_ref.linear_lora_fwd_fp32(xs[ti], w_cpu, a, b, scale_list[i], ms[ti], p_list[i])
        dxe, *_ = lora_ref.linear_lora_bwd_fp32(dys[ti], xs[ti], w_cpu, a, b, scale_list[i], ms[ti], p_list[i])
        _close(y[sl][ti.cuda()], ye, f"y rows of segment {i}")
        _close(dx[sl][ti.cuda()], dxe, f"dx rows of segment {i}")
        # padded rows: base GEMM only
        if pl > n:
            pad = torch.arange(start + n, start + pl)[:4]
            xp, dyp = x.detach()[pad.cuda()].cpu(), dy[pad.cuda()].cpu()
            ype, _ = lora_ref.linear_lora_fwd_fp32(xp, w_cpu, a, b, 0.0)
            dxpe, *_ = lora_ref.linear_lora_bwd_fp32(dyp, xp, w_cpu, a, b, 0.0)
            _close(y[pad.cuda()], ype, f"y padded rows of segment {i}")
            _close(dx[pad.cuda()], dxpe, f"dx padded rows of segment {i}")
        start += pl


@pytest.mark.parametrize("K,N", [(4096, 4096), (4096, 6144), (4096, 1024), (4096, 14336), (4096, 28672), (14336, 4096)])
def test_8b_layer_projections(K, N):
    """16384 packed tokens, 4 adapters r=16, scales {1,2,2,4}, p {0,.05,.1,.1}."""
    _run_multi(16384, K, N, [16] * 4, [0.0, 0.05, 0.1, 0.1], [1.0, 2.0, 2.0, 4.0])


@pytest.mark.parametrize("tokens,K,N,n_adapters,seed", [(2048, 5120, 5120, 2, 1), (4096, 5120, 5120, 4, 0),
                                                        (8192, 5120, 5120, 4, 0), (2048, 8192, 8192, 2, 1)])
def test_kernel_grid_shapes(tokens, K, N, n_adapters, seed):
    """The square shapes of the reference's kernel benchmark grid that no layer above has (hidden 5120: 20 tile
    columns of 256, a K of 80 steps of 64; 2048 tokens x 8192: one round of 128x256 tiles), adapters of r=16.  (Seeds
    whose segments all hold several hundred tokens: sums over a handful of rows are covered by the few-term
    regression list of test_gpu_layer_fullsize.py, with the bound that applies to them.)"""
    _run_multi(tokens, K, N, [16] * n_adapters, [0.05, 0.1, 0.0, 0.1][:n_adapters], [2.0, 1.0, 2.0, 4.0][:n_adapters], seed=seed)


def test_one_round_of_128_row_persistent_tiles():
    """1800 tokens of two adapters over a 4096 x 4096 weight: the padded batch is between half a round and one round of
    128x256 tiles, which the library runs on the persistent kernel's three-stage instance in both products (asserted
    from the launch plan, so the case keeps its meaning if the plan changes)."""
    import ctypes

    from lorafusion_amd import _lib as L
    from lorafusion_amd.ops.multi_lora import prepare_multi_lora_batch_info

    seq = lognormal_segments(1800, 2, seed=1)
    info = prepare_multi_lora_batch_info(seq, [0, 1], [16, 16], [0.05, 0.1], [2.0, 1.0], 128, output_dtype=torch.float32)
    Mp = sum(info.padded_seq_len_list)
    rows, ch, ct = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    L.check(L.lib().lf_gemm_plan(Mp, 4096, 4096, 128, ctypes.byref(rows), ctypes.byref(ch), ctypes.byref(ct)), "lf_gemm_plan")
    assert (rows.value, ch.value, ct.value) == (Mp, 8, -1)
    _run_multi(1800, 4096, 4096, [16, 16], [0.05, 0.1], [2.0, 1.0], seed=1)


@pytest.mark.parametrize("K,N", [(8192, 8192), (8192, 1024), (8192, 10240), (8192, 28672), (8192, 57344), (28672, 8192)])
def test_70b_layer_projections_nf4(K, N):
    """8192 tokens, 8 adapters r=64, base weight quantised to NF4 and dequantised on the device; the separate
    projections and the merged ones (q+k+v: N = 10240, gate+up: N = 57344)."""
    _run_multi(8192, K, N, [64] * 8, [0.0, 0.05, 0.1, 0.1, 0.0, 0.05, 0.1, 0.1], [1.0, 2.0, 2.0, 4.0] * 2, nf4=True)


def test_nf4_linear_4096_to_14336():
    """Single adapter, NF4 base weight [14336, 4096], 4096 tokens, r=16, p=0.1, scale 2."""
    from lorafusion_amd.ops.nf4 import fused_linear_lora_nf4

    M, K, N, r, p, scale = 4096, 4096, 14336, 16, 0.1, 2.0
    x = _gpu_randn((M, K), 1).requires_grad_(True)
    w0 = _gpu_randn((N, K), 2, 0.02)
    dy = _gpu_randn((M, N), 3)
    a = (_gpu_randn((r, K), 10) / math.sqrt(K)).requires_grad_(True)
    b = _gpu_randn((N, r), 30, 0.01).requires_grad_(True)
    gm = torch.Generator(device="cuda").manual_seed(4)
    mask = torch.rand((M, K), generator=gm, device="cuda") >= p
    packed, qs, w_cpu = _nf4_weight(w0)
    y = fused_linear_lora_nf4(x, packed, qs, a, b, scale, dropout_p=p, dropout_mask=mask)
    y.backward(dy)
    torch.cuda.synchronize()
    xs, dys, ms, ac, bc = x.detach().cpu(), dy.cpu(), mask.cpu(), a.detach().cpu(), b.detach().cpu()
    _, dae, dbe, _ = lora_ref.linear_lora_bwd_fp32(dys, xs, None, ac, bc, scale, ms, p)
    _close(a.grad, dae, "da")
    _close(b.grad, dbe, "db")
    ti = torch.from_numpy(np.unique(np.concatenate([[0, M - 1], np.random.default_rng(0).integers(0, M, 64)])))
    ye, _ = lora_ref.linear_lora_fwd_fp32(xs[ti], w_cpu, ac, bc, scale, ms[ti], p)
    dxe, *_ = lora_ref.linear_lora_bwd_fp32(dys[ti], xs[ti], w_cpu, ac, bc, scale, ms[ti], p)
    _close(y.detach()[ti.cuda()], ye, "y rows")
    _close(x.grad[ti.cuda()], dxe, "dx rows")


def test_activation_above_2_gib():
    """270000 tokens x 4096 (2.2 GB of X, 1.1 GB of mask) through the single-adapter op: 32-bit offsets inside the
    kernels must not span the whole operand.  dA and dB (sums over all rows) against the oracle in full, Y and dX
    on sampled rows including the last ones."""
    from lorafusion_amd.ops.lora_v1 import fused_linear_lora

    M, K, N, r, p, scale = 270_000, 4096, 128, 16, 0.1, 2.0
    x = _gpu_randn((M, K), 1).requires_grad_(True)
    w = _gpu_randn((N, K), 2, 0.02)
    dy = _gpu_randn((M, N), 3)
    a = (_gpu_randn((r, K), 4) / math.sqrt(K)).requires_grad_(True)
    b = _gpu_randn((N, r), 5, 0.01).requires_grad_(True)
    mask = torch.rand((M, K), generator=torch.Generator(device="cuda").manual_seed(6), device="cuda") >= p
    y = fused_linear_lora(x, w, a, b, scale, dropout_p=p, dropout_mask=mask)
    y.backward(dy)
    torch.cuda.synchronize()
    xs, dys, ms = x.detach().cpu(), dy.cpu(), mask.cpu()
    ac, bc, wc = a.detach().cpu(), b.detach().cpu(), w.cpu()
    _, dae, dbe, _ = lora_ref.linear_lora_bwd_fp32(dys, xs, None, ac, bc, scale, ms, p)
    _close(a.grad, dae, "da over 270000 rows")
    _close(b.grad, dbe, "db over 270000 rows")
    ti = torch.tensor([0, 1, 127, 128, 131_071, 131_072, 262_143, 262_144, 262_145, M - 129, M - 2, M - 1])
    ye, _ = lora_ref.linear_lora_fwd_fp32(xs[ti], wc, ac, bc, scale, ms[ti], p)
    dxe, *_ = lora_ref.linear_lora_bwd_fp32(dys[ti], xs[ti], wc, ac, bc, scale, ms[ti], p)
    _close(y.detach()[ti.cuda()], ye, "y rows")
    _close(x.grad[ti.cuda()], dxe, "dx rows")

