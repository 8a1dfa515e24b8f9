"""GPU parity: NF4 dequantisation is bit-exact against the C oracle; QLoRA linear within tolerance."""

import numpy as np
import pytest
import torch

from oracle import lora_ref, nf4 as onf4
from tests.util import single_inputs

pytestmark = pytest.mark.gpu


def _to_state(st: onf4.NF4State, dtype=torch.bfloat16):
    from lorafusion_amd.ops.nf4 import QuantState, QuantState2

    dev = "cuda"
    packed = torch.from_numpy(st.packed).to(dev)
    if st.nested:
        qs = QuantState(torch.Size(st.shape), dtype, st.blocksize, torch.from_numpy(st.absmax).to(dev),
                        torch.from_numpy(st.offset).to(dev),
                        QuantState2(torch.from_numpy(st.absmax2).to(dev), torch.from_numpy(st.code2).to(dev), st.blocksize2))
    else:
        qs = QuantState(torch.Size(st.shape), dtype, st.blocksize, torch.from_numpy(st.absmax).to(dev))
    return packed, qs


def _bits(t: torch.Tensor) -> np.ndarray:
    return t.reshape(-1).view(torch.int16).cpu().numpy().view(np.uint16)


@pytest.mark.parametrize("shape,bs,nested", [
    ((64, 256), 64, True), ((128, 1024), 64, True), ((256, 4096), 64, True), ((16, 2048), 128, True),
    ((8, 64), 64, False), ((3, 1024), 32, False), ((64, 3584), 64, True),
    ((1, 16384), 64, True),  # one second-level block exactly
])
def test_dequant_bit_exact(shape, bs, nested):
    from lorafusion_amd.ops.nf4 import dequantize_nf4_triton

    rng = np.random.default_rng(hash(shape) % 1000)
    w = (rng.standard_normal(shape) * 0.02).astype(np.float32)
    st = onf4.quantize_nf4(w, blocksize=bs, nested=nested)
    expect = onf4.dequantize(st)
    packed, qs = _to_state(st)
    got = dequantize_nf4_triton(packed, qs)
    assert got.shape == tuple(shape) and got.dtype == torch.bfloat16
    assert np.array_equal(_bits(got), expect)


def test_dequant_all_codes_random_state():
    """Every 4-bit code against random absmax codes / scales / offset (not from the quantiser)."""
    from lorafusion_amd.ops.nf4 import dequantize_nf4_triton

    rng = np.random.default_rng(1)
    n = 256 * 64 * 4
    st = onf4.NF4State(
        packed=rng.integers(0, 256, n // 2, dtype=np.uint8), shape=(n,), blocksize=64,
        absmax=rng.integers(0, 256, n // 64, dtype=np.uint8), code2=onf4.dynamic_code_table(),
        absmax2=(rng.random(n // 64 // 256) * 0.05 + 1e-3).astype(np.float32),
        offset=np.asarray([0.0173], dtype=np.float32))
    packed, qs = _to_state(st)
    assert np.array_equal(_bits(dequantize_nf4_triton(packed, qs)), onf4.dequantize(st))


@pytest.mark.parametrize("n,bs,nested", [
    # blocksizes either side of the kernel's chunk of 2048 elements (512 below blocksize 32), lengths that end inside
    # a chunk and inside a second-level block
    (240, 8, False), (8 * 1000, 8, True), (560, 16, True), (16 * 4097, 16, False), (32 * 70, 32, True), (64, 64, True),
    (64 * 33, 64, True), (64 * 629, 64, False), (256 * 10, 256, True), (1024 * 9, 1024, True), (2048 * 3, 2048, True),
    (4096 * 3, 4096, False), (4096 * 5, 4096, True), (64 * 257, 64, True), (64 * (256 * 3 + 17), 64, True),
    (1031 * 2112, 64, True),  # 2.2 M elements: a thousand chunks, ragged end
])
def test_dequant_random_state_sizes(n, bs, nested):
    """Random codes and scales (not from the quantiser) at every power-of-two blocksize class."""
    from lorafusion_amd.ops.nf4 import dequantize_nf4_triton

    rng = np.random.default_rng(n % 9973 + bs)
    nb = n // bs
    if nested:
        st = onf4.NF4State(
            packed=rng.integers(0, 256, n // 2, dtype=np.uint8), shape=(n,), blocksize=bs,
            absmax=rng.integers(0, 256, nb, dtype=np.uint8), code2=onf4.dynamic_code_table(),
            absmax2=(rng.random((nb + 255) // 256) * 0.05 + 1e-3).astype(np.float32),
            offset=np.asarray([0.0173], dtype=np.float32))
    else:
        st = onf4.NF4State(rng.integers(0, 256, n // 2, dtype=np.uint8), (n,), bs,
                           (rng.random(nb) * 0.1 + 1e-3).astype(np.float32), None, None, None, 256)
    packed, qs = _to_state(st)
    got = _bits(dequantize_nf4_triton(packed, qs))
    assert np.array_equal(got, onf4.dequantize(st))


def test_dequant_fp16_output():
    from lorafusion_amd.ops.nf4 import dequantize_nf4_triton

    rng = np.random.default_rng(2)
    st = onf4.quantize_nf4((rng.standard_normal((32, 512)) * 0.02).astype(np.float32))
    _, f32 = onf4.dequantize(st, want_f32=True)
    packed, qs = _to_state(st, torch.float16)
    got = dequantize_nf4_triton(packed, qs)
    assert np.array_equal(got.reshape(-1).view(torch.int16).cpu().numpy().view(np.uint16),
                          f32.astype(np.float16).view(np.uint16))


def test_dequant_config2_shape_and_roundtrip():
    """The NF4 linear configuration's weight: [14336, 4096], blocksize 64, double quantised.  Bit-exact vs the
    oracle, and the size-independent property |dequant(quant(w)) - w| <= half the widest code gap * absmax."""
    from lorafusion_amd.ops.nf4 import dequantize_nf4_triton

    rng = np.random.default_rng(3)
    w = (rng.standard_normal((14336, 4096)) * 0.02).astype(np.float32)
    st = onf4.quantize_nf4(w)
    packed, qs = _to_state(st)
    got = dequantize_nf4_triton(packed, qs)
    assert np.array_equal(_bits(got), onf4.dequantize(st))
    absmax_true = np.abs(w.reshape(-1, 64)).max(axis=1)
    err = np.abs(got.float().cpu().numpy().reshape(-1, 64) - w.reshape(-1, 64)).max(axis=1)
    # widest gap in the code is -0.6962 - (-1.0) = 0.3038; half of it, plus slack for the 8-bit absmax code and bf16
    assert (err <= (0.1520 + 0.03) * absmax_true + 1e-6).all()


def test_quantiser_short_last_second_level_block():
    """A weight whose block count is not a multiple of the second-level block size (896 x 896 at block size
    128: 6272 blocks, 24.5 groups of 256): the product quantiser pads the last group, the state it returns
    dequantises bit-exactly against the oracle, and the round trip stays within the code's resolution."""
    from lorafusion_amd.ops.nf4 import dequantize_nf4_triton, quantize_nf4

    g = torch.Generator(device="cuda").manual_seed(5)
    w = torch.randn(896, 896, generator=g, device="cuda") * 0.02
    packed, qs = quantize_nf4(w, blocksize=128)
    assert qs.absmax.numel() == 6272 and qs.state2.absmax.numel() == 25
    st = onf4.NF4State(packed=packed.cpu().numpy().reshape(-1), shape=(896, 896), blocksize=128, absmax=qs.absmax.cpu().numpy(),
                       code2=qs.state2.code.cpu().numpy(), absmax2=qs.state2.absmax.cpu().numpy(),
                       offset=qs.offset.cpu().numpy().reshape(1).astype(np.float32), blocksize2=256)
    got = dequantize_nf4_triton(packed, qs)
    assert np.array_equal(_bits(got), onf4.dequantize(st))
    blocks = w.reshape(-1, 128)
    err = (got.float().reshape(-1, 128) - blocks).abs().amax(dim=1)
    assert bool((err <= (0.1520 + 0.03) * blocks.abs().amax(dim=1) + 1e-6).all())


def test_dequant_errors():
    from lorafusion_amd.ops.nf4 import QuantState, dequantize_nf4_triton

    packed = torch.zeros(64, dtype=torch.uint8, device="cuda")
    with pytest.raises(ValueError):
        dequantize_nf4_triton(packed, QuantState(torch.Size([128]), torch.float32, 64, torch.ones(2, device="cuda")))
    with pytest.raises(ValueError):
        dequantize_nf4_triton(packed, QuantState(torch.Size([256]), torch.bfloat16, 64, torch.ones(4, device="cuda")))
    with pytest.raises(ValueError):
        dequantize_nf4_triton(packed.float(), QuantState(torch.Size([128]), torch.bfloat16, 64, torch.ones(2, device="cuda")))


def test_qlora_linear_parity():
    """NF4 base weight + LoRA fwd/bwd vs the oracle evaluated on the oracle-dequantised weight."""
    from lorafusion_amd.ops.nf4 import fused_linear_lora_nf4

    M, K, N, r, p, scale = 384, 512, 768, 16, 0.1, 2.0
    d = single_inputs(M, K, N, r, p=p, seed=9)
    st = onf4.quantize_nf4(d["w"].float().numpy())
    wq = torch.from_numpy(onf4.dequantize(st).view(np.int16)).view(torch.bfloat16).reshape(N, K)
    packed, qs = _to_state(st)
    x = d["x"].cuda().requires_grad_(True)
    a = d["a"].cuda().requires_grad_(True)
    b = d["b"].cuda().requires_grad_(True)
    y = fused_linear_lora_nf4(x, packed, qs, a, b, scale, dropout_p=p, dropout_mask=d["mask"].cuda())
    y.backward(d["dy"].cuda())
    ye, _ = lora_ref.linear_lora_fwd_fp32(d["x"], wq, d["a"], d["b"], scale, d["mask"], p)
    dxe, dae, dbe, _ = lora_ref.linear_lora_bwd_fp32(d["dy"], d["x"], wq, d["a"], d["b"], scale, d["mask"], p)
    for got, exp, name in ((y, ye, "y"), (x.grad, dxe, "dx"), (a.grad, dae, "da"), (b.grad, dbe, "db")):
        ok, rel, excess = lora_ref.check_close(got.detach().float().cpu(), exp, rtol=1e-2)
        assert ok, f"{name}: rel {rel:.3e} excess {excess:.3e}"


def test_qlora_linear_adapter_grads_only_and_seeded_mask():
    """x without grad: the backward call gets dX = NULL and dequantises nothing; dropout mask from a seed."""
    from lorafusion_amd.ops.hip_ops import make_dropout_mask
    from lorafusion_amd.ops.nf4 import fused_linear_lora_nf4

    M, K, N, r, p, scale = 256, 512, 384, 32, 0.25, 0.5
    d = single_inputs(M, K, N, r, p=p, seed=11)
    st = onf4.quantize_nf4(d["w"].float().numpy())
    wq = torch.from_numpy(onf4.dequantize(st).view(np.int16)).view(torch.bfloat16).reshape(N, K)
    packed, qs = _to_state(st)
    x = d["x"].cuda()
    a = d["a"].cuda().requires_grad_(True)
    b = d["b"].cuda().requires_grad_(True)
    y = fused_linear_lora_nf4(x, packed, qs, a, b, scale, seed=77, dropout_p=p)
    y.backward(d["dy"].cuda())
    mask = make_dropout_mask((M, K), p, 77, "cuda").cpu()
    ye, _ = lora_ref.linear_lora_fwd_fp32(d["x"], wq, d["a"], d["b"], scale, mask, p)
    _, dae, dbe, _ = lora_ref.linear_lora_bwd_fp32(d["dy"], d["x"], None, d["a"], d["b"], scale, mask, p)
    for got, exp, name in ((y, ye, "y"), (a.grad, dae, "da"), (b.grad, dbe, "db")):
        ok, rel, excess = lora_ref.check_close(got.detach().float().cpu(), exp, rtol=1e-2)
        assert ok, f"{name}: rel {rel:.3e} excess {excess:.3e}"


def test_qlora_keep_dequantized_weight_is_bit_identical():
    """One dequantisation per step: the forward leaves the dequantised weight in a tensor of its own and the
    backward reuses it.  Outputs and gradients equal the dequantise-twice path bit for bit (single and packed
    multi-adapter op), and the kept tensor is the oracle's dequantised weight."""
    from lorafusion_amd.ops import hip_ops
    from lorafusion_amd.ops.multi_lora import fused_linear_multi_lora, prepare_multi_lora_batch_info
    from lorafusion_amd.ops.nf4 import NF4WeightRef, fused_linear_lora_nf4
    from lorafusion_amd import _lib as L
    from tests.util import multi_inputs

    M, K, N, r, p, scale = 384, 512, 768, 16, 0.1, 2.0
    d = single_inputs(M, K, N, r, p=p, seed=9)
    st = onf4.quantize_nf4(d["w"].float().numpy())
    wq = torch.from_numpy(onf4.dequantize(st).view(np.int16)).view(torch.bfloat16).reshape(N, K)
    packed, qs = _to_state(st)
    outs = []
    for keep in (False, True):
        x = d["x"].cuda().requires_grad_(True)
        a = d["a"].cuda().requires_grad_(True)
        b = d["b"].cuda().requires_grad_(True)
        y = fused_linear_lora_nf4(x, packed, qs, a, b, scale, dropout_p=p, dropout_mask=d["mask"].cuda(), keep_dequantized=keep)
        y.backward(d["dy"].cuda())
        outs.append((y.detach(), x.grad, a.grad, b.grad))
    for t0, t1 in zip(*outs):
        assert torch.equal(t0, t1)
    # the raw ops: the kept tensor is the dequantised weight; a backward handed a weight uses exactly that weight
    routing = L.single_routing(r, scale, p)
    wref = NF4WeightRef(packed, qs)
    xd, ad, bd, mk, dyd = d["x"].cuda(), d["a"].cuda(), d["b"].cuda(), d["mask"].cuda(), d["dy"].cuda()
    y, s, dense = hip_ops.nf4_lora_forward(xd, wref, [ad], [bd], routing, 16, mk, None, keep_dense=True)
    assert torch.equal(dense.cpu().view(torch.int16), wq.view(torch.int16))
    dx_kept, _, _ = hip_ops.nf4_lora_backward(dyd, xd, wref, [ad], [bd], s, routing, 16, mk, [r], dense=dense)
    assert torch.equal(dx_kept, outs[0][1])
    dx_zero_w, _, _ = hip_ops.nf4_lora_backward(dyd, xd, wref, [ad], [bd], s, routing, 16, mk, [r], dense=torch.zeros_like(dense))
    lora_only = dx_zero_w.float().cpu()          # dY * 0 + the LoRA term alone
    dxe, *_ = lora_ref.linear_lora_bwd_fp32(d["dy"], d["x"], torch.zeros(N, K), d["a"], d["b"], scale, d["mask"], p)
    ok, rel, excess = lora_ref.check_close(lora_only, dxe, rtol=1e-2)
    assert ok, f"dx from a handed-over zero weight: rel {rel:.3e} excess {excess:.3e}"
    with pytest.raises(ValueError):
        hip_ops.nf4_lora_backward(dyd, xd, wref, [ad], [bd], s, routing, 16, mk, [r], dense=dense[:, :64])

    # packed multi-adapter op
    seq, ranks, p_list, scales = [130, 257], [16, 32], [0.0, 0.1], [1.0, 2.0]
    dm = multi_inputs(seq, 512, 384, ranks, p_list, seed=4)
    stm = onf4.quantize_nf4(dm["w"].float().numpy())
    packed_m, qs_m = _to_state(stm)
    info = prepare_multi_lora_batch_info(seq, [0, 1], ranks, p_list, scales, 128)
    outs = []
    for keep in (False, True):
        x = dm["x"].cuda().requires_grad_(True)
        al = [t.cuda().requires_grad_(True) for t in dm["a_list"]]
        bl = [t.cuda().requires_grad_(True) for t in dm["b_list"]]
        y = fused_linear_multi_lora(
            x.unsqueeze(0), packed_m, lora_a_list=al, lora_b_list=bl, seq_len_list=seq,
            padded_seq_len_list=info.padded_seq_len_list, block_to_lookup_table=info.block_to_lookup_table,
            block_to_dropout_p=info.block_to_dropout_p, block_to_alpha=info.block_to_alpha, enable_dropout=True,
            same_dropout_p_value=None, max_r=32, dropout_mask=dm["mask"].cuda(), quant_state=qs_m, keep_dequantized=keep)
        y.backward(dm["dy"].cuda().unsqueeze(0))
        outs.append([y.detach(), x.grad] + [t.grad for t in al + bl])
    for t0, t1 in zip(*outs):
        assert torch.equal(t0, t1)
