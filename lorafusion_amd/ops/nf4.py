"""NF4 (4-bit NormalFloat) weights: quant state, dequantisation through HIP, QLoRA linear.

``dequantize_nf4_triton(A, quant_state)`` keeps the name and argument meaning of
lorafusion/ops/triton_ops/dequantize_nf4.py:271-346 and accepts any object with the
bitsandbytes ``QuantState`` attributes it reads there (``shape, dtype, blocksize, absmax,
offset, state2.code, state2.absmax, state2.blocksize``).  ``quantize_nf4`` produces such a
state for synthetic weights (the reference gets it from bitsandbytes, which is not a
dependency here).
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from lorafusion_amd import _lib as L

# lorafusion/ops/triton_ops/dequantize_nf4.py:16-33
NF4_LUT = (
    -1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453, -0.28444138169288635,
    -0.18477343022823334, -0.09105003625154495, 0.0, 0.07958029955625534, 0.16093020141124725,
    0.24611230194568634, 0.33791524171829224, 0.44070982933044434, 0.5626170039176941,
    0.7229568362236023, 1.0,
)


@dataclass
class QuantState2:
    """Second-level state: fp32 absmax per ``blocksize`` first-level blocks and the 256-entry code."""

    absmax: torch.Tensor
    code: torch.Tensor
    blocksize: int = 256


@dataclass
class QuantState:
    """The subset of bitsandbytes' ``QuantState`` that NF4 dequantisation reads."""

    shape: torch.Size
    dtype: torch.dtype
    blocksize: int
    absmax: torch.Tensor          # uint8 codes when nested, else fp32
    offset: torch.Tensor | None = None
    state2: QuantState2 | None = None
    quant_type: str = "nf4"

    @property
    def nested(self) -> bool:
        return self.state2 is not None


def _checked_state(A: torch.Tensor, quant_state):
    """Validate packed codes + quant state; returns the contiguous device tensors the kernels read."""
    L.require_gpu(A, "A")
    if A.dtype != torch.uint8:
        raise ValueError(f"A must be a uint8 tensor of packed 4-bit codes, but got {A.dtype}.")
    shape = torch.Size(quant_state.shape)
    n = shape.numel()
    if A.numel() * 2 != n:
        raise ValueError(f"A holds {A.numel() * 2} codes but quant_state.shape has {n} elements.")
    out_dtype = quant_state.dtype
    if out_dtype not in (torch.bfloat16, torch.float16):
        raise ValueError(f"Unsupported output dtype: {out_dtype}")
    blocksize = int(quant_state.blocksize)
    if blocksize < 8 or blocksize & (blocksize - 1) or n % blocksize:
        raise ValueError(f"blocksize must be a power of two >= 8 dividing the element count, got {blocksize}.")
    state2 = getattr(quant_state, "state2", None)
    nested = state2 is not None
    A = A.contiguous()
    absmax = quant_state.absmax.contiguous()
    if absmax.numel() != n // blocksize:
        raise ValueError(f"absmax must have {n // blocksize} entries, got {absmax.numel()}.")
    if nested:
        if absmax.dtype != torch.uint8:
            raise ValueError("nested quant state: absmax must be uint8 codes.")
        bs2 = int(state2.blocksize)
        code = state2.code.to(device=A.device, dtype=torch.float32).contiguous()
        absmax2 = state2.absmax.to(device=A.device, dtype=torch.float32).contiguous()
        offset = quant_state.offset.to(device=A.device, dtype=torch.float32).reshape(1).contiguous()
        if code.numel() != 256:
            raise ValueError("state2.code must have 256 entries.")
        if bs2 & (bs2 - 1) or absmax2.numel() * bs2 < absmax.numel():
            raise ValueError("state2.absmax does not cover all first-level blocks.")
    else:
        if absmax.dtype != torch.float32:
            raise ValueError("non-nested quant state: absmax must be float32.")
        bs2, code, absmax2, offset = 0, None, None, None
    return A, absmax, code, absmax2, offset, blocksize, bs2, shape, out_dtype


def dequantize_nf4_triton(A: torch.Tensor, quant_state, out: torch.Tensor | None = None) -> torch.Tensor:
    """Dequantise packed NF4 weights to ``quant_state.dtype`` (bf16 / fp16), shape ``quant_state.shape``."""
    A, absmax, code, absmax2, offset, blocksize, bs2, shape, out_dtype = _checked_state(A, quant_state)
    n = shape.numel()
    if out is None:
        out = torch.empty(n, dtype=out_dtype, device=A.device)
    elif out.numel() != n or out.dtype != out_dtype or not out.is_contiguous():
        raise ValueError("out must be a contiguous tensor of quant_state.dtype with as many elements as the weight.")
    rc = L.lib().lf_nf4_dequant(L.ptr(A), L.ptr(absmax), L.ptr(code), L.ptr(absmax2), L.ptr(offset), L.ptr(out), n,
                                blocksize, bs2, L.dtype_id(out_dtype), L.stream_of(A))
    L.check(rc, "lf_nf4_dequant")
    return out.view(shape)


class NF4WeightRef:
    """``struct lf_nf4_weight`` for a packed weight + quant state; keeps the tensors it points to alive."""

    def __init__(self, A: torch.Tensor, quant_state):
        tensors = _checked_state(A, quant_state)
        A, absmax, code, absmax2, offset, blocksize, bs2, shape, out_dtype = tensors
        if len(shape) != 2:
            raise ValueError(f"the quantised weight must be 2-D [N, K], got shape {tuple(shape)}.")
        self.keep = (A, absmax, code, absmax2, offset)
        self.shape, self.dtype = shape, out_dtype
        self.c = L.NF4Weight(L.ptr(A), L.ptr(absmax), L.ptr(code), L.ptr(absmax2), L.ptr(offset), blocksize, bs2, None, 0, 0)

    def with_dense(self, dense, *, valid: bool):
        """The struct with ``dense`` (a [N, K] tensor for the dequantised weight, or None) filled in."""
        if dense is None:
            return self.c
        c = self.c
        return L.NF4Weight(c.packed, c.absmax, c.code2, c.absmax2, c.offset, c.blocksize, c.blocksize2,
                           dense.data_ptr(), 1 if valid else 0, 0)


dequantize_nf4 = dequantize_nf4_triton


def dynamic_code_table(device=None) -> torch.Tensor:
    """256-entry signed dynamic-exponent code table (7 exponent bits) for second-level absmax."""
    data = []
    for i in range(7):
        items = 2 ** i + 1
        b = torch.linspace(0.1, 1, items, dtype=torch.float64)
        means = (b[:-1] + b[1:]) / 2.0
        data += (10.0 ** (-6 + i) * means).tolist()
        data += (-(10.0 ** (-6 + i)) * means).tolist()
    data += [0.0, 1.0]
    data += [0.0] * (256 - len(data))
    return torch.tensor(sorted(data), dtype=torch.float32, device=device)


def _nearest(x: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    mids = (table[:-1].double() + table[1:].double()) / 2.0
    return torch.bucketize(x.double(), mids, right=False).to(torch.uint8)


def quantize_nf4(w: torch.Tensor, blocksize: int = 64, compress_statistics: bool = True,
                 blocksize2: int = 256, dtype: torch.dtype | None = None):
    """Blockwise NF4 quantisation over the row-major flattening of ``w``.

    Returns ``(packed uint8 [n/2, 1], QuantState)``; element 2i sits in the high nibble of byte i.
    """
    shape = w.shape
    flat = w.detach().float().reshape(-1)
    n = flat.numel()
    if n % blocksize or n % 2:
        raise ValueError("element count must be a multiple of the blocksize")
    blocks = flat.reshape(-1, blocksize)
    absmax = blocks.abs().amax(dim=1)
    safe = torch.where(absmax > 0, absmax, torch.ones_like(absmax))
    lut = torch.tensor(NF4_LUT, dtype=torch.float32, device=w.device)
    idx = _nearest((blocks / safe[:, None]).reshape(-1), lut)
    packed = ((idx[0::2] << 4) | idx[1::2]).reshape(-1, 1)
    out_dtype = dtype or (w.dtype if w.dtype in (torch.bfloat16, torch.float16) else torch.bfloat16)
    if not compress_statistics:
        return packed, QuantState(shape, out_dtype, blocksize, absmax)
    offset = absmax.double().mean().float().reshape(1)
    nb = absmax.numel()
    pad = (-nb) % blocksize2          # a short last second-level block is padded with zeros, which change no maximum
    centred = torch.nn.functional.pad(absmax - offset, (0, pad)).reshape(-1, blocksize2)
    absmax2 = centred.abs().amax(dim=1)
    safe2 = torch.where(absmax2 > 0, absmax2, torch.ones_like(absmax2))
    code = dynamic_code_table(w.device)
    absq = _nearest((centred / safe2[:, None]).reshape(-1), code)[:nb].contiguous()
    return packed, QuantState(shape, out_dtype, blocksize, absq, offset, QuantState2(absmax2, code, blocksize2))


class FusedLinearLoRANF4(torch.autograd.Function):
    """QLoRA linear: NF4 base weight dequantised on the fly, bf16/fp16 adapters.

    Forward and backward each dequantise the weight into the call's workspace
    (``lf_nf4_lora_fwd`` / ``lf_nf4_lora_bwd``) and run the fused LoRA GEMMs on it; only the
    packed weight stays resident.  With ``keep_dequantized`` the forward's dequantised weight is
    kept for the backward instead (one dequantisation per step, 2*N*K bytes held in between).
    """

    @staticmethod
    def forward(ctx, x, packed_w, quant_state, lora_a, lora_b, alpha, dropout_p, seed, linear_bias, dropout_mask,
                keep_dequantized=False):
        from lorafusion_amd.ops import hip_ops
        from lorafusion_amd.ops.lora_v1 import _validate_shapes

        if x.ndim == 3:
            lead = x.shape[:2]
            x2d = x.reshape(lead[0] * lead[1], -1)
        elif x.ndim == 2:
            lead, x2d = None, x
        else:
            raise ValueError(f"Expected x to have 2 or 3 dimensions, got {x.ndim}.")
        x2d = x2d.contiguous()
        if quant_state.dtype != x2d.dtype:
            raise ValueError(f"quant_state.dtype {quant_state.dtype} must match x.dtype {x2d.dtype}.")
        wref = NF4WeightRef(packed_w, quant_state)
        lora_a, lora_b = lora_a.contiguous(), lora_b.contiguous()
        M, N, K, r = _validate_shapes(x2d, tuple(wref.shape), x2d.dtype, lora_a, lora_b, linear_bias, dropout_p)
        mask = None
        bias = linear_bias.contiguous() if linear_bias is not None else None
        if dropout_p > 0:
            if dropout_mask is None:
                dropout_mask = hip_ops.make_dropout_mask((M, K), dropout_p, seed, x2d.device)
            mask = hip_ops._check_mask(dropout_mask.reshape(M, -1), (M, K))
            if not hip_ops.is_packed_mask(mask, K):
                mask = hip_ops.pack_mask(mask)   # read three times (rank-r forward, dA, dX): an eighth of the bytes each
        p_eff = dropout_p if mask is not None else 0.0
        routing = L.single_routing(r, alpha, p_eff)
        dense = None
        if keep_dequantized:
            y, s, dense = hip_ops.nf4_lora_forward(x2d, wref, [lora_a], [lora_b], routing, L.round_rank(r), mask, bias,
                                                   keep_dense=True)
        else:
            y, s = hip_ops.nf4_lora_forward(x2d, wref, [lora_a], [lora_b], routing, L.round_rank(r), mask, bias)
        ctx.save_for_backward(x2d, packed_w, lora_a, lora_b, mask, s, dense)
        ctx.quant_state, ctx.alpha, ctx.p, ctx.lead = quant_state, alpha, p_eff, lead
        return y if lead is None else y.reshape(*lead, N)

    @staticmethod
    def backward(ctx, dy):
        from lorafusion_amd.ops import hip_ops

        x2d, packed_w, lora_a, lora_b, mask, s, dense = ctx.saved_tensors
        dy2d = dy.reshape(-1, dy.shape[-1]).contiguous()
        r = lora_a.shape[0]
        wref = NF4WeightRef(packed_w, ctx.quant_state)
        routing = L.single_routing(r, ctx.alpha, ctx.p)
        dx, da_list, db_list = hip_ops.nf4_lora_backward(dy2d, x2d, wref, [lora_a], [lora_b], s, routing,
                                                         L.round_rank(r), mask, [r],
                                                         requires_dx=ctx.needs_input_grad[0], dense=dense)
        if dx is not None and ctx.lead is not None:
            dx = dx.reshape(*ctx.lead, -1)
        return dx, None, None, da_list[0], db_list[0], None, None, None, None, None, None


def fused_linear_lora_nf4(x, packed_w, quant_state, lora_a, lora_b, alpha, seed=None, dropout_p=0.0,
                          linear_bias=None, dropout_mask=None, *, keep_dequantized: bool = False):
    """``fused_linear_lora`` with the base weight stored as NF4 (``packed_w`` + ``quant_state``).

    ``keep_dequantized``: keep the forward's dequantised weight (2*N*K bytes) until the backward has run, which
    then dequantises nothing -- for a backward that follows its forward closely (one layer at a time, or a
    recomputed forward under activation checkpointing); the default holds only the packed weight."""
    return FusedLinearLoRANF4.apply(x, packed_w, quant_state, lora_a, lora_b, alpha, dropout_p, seed,
                                    linear_bias, dropout_mask, keep_dequantized)
