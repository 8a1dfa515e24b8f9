"""Merged projections of a decoder layer, as LoRA linears on the fused HIP ops.

The reference merges ``q_proj``/``k_proj``/``v_proj`` into one ``qkv_proj`` before LoRA is applied
(lorafusion/patch/patch_transformers.py:50-163: one [q+2kv, hidden] weight, the three outputs are column
slices of one GEMM) so that a layer runs fewer, larger LoRA linears.  This module does the same without
depending on ``transformers``: any attention / MLP object that holds ``nn.Linear``-like ``q_proj, k_proj,
v_proj, o_proj`` / ``gate_proj, up_proj, down_proj`` can be converted, and ``gate``/``up`` are merged the
same way (two GEMMs that share their input).  Attention itself, rotary embedding and norms stay with the
caller; the default activation of the layer harness is SiLU-multiply on the merged gate/up output, computed inside
the first kernel of the down projection (``swiglu_lora_forward``).

``LoRALinear`` carries the attributes ``patch_lora.lora_forward`` reads from a PEFT LoRA layer
(``base_layer``, ``lora_A``, ``lora_B``, ``lora_dropout``, ``scaling``), so single adapter, packed
multi-adapter batches (through the ``MultiLoRAManager``) and NF4 base weights all work as they do
for a patched PEFT model.  With a manager, the routing of a micro-batch is built once
(``MultiLoRABatchInfo.routing``) and shared by all four linears of every layer.
"""

from __future__ import annotations

import math
from typing import Callable, Iterable

import torch
from torch import nn

from lorafusion_amd.patch.patch_lora import lora_forward, swiglu_lora_forward


@torch.no_grad()
def align_linear_layer_attrs(original_linear, new_linear) -> None:
    """Device, dtype and ``requires_grad`` of ``new_linear`` follow ``original_linear``
    (lorafusion/patch/patch_transformers.py:38-47)."""
    new_linear.weight.requires_grad = original_linear.weight.requires_grad
    new_linear.weight.data = new_linear.weight.data.to(device=original_linear.weight.device, dtype=original_linear.weight.dtype)
    if getattr(original_linear, "bias", None) is not None and getattr(new_linear, "bias", None) is not None:
        new_linear.bias.requires_grad = original_linear.bias.requires_grad
        new_linear.bias.data = new_linear.bias.data.to(device=original_linear.bias.device, dtype=original_linear.bias.dtype)


def merge_linears(linears: Iterable) -> nn.Linear:
    """One ``nn.Linear`` whose weight rows are the rows of ``linears`` stacked in order (a missing bias among
    biased layers counts as zero), as QKVMergedCommonAttention.from_original stacks q, k and v."""
    linears = list(linears)
    first = linears[0]
    in_features = first.weight.shape[1]
    if any(l.weight.shape[1] != in_features for l in linears):
        raise ValueError("merged projections must share their input width")
    has_bias = any(getattr(l, "bias", None) is not None for l in linears)
    out = sum(l.weight.shape[0] for l in linears)
    merged = nn.Linear(in_features, out, bias=has_bias, device="meta")
    merged = merged.to_empty(device=first.weight.device)
    align_linear_layer_attrs(first, merged)
    with torch.no_grad():
        row = 0
        for l in linears:
            n = l.weight.shape[0]
            merged.weight[row:row + n] = l.weight
            if has_bias:
                if getattr(l, "bias", None) is not None:
                    merged.bias[row:row + n] = l.bias
                else:
                    merged.bias[row:row + n] = 0
            row += n
    return merged


class LoRALinear(nn.Module):
    """A LoRA linear with the attribute layout of ``peft.tuners.lora.Linear``; ``forward`` is
    ``patch_lora.lora_forward``.

    ``adapters``: name -> ``(r, lora_alpha, dropout_p)``; with the ``MultiLoRAManager`` the names are
    ``lora_<idx>`` (lorafusion/patch/patch_lora.py:96-97).  ``A`` is initialised kaiming-uniform(a=sqrt 5), ``B``
    zero, as PEFT does.  The base weight may be a 16-bit ``nn.Linear`` weight or packed NF4 codes that carry
    ``.quant_state``.
    """

    def __init__(self, base_layer, adapters: dict[str, tuple[int, float, float]], *, use_fused: bool = True,
                 dtype: torch.dtype | None = None) -> None:
        super().__init__()
        self.base_layer = base_layer
        self.use_fused = use_fused
        w = base_layer.weight
        qs = getattr(w, "quant_state", None)
        out_features, in_features = tuple(qs.shape) if qs is not None else tuple(w.shape)
        dtype = dtype or (qs.dtype if qs is not None else w.dtype)
        self.in_features, self.out_features = in_features, out_features
        self.lora_A, self.lora_B, self.lora_dropout = nn.ModuleDict(), nn.ModuleDict(), nn.ModuleDict()
        self.scaling: dict[str, float] = {}
        for name, (r, alpha, p) in adapters.items():
            la = nn.Linear(in_features, r, bias=False, device=w.device, dtype=dtype)
            lb = nn.Linear(r, out_features, bias=False, device=w.device, dtype=dtype)
            nn.init.kaiming_uniform_(la.weight, a=math.sqrt(5))
            nn.init.zeros_(lb.weight)
            self.lora_A[name], self.lora_B[name] = la, lb
            self.lora_dropout[name] = nn.Dropout(p) if p > 0 else nn.Identity()
            self.scaling[name] = alpha / r

    def forward(self, x: torch.Tensor, *args, **kwargs) -> torch.Tensor:
        return lora_forward(self, x, *args, use_fused=self.use_fused, **kwargs)


class MergedProjections(nn.Module):
    """One LoRA linear that computes several projections of the same input; ``forward`` returns the column
    slices (views of one output tensor) in the order the projections were given."""

    def __init__(self, linears: Iterable, adapters, *, use_fused: bool = True) -> None:
        super().__init__()
        linears = list(linears)
        self.sizes = [l.weight.shape[0] for l in linears]
        self.proj = LoRALinear(merge_linears(linears), adapters, use_fused=use_fused)

    def forward(self, x: torch.Tensor):
        return torch.split(self.proj(x), self.sizes, dim=-1)


class DecoderLayerLoRAProjections(nn.Module):
    """The seven projections of a Llama-style decoder layer as four LoRA linears: ``qkv_proj`` (q, k and v
    merged, N = q + 2 kv), ``o_proj``, ``gate_up_proj`` (N = 2 mlp) and ``down_proj``.

    ``forward(hidden, attention=..., activation=...)`` strings them together with the caller's attention
    (``(q, k, v) -> [tokens, q]``) and activation (``(gate, up) -> [tokens, mlp]``; by default SiLU(gate) * up, computed on the merged tensor), without
    norms or residuals: a harness for layer-shaped runs of the linears, not a transformer block.
    """

    def __init__(self, attn, mlp, adapters, *, use_fused: bool = True) -> None:
        super().__init__()
        self.qkv_proj = MergedProjections([attn.q_proj, attn.k_proj, attn.v_proj], adapters, use_fused=use_fused)
        self.o_proj = LoRALinear(attn.o_proj, adapters, use_fused=use_fused)
        self.gate_up_proj = MergedProjections([mlp.gate_proj, mlp.up_proj], adapters, use_fused=use_fused)
        self.down_proj = LoRALinear(mlp.down_proj, adapters, use_fused=use_fused)

    @classmethod
    def from_shapes(cls, hidden: int, kv: int, mlp: int, adapters, *, device="cuda", dtype=torch.bfloat16,
                    std: float = 0.02, use_fused: bool = True, seed: int = 0) -> "DecoderLayerLoRAProjections":
        """Random-init base weights ~ N(0, std) of a layer with ``hidden`` model width, ``kv`` key/value width
        and ``mlp`` intermediate width (an 8B-class layer: 4096, 1024, 14336)."""
        g = torch.Generator(device=device).manual_seed(seed)

        def lin(k, n):
            l = nn.Linear(k, n, bias=False, device="meta").to_empty(device=device).to(dtype)
            with torch.no_grad():
                l.weight.copy_(torch.randn(n, k, generator=g, device=device) * std)
            l.weight.requires_grad = False
            return l

        attn, mlp_m = nn.Module(), nn.Module()
        attn.q_proj, attn.k_proj, attn.v_proj, attn.o_proj = lin(hidden, hidden), lin(hidden, kv), lin(hidden, kv), lin(hidden, hidden)
        mlp_m.gate_proj, mlp_m.up_proj, mlp_m.down_proj = lin(hidden, mlp), lin(hidden, mlp), lin(mlp, hidden)
        return cls(attn, mlp_m, adapters, use_fused=use_fused)

    def linears(self) -> dict[str, LoRALinear]:
        return {"qkv": self.qkv_proj.proj, "o": self.o_proj, "gate_up": self.gate_up_proj.proj, "down": self.down_proj}

    def forward(self, hidden: torch.Tensor, attention: Callable | None = None, activation: Callable | None = None):
        q, k, v = self.qkv_proj(hidden)
        ctx = attention(q, k, v) if attention is not None else q
        h = self.o_proj(ctx.contiguous())
        if activation is None:
            # SiLU(gate) * up on the merged projection output, as the prologue of the down projection's rank-r pass:
            # the two halves are read in place, once, and the backward writes the gradient of the merged tensor
            return swiglu_lora_forward(self.down_proj, self.gate_up_proj.proj(h), use_fused=self.down_proj.use_fused)
        gate, up = self.gate_up_proj(h)
        return self.down_proj(activation(gate, up).contiguous())


def patch_module(model: nn.Module, from_type, transform: Callable, layer_indices: list[int] | None = None) -> nn.Module:
    """Replace every sub-module of ``from_type`` by ``transform(sub_module)``; with ``layer_indices`` only inside
    layers whose index appears in the module path (lorafusion/patch/patch_transformers.py:251-275)."""
    for name, module in model.named_modules():
        for sub_name, sub in list(module.named_children()):
            if isinstance(sub, from_type):
                full = f"{name}.{sub_name}."
                if layer_indices is not None and all(f".{i}." not in full for i in layer_indices):
                    continue
                setattr(module, sub_name, transform(sub))
    return model
