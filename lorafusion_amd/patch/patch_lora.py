"""Route PEFT LoRA linear layers through the fused HIP ops.

Same behaviour as lorafusion/patch/patch_lora.py:11-184: ``apply_lora`` replaces
``peft.tuners.lora.Linear.forward`` with ``lora_forward``, which picks the single- or
multi-adapter op depending on the ``MultiLoRAManager`` and falls back to the unfused torch
expressions when ``use_fused=False``.  The layer is duck-typed (``base_layer.weight/.bias``,
``lora_A/lora_B[name].weight``, ``lora_dropout[name].p``, ``scaling[name]``, ``training``), so
any module with those attributes works when peft is not installed.

Extension: a base layer whose weight is stored as NF4 the way bitsandbytes' ``Linear4bit`` holds it
(a packed ``uint8`` tensor carrying a ``quant_state`` attribute) goes through the QLoRA ops
(``fused_linear_lora_nf4`` / ``fused_linear_multi_lora(quant_state=...)``), which the reference's
patch does not cover.
"""

from __future__ import annotations

import torch

from lorafusion_amd.ops.lora_torch_ref import torch_ref_linear_lora, torch_ref_linear_multi_lora
from lorafusion_amd.ops.lora_v1 import fused_linear_lora
from lorafusion_amd.ops.multi_lora import fused_linear_multi_lora, get_multi_lora_manager

try:  # peft is optional
    from peft.tuners.lora import Linear as LoRALinear
except Exception:  # noqa: BLE001
    LoRALinear = None

_REQUIRED_ATTRS = ("base_layer", "lora_A", "lora_B", "lora_dropout", "scaling")


def _is_lora_linear(model) -> bool:
    if LoRALinear is not None and isinstance(model, LoRALinear):
        return True
    return all(hasattr(model, a) for a in _REQUIRED_ATTRS)


def _cast_input(model, x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    cast = getattr(model, "_cast_input_dtype", None)
    return cast(x, dtype) if cast is not None else x.to(dtype)


def _nf4_state(weight):
    """The quant state of an NF4-packed base weight, or None for an ordinary 16-bit weight."""
    qs = getattr(weight, "quant_state", None)
    if qs is None or weight.dtype != torch.uint8:
        return None
    if getattr(qs, "quant_type", "nf4") != "nf4":
        raise ValueError(f"only NF4 4-bit base weights are supported, got quant_type={qs.quant_type!r}")
    return qs


def _dense_weight(weight, qs):
    from lorafusion_amd.ops.nf4 import dequantize_nf4_triton

    return weight if qs is None else dequantize_nf4_triton(weight.detach().reshape(-1), qs)


def _single(model, x, adapter_key, linear_bias, use_fused):
    lora_a = model.lora_A[adapter_key].weight
    lora_b = model.lora_B[adapter_key].weight
    p = float(getattr(model.lora_dropout[adapter_key], "p", 0.0)) if model.training else 0.0
    scaling = model.scaling[adapter_key]
    x = _cast_input(model, x, lora_a.dtype)
    weight = model.base_layer.weight
    qs = _nf4_state(weight)
    if use_fused and qs is not None:
        from lorafusion_amd.ops.nf4 import fused_linear_lora_nf4

        return fused_linear_lora_nf4(x, weight.detach().reshape(-1), qs, lora_a, lora_b, scaling, dropout_p=p,
                                     linear_bias=linear_bias)
    fn = fused_linear_lora if use_fused else torch_ref_linear_lora
    return fn(x=x, linear_w=_dense_weight(weight, qs), lora_a=lora_a, lora_b=lora_b, alpha=scaling,
              dropout_p=p, linear_bias=linear_bias)


def lora_forward(model, x: torch.Tensor, *args, use_fused: bool = True, **kwargs) -> torch.Tensor:
    """Forward of a LoRA linear layer through the fused (or unfused) op."""
    if not _is_lora_linear(model):
        raise TypeError(f"model must be a LoRALinear, but got {type(model)}")
    manager = get_multi_lora_manager()
    result_dtype = x.dtype
    linear_bias = getattr(model.base_layer, "bias", None)

    if manager is None:
        if len(model.lora_A) > 1:
            raise ValueError("Multi-LoRA is not enabled, but the model has multiple LoRA adapters.")
        result = _single(model, x, next(iter(model.lora_A.keys())), linear_bias, use_fused)
        return result.to(result_dtype)

    manager.register_lora_linear(model)
    info = manager.get_newest_batch_info() if manager.is_in_forward else manager.get_oldest_batch_info()
    if info is None:
        raise ValueError("no MultiLoRABatchInfo registered with the manager for this pass")
    if info.num_active_adapters == 1:
        result = _single(model, x, f"lora_{info.lora_idx_list[0]}", linear_bias, use_fused)
        return result.to(result_dtype)

    lora_a_list = [model.lora_A[f"lora_{i}"].weight for i in info.lora_idx_list]
    lora_b_list = [model.lora_B[f"lora_{i}"].weight for i in info.lora_idx_list]
    x = _cast_input(model, x, lora_a_list[0].dtype)
    weight = model.base_layer.weight
    qs = _nf4_state(weight)
    if use_fused:
        enable_dropout = bool(model.training and info.enable_dropout)
        result = fused_linear_multi_lora(
            padded_x=x,
            linear_w=weight if qs is None else weight.detach().reshape(-1),
            quant_state=qs,
            lora_a_list=lora_a_list,
            lora_b_list=lora_b_list,
            seq_len_list=info.seq_len_list,
            padded_seq_len_list=info.padded_seq_len_list,
            block_to_lookup_table=info.block_to_lookup_table,
            block_to_dropout_p=info.block_to_dropout_p,
            block_to_alpha=info.block_to_alpha,
            enable_dropout=enable_dropout,
            same_dropout_p_value=info.same_dropout_p_value,
            max_r=info.max_r,
            linear_bias=linear_bias,
            routing=info.routing(enable_dropout=enable_dropout),
        )
    else:
        result = torch_ref_linear_multi_lora(
            padded_x=x,
            linear_w=_dense_weight(weight, qs),
            lora_a_list=lora_a_list,
            lora_b_list=lora_b_list,
            seq_len_list=info.seq_len_list,
            padded_seq_len_list=info.padded_seq_len_list,
            alpha_list=info.alpha_list,
            dropout_p_list=[p if model.training else 0.0 for p in info.dropout_p_list],
            linear_bias=linear_bias,
        )
    return result.to(result_dtype)


def swiglu_lora_forward(model, gate_up: torch.Tensor, up: "torch.Tensor | None" = None, *, use_fused: bool = True) -> torch.Tensor:
    """``lora_forward(model, silu(gate) * up)`` for the down projection of a SwiGLU MLP, with gate and up the two halves
    of ``gate_up`` (or ``gate_up`` the gate tensor and ``up`` given separately): on the fused path the activation is the prologue of the linear's rank-r pass (one pass over the
    gate/up tensor instead of an activation pass plus a pass over its output).  Same adapter selection as
    ``lora_forward``; NF4 base weights and ``use_fused=False`` take the activation kernel followed by ``lora_forward``."""
    from lorafusion_amd.ops.norm_act import silu_mul, silu_mul_merged
    from lorafusion_amd.ops.swiglu_lora import fused_swiglu_linear_lora, fused_swiglu_linear_multi_lora

    if not _is_lora_linear(model):
        raise TypeError(f"model must be a LoRALinear, but got {type(model)}")
    weight = model.base_layer.weight
    if not use_fused or _nf4_state(weight) is not None or not gate_up.is_cuda:
        if up is not None:
            act = silu_mul(gate_up, up) if gate_up.is_cuda else torch.nn.functional.silu(gate_up) * up
        elif gate_up.is_cuda:
            act = silu_mul_merged(gate_up)
        else:
            half = gate_up.shape[-1] // 2
            act = torch.nn.functional.silu(gate_up[..., :half]) * gate_up[..., half:]
        return lora_forward(model, act, use_fused=use_fused)
    manager = get_multi_lora_manager()
    result_dtype = gate_up.dtype
    linear_bias = getattr(model.base_layer, "bias", None)

    def single(adapter_key):
        lora_a = model.lora_A[adapter_key].weight
        lora_b = model.lora_B[adapter_key].weight
        p = float(getattr(model.lora_dropout[adapter_key], "p", 0.0)) if model.training else 0.0
        return fused_swiglu_linear_lora(_cast_input(model, gate_up, lora_a.dtype), weight, lora_a, lora_b,
                                        model.scaling[adapter_key], dropout_p=p, linear_bias=linear_bias,
                                        up=None if up is None else _cast_input(model, up, lora_a.dtype))

    if manager is None:
        if len(model.lora_A) > 1:
            raise ValueError("Multi-LoRA is not enabled, but the model has multiple LoRA adapters.")
        return single(next(iter(model.lora_A.keys()))).to(result_dtype)
    manager.register_lora_linear(model)
    info = manager.get_newest_batch_info() if manager.is_in_forward else manager.get_oldest_batch_info()
    if info is None:
        raise ValueError("no MultiLoRABatchInfo registered with the manager for this pass")
    if info.num_active_adapters == 1:
        return single(f"lora_{info.lora_idx_list[0]}").to(result_dtype)
    lora_a_list = [model.lora_A[f"lora_{i}"].weight for i in info.lora_idx_list]
    lora_b_list = [model.lora_B[f"lora_{i}"].weight for i in info.lora_idx_list]
    enable_dropout = bool(model.training and info.enable_dropout)
    g = _cast_input(model, gate_up, lora_a_list[0].dtype)
    if g.ndim == 3:
        if g.shape[0] != 1:
            raise ValueError("currently, we only support batch size 1 for multi-linear LoRA")
    return fused_swiglu_linear_multi_lora(g, weight, lora_a_list, lora_b_list, info.routing(enable_dropout=enable_dropout),
                                          linear_bias=linear_bias,
                                          up=None if up is None else _cast_input(model, up, lora_a_list[0].dtype)).to(result_dtype)


def apply_lora(*, use_fused: bool = True, target_cls=None) -> None:
    """Replace ``forward`` of peft's LoRA ``Linear`` (or of ``target_cls``) with ``lora_forward``."""
    cls = target_cls if target_cls is not None else LoRALinear
    if cls is None:
        raise ImportError("peft is not installed; pass target_cls=<your LoRA linear class> to apply_lora().")

    def forward_wrapper(self, x: torch.Tensor, *args, **kwargs) -> torch.Tensor:
        return lora_forward(self, x, *args, use_fused=use_fused, **kwargs)

    cls.forward = forward_wrapper
    cls._lorafusion_use_fused = use_fused   # read by the SwiGLU MLP forward to pick the prologue path for down_proj
