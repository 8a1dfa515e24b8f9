"""``apply_liger_kernel`` on the HIP kernels (lorafusion/utils/module.py:32-71).

The reference calls liger-kernel's ``apply_liger_kernel_to_{llama,qwen2,mixtral}`` with cross-entropy off, which
replaces the models' RMSNorm and SwiGLU MLP forwards (and the rotary embedding, which is not part of this build:
it stays HF's).  Here the same switch patches the forwards of HF transformers' classes with
``lorafusion_amd.ops.norm_act``: ``{Llama,Qwen2,Mixtral}RMSNorm.forward`` -> ``rms_norm`` and
``{Llama,Qwen2}MLP.forward`` -> ``swiglu_mlp_forward``.  Mixtral's experts keep HF's MLP (their gate/up are batched
per expert in current transformers, not an ``[M, I]`` pair).  ``restore_liger_kernel`` undoes the patch.
"""

from __future__ import annotations

import importlib
from enum import Enum

import torch

from lorafusion_amd.ops.norm_act import rms_norm, swiglu_mlp_forward


class LigerKernelLevel(str, Enum):
    """lorafusion/utils/module.py:32-38."""

    ALL = "all"
    NO_RMS_NORM = "no_rms_norm"
    DISABLE = "disable"

    def __str__(self) -> str:
        return self.value


_MODELS = {
    "llama": ("transformers.models.llama.modeling_llama", "LlamaRMSNorm", "LlamaMLP"),
    "qwen2": ("transformers.models.qwen2.modeling_qwen2", "Qwen2RMSNorm", "Qwen2MLP"),
    "mixtral": ("transformers.models.mixtral.modeling_mixtral", "MixtralRMSNorm", None),
}
_saved: dict[tuple[type, str], object] = {}


def _original_forward(module):
    """HF's own forward of the patched class `module` belongs to -- found along the MRO, so that a subclass of a
    patched class (which inherits the patched forward but is no key of `_saved` itself) falls back correctly."""
    for cls in type(module).__mro__:
        fn = _saved.get((cls, "forward"))
        if fn is not None:
            return fn
    raise RuntimeError(f"{type(module).__name__}: no saved forward (apply_liger_kernel did not patch this class)")


def _rms_norm_forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
    h = hidden_states.shape[-1]
    if (not hidden_states.is_cuda or hidden_states.dtype != self.weight.dtype or hidden_states.dtype == torch.float32
            or h % 8 != 0 or h > 8192):
        # fp32 activations, mixed dtypes, or a width the kernel does not take (rows of 16-byte pieces, at most 8192
        # wide): HF's own arithmetic
        return _original_forward(self)(self, hidden_states)
    return rms_norm(hidden_states, self.weight, self.variance_epsilon)


def _mlp_forward(self, x: torch.Tensor) -> torch.Tensor:
    act = getattr(getattr(self, "config", None), "hidden_act", "silu")
    inter = getattr(getattr(self, "gate_proj", None), "out_features", 0)
    if act not in ("silu", "swish") or not x.is_cuda or x.dtype == torch.float32 or inter % 8 != 0:
        return _original_forward(self)(self, x)
    return swiglu_mlp_forward(self, x)


def _patch(cls: type, fn) -> None:
    key = (cls, "forward")
    if key not in _saved:
        _saved[key] = cls.forward
    cls.forward = fn


def apply_liger_kernel(level: "LigerKernelLevel | str" = LigerKernelLevel.ALL) -> None:
    """Patch HF's Llama / Qwen2 / Mixtral classes; ``level`` as in lorafusion/utils/module.py:41-71 (an unknown
    level raises ``ValueError``)."""
    try:
        level = LigerKernelLevel(level)
    except ValueError:
        raise ValueError(f"Invalid Liger kernel level: {level}") from None
    if level == LigerKernelLevel.DISABLE:
        return
    for module_name, norm_name, mlp_name in _MODELS.values():
        mod = importlib.import_module(module_name)
        if level == LigerKernelLevel.ALL:
            _patch(getattr(mod, norm_name), _rms_norm_forward)
        if mlp_name is not None:
            _patch(getattr(mod, mlp_name), _mlp_forward)


def restore_liger_kernel() -> None:
    """Put back every forward ``apply_liger_kernel`` replaced."""
    for (cls, name), fn in list(_saved.items()):
        setattr(cls, name, fn)
    _saved.clear()
