"""Kernel configuration names of the reference (lorafusion/ops/triton_ops/config.py:14-152).

The HIP kernels choose their own tiles; the one value that is part of the data contract is the
routing block size.  ``LoRATritonConfig`` is accepted (and ignored apart from ``block_size_m``)
wherever the reference takes ``config=``.
"""

from __future__ import annotations

from dataclasses import dataclass

from lorafusion_amd.ops.multi_lora import get_lora_kernel_config  # noqa: F401


@dataclass
class LoRATritonConfig:
    block_size_m: int | None = None
    block_size_n: int | None = None
    block_size_k: int | None = None
    group_size_m: int | None = None
    num_stages: int | None = None
    num_warps: int | None = None
