"""Import-compatible aliases for ``lorafusion.ops.triton_ops``.

The reference keeps one Triton wrapper per module under this name; here the same function
names resolve to the HIP-backed wrappers in ``lorafusion_amd.ops.hip_ops`` / ``nf4``.
"""

from lorafusion_amd.ops.hip_ops import (  # noqa: F401
    fused_dropout_matmul,
    fused_lora_da,
    fused_lora_dys_dyb,
    fused_lora_dyw_dsa,
    fused_lora_xw_sb,
    fused_multi_lora_da,
    fused_multi_lora_dys_dyb,
    fused_multi_lora_dyw_dsa,
    fused_multi_lora_xa,
    fused_multi_lora_xw_sb,
    seeded_dropout,
)
from lorafusion_amd.ops.multi_lora import get_lora_kernel_config  # noqa: F401
from lorafusion_amd.ops.nf4 import NF4_LUT, dequantize_nf4_triton  # noqa: F401
