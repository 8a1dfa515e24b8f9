"""Import-compatible aliases for ``lorafusion.ops.triton_ops``.

The reference keeps one Triton wrapper per module under this name; here the same module and
function names resolve to the HIP-backed wrappers in ``lorafusion_amd.ops.hip_ops`` / ``nf4``
(the multi-adapter wrappers with the reference's keyword signatures, see ``_multi_compat``).
"""

from lorafusion_amd.ops.hip_ops import (  # noqa: F401
    blocked_seeded_dropout,
    fused_dropout_matmul,
    fused_lora_da,
    fused_lora_dys_dyb,
    fused_lora_dyw_dsa,
    fused_lora_xw_sb,
    fused_multi_lora_da,
    fused_multi_lora_xa,
    seeded_dropout,
)
from lorafusion_amd.ops.triton_ops._multi_compat import (  # noqa: F401
    construct_ds_and_a_ptrs_list,
    construct_s_and_b_ptrs_list,
    fused_multi_lora_dys_dyb,
    fused_multi_lora_dyw_dsa,
    fused_multi_lora_xw_sb,
)
from lorafusion_amd.ops.multi_lora import get_lora_kernel_config  # noqa: F401
from lorafusion_amd.ops.nf4 import NF4_LUT, dequantize_nf4_triton  # noqa: F401
