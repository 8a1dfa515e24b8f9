"""``fused_lora_dyw_dsa`` (lorafusion/ops/triton_ops/fused_lora_dyw_dsa.py:184-297)."""

from lorafusion_amd.ops.hip_ops import fused_lora_dyw_dsa  # noqa: F401
