"""``fused_lora_xw_sb`` (lorafusion/ops/triton_ops/fused_lora_xw_sb.py:209-316)."""

from lorafusion_amd.ops.hip_ops import fused_lora_xw_sb  # noqa: F401
