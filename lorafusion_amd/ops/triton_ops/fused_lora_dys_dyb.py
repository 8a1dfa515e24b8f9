"""``fused_lora_dys_dyb`` (lorafusion/ops/triton_ops/fused_lora_dys_dyb.py:182-301)."""

from lorafusion_amd.ops.hip_ops import fused_lora_dys_dyb  # noqa: F401
