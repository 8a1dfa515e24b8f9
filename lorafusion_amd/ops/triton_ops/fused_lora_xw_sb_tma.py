"""The TMA twin of the reference (fused_lora_xw_sb_tma.py:244-392) is the same HIP kernel here."""

from lorafusion_amd.ops.hip_ops import fused_lora_xw_sb  # noqa: F401

fused_lora_xw_sb_tma = fused_lora_xw_sb
