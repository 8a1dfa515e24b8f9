"""The TMA twin of the reference (fused_lora_dyw_dsa_tma.py:221-388) is the same HIP kernel here."""

from lorafusion_amd.ops.hip_ops import fused_lora_dyw_dsa  # noqa: F401

fused_lora_dyw_dsa_tma = fused_lora_dyw_dsa
