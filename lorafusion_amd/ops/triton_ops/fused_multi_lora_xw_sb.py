"""``fused_multi_lora_xw_sb`` with the reference's signature (fused_multi_lora_xw_sb.py:21-62, 221-339)."""

from lorafusion_amd.ops.triton_ops._multi_compat import construct_s_and_b_ptrs_list, fused_multi_lora_xw_sb  # noqa: F401
