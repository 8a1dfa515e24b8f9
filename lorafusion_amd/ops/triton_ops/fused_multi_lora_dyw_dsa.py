"""``fused_multi_lora_dyw_dsa`` with the reference's signature (fused_multi_lora_dyw_dsa.py:21-56, 188-305)."""

from lorafusion_amd.ops.triton_ops._multi_compat import construct_ds_and_a_ptrs_list, fused_multi_lora_dyw_dsa  # noqa: F401
