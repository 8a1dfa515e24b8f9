"""``fused_multi_lora_dys_dyb`` with the reference's signature (fused_multi_lora_dys_dyb.py:21-57, 188-321)."""

from lorafusion_amd.ops.triton_ops._multi_compat import construct_s_and_b_ptrs_list, fused_multi_lora_dys_dyb  # noqa: F401
