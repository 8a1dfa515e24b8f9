"""``dequantize_nf4_triton`` and the NF4 code table (lorafusion/ops/triton_ops/dequantize_nf4.py:16-33, 271-346)."""

from lorafusion_amd.ops.nf4 import NF4_LUT, dequantize_nf4_triton  # noqa: F401
