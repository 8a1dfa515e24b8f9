"""``fused_dropout_matmul`` (lorafusion/ops/triton_ops/fused_dropout_matmul.py:280-354)."""

from lorafusion_amd.ops.hip_ops import fused_dropout_matmul  # noqa: F401
