"""``blocked_seeded_dropout`` (lorafusion/ops/triton_ops/blocked_dropout.py:78-135) on the HIP mask kernel."""

from lorafusion_amd.ops.hip_ops import blocked_seeded_dropout  # noqa: F401
