"""``seeded_dropout`` (lorafusion/ops/triton_ops/dropout.py:71-93) on the HIP mask kernel."""

from lorafusion_amd.ops.hip_ops import seeded_dropout  # noqa: F401
