"""MI355X-native LoRA-linear kernels behind the ``lorafusion.ops`` call signatures.

Sub-packages mirror the reference's module names: ``lorafusion_amd.ops.lora_v1``,
``lorafusion_amd.ops.multi_lora``, ``lorafusion_amd.ops.lora_torch_ref``,
``lorafusion_amd.ops.triton_ops`` (kernel-level wrappers; the name is kept so imports of
the reference map one-to-one, the kernels are HIP) and ``lorafusion_amd.patch.patch_lora``.
"""

__version__ = "0.1.0"
