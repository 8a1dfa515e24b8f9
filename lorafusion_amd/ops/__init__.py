"""Mirror of ``lorafusion.ops``: the fused LoRA-linear ops and their kernel wrappers."""
