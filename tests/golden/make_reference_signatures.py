#!/usr/bin/env python3
"""Writes reference_signatures.json: the parameter lists of the reference's public ops on the
fused-LoRA path, read from its source files as text (``ast.parse``; nothing of the reference is
imported or run).  Usage: python tests/golden/make_reference_signatures.py /root/reference

Per function: the module of this package that mirrors it, the positional-or-keyword parameters in
order, the keyword-only parameters, the defaults (source text of the default expression), and
whether it takes *args / **kwargs.
"""

import ast
import json
import os
import sys

# reference file -> (mirror module in lorafusion_amd, function names)
PUBLIC = {
    "lorafusion/ops/lora_v1.py": ("lorafusion_amd.ops.lora_v1", ["fused_linear_lora"]),
    "lorafusion/ops/multi_lora.py": ("lorafusion_amd.ops.multi_lora", [
        "init_multi_lora_manager", "get_multi_lora_manager", "prepare_multi_lora_batch_info", "fused_linear_multi_lora"]),
    "lorafusion/ops/lora_torch_ref.py": ("lorafusion_amd.ops.lora_torch_ref", [
        "torch_ref_linear_lora", "torch_ref_linear_multi_lora"]),
    "lorafusion/ops/triton_ops/dropout.py": ("lorafusion_amd.ops.triton_ops.dropout", ["seeded_dropout"]),
    "lorafusion/ops/triton_ops/blocked_dropout.py": ("lorafusion_amd.ops.triton_ops.blocked_dropout", ["blocked_seeded_dropout"]),
    "lorafusion/ops/triton_ops/fused_dropout_matmul.py": ("lorafusion_amd.ops.triton_ops.fused_dropout_matmul", ["fused_dropout_matmul"]),
    "lorafusion/ops/triton_ops/fused_lora_xw_sb.py": ("lorafusion_amd.ops.triton_ops.fused_lora_xw_sb", ["fused_lora_xw_sb"]),
    "lorafusion/ops/triton_ops/fused_lora_dys_dyb.py": ("lorafusion_amd.ops.triton_ops.fused_lora_dys_dyb", ["fused_lora_dys_dyb"]),
    "lorafusion/ops/triton_ops/fused_lora_dyw_dsa.py": ("lorafusion_amd.ops.triton_ops.fused_lora_dyw_dsa", ["fused_lora_dyw_dsa"]),
    "lorafusion/ops/triton_ops/fused_multi_lora_xw_sb.py": ("lorafusion_amd.ops.triton_ops.fused_multi_lora_xw_sb", [
        "construct_s_and_b_ptrs_list", "fused_multi_lora_xw_sb"]),
    "lorafusion/ops/triton_ops/fused_multi_lora_dys_dyb.py": ("lorafusion_amd.ops.triton_ops.fused_multi_lora_dys_dyb", [
        "construct_s_and_b_ptrs_list", "fused_multi_lora_dys_dyb"]),
    "lorafusion/ops/triton_ops/fused_multi_lora_dyw_dsa.py": ("lorafusion_amd.ops.triton_ops.fused_multi_lora_dyw_dsa", [
        "construct_ds_and_a_ptrs_list", "fused_multi_lora_dyw_dsa"]),
    "lorafusion/ops/triton_ops/dequantize_nf4.py": ("lorafusion_amd.ops.triton_ops.dequantize_nf4", ["dequantize_nf4_triton"]),
    "lorafusion/ops/triton_ops/config.py": ("lorafusion_amd.ops.triton_ops.config", ["get_lora_kernel_config"]),
    "lorafusion/patch/patch_lora.py": ("lorafusion_amd.patch.patch_lora", ["lora_forward", "apply_lora"]),
    "lorafusion/utils/module.py": ("lorafusion_amd.utils.module", ["apply_liger_kernel"]),
}


def main(ref_root: str) -> None:
    out = []
    for rel, (mirror, names) in PUBLIC.items():
        with open(os.path.join(ref_root, rel)) as f:
            tree = ast.parse(f.read())
        found = {n.name: n for n in tree.body if isinstance(n, ast.FunctionDef)}
        for name in names:
            node = found[name]
            a = node.args
            pos = [x.arg for x in a.posonlyargs + a.args]
            defaults = {pos[len(pos) - len(a.defaults) + i]: ast.unparse(d) for i, d in enumerate(a.defaults)}
            defaults.update({k.arg: ast.unparse(d) for k, d in zip(a.kwonlyargs, a.kw_defaults) if d is not None})
            out.append({
                "reference": f"{rel}:{node.lineno}", "module": mirror, "name": name, "positional": pos,
                "keyword_only": [x.arg for x in a.kwonlyargs], "defaults": defaults,
                "var_positional": a.vararg is not None, "var_keyword": a.kwarg is not None,
            })
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_signatures.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1)
        f.write("\n")
    print(f"wrote {len(out)} signatures to {path}")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
