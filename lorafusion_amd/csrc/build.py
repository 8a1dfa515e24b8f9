"""Build liblorafusion_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

Usage: python -m lorafusion_amd.csrc.build   (or call build())
"""

from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
LIB = os.path.join(PKG, "liblorafusion_hip.so")
SOURCES = ["gemm_lora.hip", "gemm_big.hip", "lora_skinny.hip", "nf4_dequant.hip", "dropout_mask.hip", "norm_act.hip", "lf_api.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++20", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-inline-asm",
]


# sources whose kernels issue memory instructions from inline assembly: their generated code is checked for the
# hazards the compiler does not resolve there (asm_lint.py)
LINTED = ["gemm_big.hip", "gemm_lora.hip", "lora_skinny.hip"]


def _assembly(src: str) -> str:
    out = os.path.join(HERE, "build", src.replace(".hip", ".s"))
    cmd = ["hipcc", *FLAGS, "-S", "--cuda-device-only", os.path.join(HERE, src), "-o", out]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc -S failed on {src}:\n{res.stderr}")
    return out


def _compile(src: str) -> str:
    obj = os.path.join(HERE, "build", src.replace(".hip", ".o"))
    cmd = ["hipcc", *FLAGS, "-c", os.path.join(HERE, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = True) -> str:
    os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
    from lorafusion_amd.csrc.asm_lint import lint

    with ThreadPoolExecutor(max_workers=6) as ex:
        asm = [ex.submit(_assembly, s) for s in LINTED]
        objs = list(ex.map(_compile, SOURCES))
        hazards = [v for a in asm for v in lint(a.result())]
    if hazards:
        raise RuntimeError("hazards in generated code that inline assembly hides from the compiler:\n" + "\n".join(hazards))
    res = subprocess.run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-Wl,-z,defs", "-o", LIB, *objs],
                         capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    if verbose:
        print(f"built {LIB}")
    return LIB


if __name__ == "__main__":
    build()
