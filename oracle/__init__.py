"""CPU oracle for the LoRA-linear hot path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``lorafusion_amd/`` may import this
package; only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline``
leg of ``bench.py`` use it, and only as the checker.

Contents (each function cites the reference file:line it restates):

* ``lora_ref``  -- unfused LoRA linear forward / closed-form backward, single
  adapter and segmented multi-adapter, with the dropout keep-mask explicit.
* ``routing``   -- the per-block routing tables of the multi-LoRA batch info.
* ``nf4``       -- NF4 block dequantisation (double-quantised absmax); the
  arithmetic lives in ``nf4_oracle.c`` (single-rounding ``fmaf``) with an
  exact-rational cross-check in Python.

Pinning status: every function here is pinned by CPU tests in
``tests/test_oracle_*.py`` against closed forms, autograd, finite differences,
brute force on tiny inputs and the reference's own worked example / constants.
The one exception is ``nf4.quantize_nf4`` and ``nf4.dynamic_code_table`` (the
reference takes both from bitsandbytes, which is neither vendored nor pinned):
**parity unpinned**; they only generate test inputs, and the dequantiser takes
their outputs as data.
"""
