"""CPU-side checks: the C-ABI library loads, exports every symbol the header declares, rejects bad
arguments before touching a GPU, and the Python layer fails loudly without a GPU / without the library."""

import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "lorafusion_hip.h")).read()
    return sorted(set(re.findall(r"\b(lf_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from lorafusion_amd import _lib

    lib = _lib.lib()
    declared = _declared_symbols()
    assert set(declared) == set(_lib.EXPORTS), (declared, _lib.EXPORTS)
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.lf_version() >= 1
    assert b"workspace" in lib.lf_strerror(-3)
    assert lib.lf_strerror(0) == b"ok"


def test_routing_struct_layout_matches_header():
    from lorafusion_amd import _lib

    # 4 int32 + 3 pointers + 2 floats + 2 x 32 int32
    assert ctypes.sizeof(_lib.Routing) == 16 + 24 + 8 + 2 * 4 * _lib.LF_MAX_SEG
    r = _lib.single_routing(16, 2.0, 0.1)
    assert r.n_seg == 1 and r.seg_rank[0] == 16 and abs(r.p - 0.1) < 1e-7
    # struct lf_nf4_weight: 5 pointers + 2 int32 + the optional dense buffer (pointer + 2 int32)
    assert ctypes.sizeof(_lib.NF4Weight) == 5 * 8 + 2 * 4 + 8 + 2 * 4


def test_argument_validation_without_gpu():
    """Error paths return codes before any launch (null pointers / bad shapes never reach a kernel)."""
    from lorafusion_amd import _lib

    lib = _lib.lib()
    r = _lib.single_routing(16, 1.0, 0.0)
    ptrs = (ctypes.c_void_p * 1)()
    # null tensors
    assert lib.lf_lora_xw_sb(None, None, None, None, ptrs, None, 128, 128, 128, 16, r, 0, None) == -1
    assert lib.lf_nf4_dequant(None, None, None, None, None, None, 64, 64, 0, 0, None) == -1
    assert lib.lf_gemm(None, None, None, None, 128, 128, 128, 1, 0, -1, None) == -1
    # unknown dtype
    one = ctypes.c_void_p(16)
    assert lib.lf_gemm(one, one, None, one, 128, 128, 128, 1, 7, -1, None) == -1
    # workspace sizes are positive and grow with the problem
    small = lib.lf_workspace_bytes(_lib.LF_OP_BWD, 256, 256, 256, 16, r)
    big = lib.lf_workspace_bytes(_lib.LF_OP_BWD, 4096, 4096, 4096, 16, r)
    assert 0 < small < big and small % 256 == 0
    # bad routing: rank not a multiple of 8, too many segments
    bad = _lib.single_routing(12, 1.0, 0.0)
    assert lib.lf_workspace_bytes(_lib.LF_OP_FWD, 256, 256, 256, 16, bad) == 0
    # NF4 entry points: the workspace holds the dequantised weight ahead of the op's own scratch
    wbytes = 256 * 256 * 2
    assert lib.lf_workspace_bytes(_lib.LF_OP_NF4_FWD, 256, 256, 256, 16, r) == wbytes + lib.lf_workspace_bytes(_lib.LF_OP_FWD, 256, 256, 256, 16, r)
    assert lib.lf_workspace_bytes(_lib.LF_OP_NF4_BWD, 256, 256, 256, 16, r) == wbytes + small
    wq = _lib.NF4Weight(16, 16, None, None, None, 64, 0, None, 0, 0)
    args_fwd = (one, ctypes.byref(wq), None, None, ptrs, ptrs, one, one)
    assert lib.lf_nf4_lora_fwd(*args_fwd, None, 0, 256, 256, 256, 16, r, 0, None) == -3           # no workspace
    assert lib.lf_nf4_lora_fwd(*args_fwd, ctypes.c_void_p(256), 100, 256, 256, 256, 16, r, 0, None) == -3   # too small
    assert lib.lf_nf4_lora_fwd(one, None, None, None, ptrs, ptrs, one, one, ctypes.c_void_p(256), 1 << 20, 256, 256, 256, 16, r, 0, None) == -1
    bad2 = _lib.single_routing(16, 1.0, 0.0)
    bad2.n_seg = 64
    assert lib.lf_lora_xa(one, None, ptrs, one, one, 1 << 20, 128, 128, 16, bad2, 0, None) == -5


def test_size_query_and_static_backward_refuse_untiled_shapes():
    """A tiled dimension below the tile (or R the passes do not take) must come back as a code, not as a host crash:
    the planners divide by the number of 64-column tiles."""
    from lorafusion_amd import _lib

    lib = _lib.lib()
    r = _lib.single_routing(16, 1.0, 0.0)
    for bad in (0, 32, 64, 192):
        assert lib.lf_workspace_bytes(_lib.LF_OP_BWD, 256, bad, 256, 16, r) == 0
        assert lib.lf_workspace_bytes(_lib.LF_OP_BWD, 256, 256, bad, 16, r) == 0
        assert lib.lf_workspace_bytes(_lib.LF_OP_DYS_DYB, 256, bad, 0, 16, r) == 0
        assert lib.lf_workspace_bytes(_lib.LF_OP_DA, 256, 0, bad, 16, r) == 0
        assert lib.lf_workspace_bytes(_lib.LF_OP_NF4_BWD, 256, bad, 256, 16, r) == 0
    # the dimension an op does not tile may be anything
    assert lib.lf_workspace_bytes(_lib.LF_OP_DYS_DYB, 256, 256, 0, 16, r) > 0
    assert lib.lf_workspace_bytes(_lib.LF_OP_DA, 256, 0, 256, 16, r) > 0
    for bad_r in (0, 8, 24, 144):
        assert lib.lf_workspace_bytes(_lib.LF_OP_BWD, 256, 256, 256, bad_r, r) == 0
    assert lib.lf_workspace_bytes(_lib.LF_OP_BWD, 0, 256, 256, 16, r) == 0
    one = ctypes.c_void_p(256)
    ptrs = (ctypes.c_void_p * 1)(256)
    call = lambda M, N, K, R, dt=0, dy=one: lib.lf_lora_bwd_static(dy, one, one, None, one, ptrs, ptrs, one, ptrs, ptrs, one, M, N, K, R, r, dt, None)
    for bad in (32, 64, 192):
        assert call(256, bad, 256, 16) == _lib.LF_ESHAPE
        assert call(256, 256, bad, 16) == _lib.LF_ESHAPE
    assert call(256, 256, 256, 24) == _lib.LF_ESHAPE
    assert call(256, 256, 256, 144) == _lib.LF_ESHAPE
    assert call(256, 0, 256, 16) == _lib.LF_EINVAL
    assert call(256, 256, 256, 16, dt=7) == _lib.LF_EINVAL       # dtype and pointers are looked at first
    assert call(256, 256, 256, 16, dy=None) == _lib.LF_EINVAL


def test_launch_plan_takes_the_contraction_length():
    """Host logic of the tile choice: left-over rows get a launch of their own when the contraction is long enough to
    pay for it, and one launch covers everything when it is short."""
    import ctypes

    from lorafusion_amd import _lib as L

    def plan(M, N, K, block=128):
        rows, head, tail = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        assert L.lib().lf_gemm_plan(M, N, K, block, ctypes.byref(rows), ctypes.byref(head), ctypes.byref(tail)) == 0
        return rows.value, head.value, tail.value

    # 16512 rows = 64 tile rows of 256 and 128 more: the persistent kernel takes the 64, a small tile the rest
    for N, K in [(6144, 4096), (4096, 6144), (28672, 4096), (4096, 28672), (4096, 14336), (14336, 4096)]:
        rows, head, tail = plan(16512, N, K)
        assert (rows, head) == (16384, 7) and tail in (4, 5, 6)
    for K in (128, 256, 512):
        assert plan(16512, 4096, K) == (16512, 7, -1)
    assert plan(2048, 4096, 4096)[0] == 2048        # nothing left over: one launch
    assert L.lib().lf_gemm_plan(16, 16, 0, 0, None, None, None) == L.LF_EINVAL
    # The persistent kernel's 128x256 tile (8) takes single launches between half a round and one round of its tiles
    # on 256 compute units; fewer rows go to small tiles, more to its 256x256 tile (7), left-over rows never to 8.
    assert plan(2048, 4096, 4096) == (2048, 8, -1) and plan(1536, 4096, 6144) == (1536, 8, -1)
    assert plan(1024, 4096, 4096)[1] not in (7, 8)
    assert plan(4096, 4096, 4096) == (4096, 7, -1) and plan(2048, 8192, 8192) == (2048, 7, -1)
    assert plan(2048, 4096, 128)[1] != 8            # its K loop needs four steps of 64
    for M in (8448, 8576, 16512, 16640):
        for N, K in [(4096, 4096), (8192, 8192), (57344, 8192), (10240, 8192)]:
            assert plan(M, N, K)[2] != 8
    # a long contraction under a wide output: the eight-wave 256x256 tile (1), not the persistent kernel
    assert plan(8192, 8192, 28672) == (8192, 1, -1) and plan(8576, 8192, 28672)[:2] == (8192, 1)
    assert plan(8192, 8192, 8192)[1] == 7 and plan(16384, 4096, 28672)[1] == 7


def test_python_layer_refuses_cpu_tensors():
    from lorafusion_amd.ops.lora_v1 import fused_linear_lora
    from lorafusion_amd.ops.nf4 import QuantState, dequantize_nf4_triton

    x = torch.zeros(128, 128, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="GPU"):
        fused_linear_lora(x, x, x[:16], x[:, :16].contiguous(), 1.0)
    with pytest.raises(ValueError, match="GPU"):
        dequantize_nf4_triton(torch.zeros(64, dtype=torch.uint8),
                              QuantState(torch.Size([128]), torch.bfloat16, 64, torch.ones(2)))


def test_missing_library_is_fatal(monkeypatch):
    from lorafusion_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", os.path.join(ROOT, "does_not_exist.so"))
    with pytest.raises(RuntimeError, match="no non-HIP fallback"):
        _lib.lib()


def test_product_does_not_import_oracle():
    for dirpath, _, files in os.walk(os.path.join(ROOT, "lorafusion_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "import oracle" not in text and "from oracle" not in text, f


def test_manager_and_patch_host_logic():
    from lorafusion_amd.ops import multi_lora as ml
    from lorafusion_amd.patch import patch_lora

    ml.reset_multi_lora_manager()
    with pytest.raises(ValueError, match="multi_lora_global_batch_sizes is not provided"):
        ml.init_multi_lora_manager([object(), object()], 2, None)   # as lorafusion/ops/multi_lora.py:92-94
    with pytest.raises(ValueError, match="Expected 2 batch sizes"):
        ml.MultiLoRAManager([object(), object()], 2, None, [8])
    assert ml.get_multi_lora_manager() is None
    mgr = ml.init_multi_lora_manager([object(), object()], 2, None, [8, 8])
    with pytest.raises(ValueError):
        ml.init_multi_lora_manager([object()], 1, None, [8])
    info_a = ml.prepare_multi_lora_batch_info([5], [0], [16], [0.0], [1.0], 128, allow_empty_micro_batch_info=True)
    info_b = ml.prepare_multi_lora_batch_info([7], [1], [16], [0.0], [1.0], 128, allow_empty_micro_batch_info=True)
    mgr.add_batch_info(info_a)
    mgr.add_batch_info(info_b)
    with pytest.raises(ValueError):
        mgr.add_batch_info(info_b)   # deque is full
    assert mgr.get_newest_batch_info() is info_b and mgr.get_oldest_batch_info() is info_a
    assert info_a.microbatch_idx == 0 and info_b.microbatch_idx == 1
    mgr.mark_backward_pass_started()
    assert not mgr.is_in_forward
    assert mgr.pop_oldest_batch_info() is info_a
    mgr.mark_forward_pass_started()
    assert mgr.is_in_forward
    strict = ml.prepare_multi_lora_batch_info([7], [1], [16], [0.0], [1.0], 128)
    with pytest.raises(ValueError):
        mgr.add_batch_info(strict)   # MicroBatchInfo missing and not allowed to be empty
    ml.reset_multi_lora_manager()
    with pytest.raises(TypeError):
        patch_lora.lora_forward(object(), torch.zeros(1))
    assert ml.get_lora_kernel_config("fused_multi_lora_block_size_m") == 128
    with pytest.raises(ValueError):
        ml.get_lora_kernel_config("fused_lora_xw_sb")


def test_torch_ref_path_matches_oracle_on_cpu():
    """The unfused (use_fused=False) product path is plain torch and runs on CPU."""
    from lorafusion_amd.ops.lora_torch_ref import torch_ref_linear_lora, torch_ref_linear_multi_lora
    from oracle import lora_ref
    from tests.util import multi_inputs, single_inputs

    d = single_inputs(32, 64, 48, 8, p=0.0, seed=0, dtype=torch.float32, bias=True)
    y = torch_ref_linear_lora(d["x"], d["w"], d["a"], d["b"], 2.0, 0.0, d["bias"])
    ye, _ = lora_ref.linear_lora_fwd_fp32(d["x"], d["w"], d["a"], d["b"], 2.0, None, 0.0, d["bias"])
    assert torch.allclose(y, ye, atol=1e-5)
    seq = [5, 9]
    m = multi_inputs(seq, 64, 48, [8, 16], [0.0, 0.0], dtype=torch.float32, block=8)
    ym = torch_ref_linear_multi_lora(m["x"].unsqueeze(0), m["w"], lora_a_list=m["a_list"], lora_b_list=m["b_list"],
                                     seq_len_list=seq, padded_seq_len_list=m["padded"], alpha_list=[1.0, 2.0],
                                     dropout_p_list=[0.0, 0.0])
    yme, _ = lora_ref.linear_multi_lora_fwd_fp32(m["x"], m["w"], m["a_list"], m["b_list"], seq, m["padded"],
                                                 [1.0, 2.0], [0.0, 0.0])
    assert torch.allclose(ym[0], yme, atol=1e-5)


def test_reference_module_and_function_names_resolve():
    """A user of the reference swaps the package prefix: every module of lorafusion.ops on the hot path
    and its public entry points exist under lorafusion_amd.ops with the same names."""
    import importlib

    names = {
        "lora_v1": ["fused_linear_lora", "FusedLinearLoRA"],
        "multi_lora": ["fused_linear_multi_lora", "FusedLinearMultiLoRA", "prepare_multi_lora_batch_info",
                       "MultiLoRABatchInfo", "MultiLoRAManager", "init_multi_lora_manager", "get_multi_lora_manager"],
        "lora_torch_ref": ["torch_ref_linear_lora", "torch_ref_linear_multi_lora"],
        "triton_ops.dropout": ["seeded_dropout"],
        "triton_ops.blocked_dropout": ["blocked_seeded_dropout"],
        "triton_ops.fused_dropout_matmul": ["fused_dropout_matmul"],
        "triton_ops.fused_lora_xw_sb": ["fused_lora_xw_sb"],
        "triton_ops.fused_lora_xw_sb_tma": ["fused_lora_xw_sb_tma"],
        "triton_ops.fused_lora_dys_dyb": ["fused_lora_dys_dyb"],
        "triton_ops.fused_lora_dyw_dsa": ["fused_lora_dyw_dsa"],
        "triton_ops.fused_lora_dyw_dsa_tma": ["fused_lora_dyw_dsa_tma"],
        "triton_ops.fused_multi_lora_xw_sb": ["fused_multi_lora_xw_sb", "construct_s_and_b_ptrs_list"],
        "triton_ops.fused_multi_lora_dys_dyb": ["fused_multi_lora_dys_dyb", "construct_s_and_b_ptrs_list"],
        "triton_ops.fused_multi_lora_dyw_dsa": ["fused_multi_lora_dyw_dsa", "construct_ds_and_a_ptrs_list"],
        "triton_ops.dequantize_nf4": ["dequantize_nf4_triton", "NF4_LUT"],
        "triton_ops.config": ["get_lora_kernel_config", "LoRATritonConfig"],
    }
    for mod, syms in names.items():
        m = importlib.import_module("lorafusion_amd.ops." + mod)
        for s in syms:
            assert hasattr(m, s), f"lorafusion_amd.ops.{mod}.{s} is missing"
    assert importlib.import_module("lorafusion_amd.patch.patch_lora").apply_lora


def test_workspace_sizes_of_the_rank_r_passes_stay_bounded():
    """The scratch of the backward passes holds fp32 partial sums: one [rows, R] slab per slice of the streamed
    matrix's columns and one [N, R] (or [R, K]) slab per chunk of an adapter's row blocks.  The split that sizes it is
    host logic (no GPU): for every shape it must give a multiple of 256 bytes that is at least one slab of each kind
    and stays below a few times the streamed operand (a split that cut every block into its own chunk did not)."""
    import torch

    from lorafusion_amd import _lib

    lib = _lib.lib()

    def routing(padded, ranks):
        nb = sum(padded) // 128
        table = torch.zeros((nb, 3), dtype=torch.int32)      # host pointers are only stored, never read on the CPU
        scale = torch.ones(nb)
        p = torch.zeros(nb)
        return _lib.multi_routing(padded, ranks, table, scale, p, 128), (table, scale, p)

    cases = []
    for R in (16, 32, 48, 64, 128):
        for (M, N, K) in ((1, 128, 128), (300, 256, 128), (2048, 4096, 4096), (8448, 4096, 4096), (16512, 28672, 4096),
                          (8576, 57344, 8192), (8576, 8192, 28672)):
            cases.append((_lib.single_routing(R, 2.0, 0.1), None, M, N, K, R, 1))
    for padded, ranks in (([1152, 640, 1152, 768, 512, 896, 1920, 1536], [64] * 8), ([2688, 4480, 4608, 4736], [16] * 4),
                          ([128] * 32, [16, 32] * 16), ([128, 8192, 128], [8, 64, 16])):
        r, keep = routing(padded, ranks)
        M, R = sum(padded), _lib.round_rank(max(ranks))
        for (N, K) in ((4096, 4096), (57344, 8192), (128, 128)):
            cases.append((r, keep, M, N, K, R, len(padded)))
    for r, keep, M, N, K, R, nseg in cases:
        rows = (M + 127) // 128 * 128
        dys = lib.lf_workspace_bytes(_lib.LF_OP_DYS_DYB, M, N, K, R, ctypes.byref(r))
        da = lib.lf_workspace_bytes(_lib.LF_OP_DA, M, N, K, R, ctypes.byref(r))
        bwd = lib.lf_workspace_bytes(_lib.LF_OP_BWD, M, N, K, R, ctypes.byref(r))
        assert dys % 256 == 0 and da % 256 == 0 and bwd == max(dys, da), (M, N, K, R)
        assert dys >= (M * R + nseg * N * R) * 4 and da >= nseg * R * K * 4, (M, N, K, R, dys, da)
        # partial sums written and read once stay within a few times the operand they are the sums of (tiny problems:
        # a few slabs of each kind are the floor)
        assert dys <= max(4 * rows * N * 2, 4 * (rows * R + nseg * N * R) * 4 + 4096), (M, N, K, R, dys)
        assert da <= max(4 * rows * K * 3, 4 * nseg * R * K * 4 + 4096), (M, N, K, R, da)
