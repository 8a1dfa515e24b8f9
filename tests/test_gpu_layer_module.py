"""A decoder layer's projections as four merged LoRA linears, driven by a scheduler micro-batch descriptor.

``DecoderLayerLoRAProjections`` (merged qkv, o, merged gate/up, down -- the merge of
lorafusion/patch/patch_transformers.py:50-163) runs a packed multi-adapter batch whose routing comes from
a ``MicroBatchInfo``-shaped descriptor (lorafusion/solver/proposed_solver.py:51-131) through
``batch_info_from_micro_batch`` and the ``MultiLoRAManager``.  Every linear is compared with the CPU oracle
(rtol 1e-2, atol 1e-2*rms, fp32-accumulated), the merged outputs with the separate projections they stand
for, and the routing of the micro-batch must be built exactly once for the whole layer.
"""

from __future__ import annotations

import math
from types import SimpleNamespace

import pytest
import torch

from oracle import lora_ref

pytestmark = pytest.mark.gpu

HIDDEN, KV, MLP = 512, 128, 1024
BLOCK = 128


def _close(got, exp, name):
    ok, rel, excess = lora_ref.check_close(got.detach().float().cpu(), exp, rtol=1e-2)
    assert ok, f"{name}: max|err|/max|e| = {rel:.3e}, worst excess over bound {excess:.3e}"


def _descriptor(tokens: dict[int, int]):
    """The fields of MicroBatchInfo that the routing and the manager read."""
    return SimpleNamespace(
        adapter_group_info=set(tokens), adapter_num_tokens_pairs=dict(tokens),
        padded_adapter_num_tokens_pairs={a: ((n - 1) // BLOCK + 1) * BLOCK for a, n in tokens.items()},
        adapter_num_samples_pairs={a: 1 for a in tokens}, adapter_padding_multiple=BLOCK, is_empty_marker=False)


def _randomise_lora(layer, seed):
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for lin in layer.linears().values():
            for name in lin.lora_A:
                a, b = lin.lora_A[name].weight, lin.lora_B[name].weight
                a.copy_(((torch.rand(a.shape, generator=g) * 2 - 1) / math.sqrt(a.shape[1])).to(a.dtype))
                b.copy_((torch.randn(b.shape, generator=g) * 0.01).to(b.dtype))


@pytest.fixture
def manager():
    from lorafusion_amd.ops import multi_lora as ml

    ml.reset_multi_lora_manager()
    yield ml
    ml.reset_multi_lora_manager()


def test_layer_linears_from_descriptor(manager, monkeypatch):
    ml = manager
    from lorafusion_amd.ops import hip_ops
    from lorafusion_amd.patch.patch_transformers import DecoderLayerLoRAProjections

    # four adapters configured, three in this micro-batch; the multiplier handed to the kernels is lora_alpha
    # itself, as the reference's data provider does (lorafusion/train/training_utils.py:1323)
    cfgs = [SimpleNamespace(r=r, lora_alpha=al, lora_dropout=0.0) for r, al in ((16, 2.0), (32, 1.0), (16, 0.5), (8, 4.0))]
    adapters = {f"lora_{i}": (c.r, c.lora_alpha, c.lora_dropout) for i, c in enumerate(cfgs)}
    layer = DecoderLayerLoRAProjections.from_shapes(HIDDEN, KV, MLP, adapters, seed=3)
    _randomise_lora(layer, seed=4)
    tokens = {3: 150, 0: 300, 1: 129}
    mb = _descriptor(tokens)

    built = []
    orig_init = hip_ops.MultiRouting.__init__

    def counting_init(self, *a, **k):
        built.append(1)
        orig_init(self, *a, **k)

    monkeypatch.setattr(hip_ops.MultiRouting, "__init__", counting_init)
    mgr = ml.init_multi_lora_manager(cfgs, 1, None, [1] * len(cfgs))
    info = ml.batch_info_from_micro_batch(mb, cfgs)
    mgr.add_batch_info(info)
    assert info.lora_idx_list == [0, 1, 3] and info.seq_len_list == [300, 129, 150]
    assert info.block_to_alpha.dtype == torch.bfloat16           # the reference's storage type
    seq, padded = info.seq_len_list, info.padded_seq_len_list
    Mp = sum(padded)
    scales = [cfgs[i].lora_alpha for i in info.lora_idx_list]
    p_list = [0.0] * len(seq)

    g = torch.Generator().manual_seed(11)
    for name, lin in layer.linears().items():
        K, N = lin.in_features, lin.out_features
        x = torch.randn(Mp, K, generator=g).to(torch.bfloat16)
        dy = torch.randn(Mp, N, generator=g).to(torch.bfloat16)
        xd = x.cuda().reshape(1, Mp, K).requires_grad_(True)
        mgr.mark_forward_pass_started()
        y = lin(xd)
        mgr.mark_backward_pass_started()
        y.backward(dy.cuda().reshape(1, Mp, N))
        torch.cuda.synchronize()
        a_list = [lin.lora_A[f"lora_{i}"].weight.detach().cpu() for i in info.lora_idx_list]
        b_list = [lin.lora_B[f"lora_{i}"].weight.detach().cpu() for i in info.lora_idx_list]
        w = lin.base_layer.weight.detach().cpu()
        ye, _ = lora_ref.linear_multi_lora_fwd_fp32(x, w, a_list, b_list, seq, padded, scales, p_list, None)
        dxe, dae, dbe, _ = lora_ref.linear_multi_lora_bwd_fp32(dy, x, w, a_list, b_list, seq, padded, scales, p_list, None)
        _close(y[0], ye, f"{name}: y")
        _close(xd.grad[0], dxe, f"{name}: dx")
        for j, i in enumerate(info.lora_idx_list):
            _close(lin.lora_A[f"lora_{i}"].weight.grad, dae[j], f"{name}: da[{i}]")
            _close(lin.lora_B[f"lora_{i}"].weight.grad, dbe[j], f"{name}: db[{i}]")
        # the idle adapter got no gradient
        assert lin.lora_A["lora_2"].weight.grad is None
    assert len(built) == 1, f"the routing of one micro-batch was built {len(built)} times for four linears"


def test_linear_driven_by_a_schedule_file(manager, tmp_path):
    """A JSON schedule of two micro-batches (grouped in one step, as the reference's planner groups them) is loaded
    and drives a multi-adapter LoRA linear micro-batch by micro-batch: forward and backward of each against the
    oracle, gradients accumulated over both, sample counts tallied by the manager."""
    ml = manager
    from lorafusion_amd.ops import schedule as sch
    from lorafusion_amd.patch.patch_transformers import DecoderLayerLoRAProjections

    cfgs = [SimpleNamespace(r=r, lora_alpha=al, lora_dropout=0.0) for r, al in ((16, 2.0), (64, 1.0), (8, 4.0))]
    adapters = {f"lora_{i}": (c.r, c.lora_alpha, c.lora_dropout) for i, c in enumerate(cfgs)}
    layer = DecoderLayerLoRAProjections.from_shapes(HIDDEN, KV, MLP, adapters, seed=7)
    _randomise_lora(layer, seed=8)
    lin = layer.linears()["down"]
    K, N = lin.in_features, lin.out_features
    steps = [{"micro_batch_infos": [
        {"data_samples": [[2, 0, 0, 100], [0, 0, 1, 77], [2, 0, 2, 60], [1, 0, 3, 200]],
         "max_microbatch_size": 1024, "adapter_padding_multiple": BLOCK, "micro_batch_idx": 0},
        {"data_samples": [[1, 1, 4, 128], [1, 1, 5, 1]],
         "max_microbatch_size": 1024, "adapter_padding_multiple": BLOCK, "micro_batch_idx": 1}]}]
    path = tmp_path / "schedule.json"
    path.write_text(__import__("json").dumps(steps))
    mbs = sch.load_schedule(path)
    assert [mb.padded_total_tokens for mb in mbs] == [256 + 128 + 256, 256]

    mgr = ml.init_multi_lora_manager(cfgs, 1, 1024, [2, 2, 2])
    g = torch.Generator().manual_seed(21)
    exp_da = {i: torch.zeros(c.r, K) for i, c in enumerate(cfgs)}
    exp_db = {i: torch.zeros(N, c.r) for i, c in enumerate(cfgs)}
    w = lin.base_layer.weight.detach().cpu()
    for mb in mbs:
        info = ml.batch_info_from_micro_batch(mb, cfgs)
        mgr.add_batch_info(info)
        seq, padded = info.seq_len_list, info.padded_seq_len_list
        assert seq == [mb.adapter_num_tokens_pairs[i] for i in info.lora_idx_list]
        Mp = sum(padded)
        assert Mp == mb.padded_total_tokens
        x = torch.randn(Mp, K, generator=g).to(torch.bfloat16)
        dy = torch.randn(Mp, N, generator=g).to(torch.bfloat16)
        xd = x.cuda().reshape(1, Mp, K).requires_grad_(True)
        mgr.mark_forward_pass_started()
        y = lin(xd)
        mgr.mark_backward_pass_started()
        y.backward(dy.cuda().reshape(1, Mp, N))
        torch.cuda.synchronize()
        mgr.pop_oldest_batch_info()
        a_list = [lin.lora_A[f"lora_{i}"].weight.detach().cpu() for i in info.lora_idx_list]
        b_list = [lin.lora_B[f"lora_{i}"].weight.detach().cpu() for i in info.lora_idx_list]
        scales = [cfgs[i].lora_alpha for i in info.lora_idx_list]
        p_list = [0.0] * len(seq)
        if len(seq) == 1:
            # one active adapter: the reference takes the single-adapter op with the layer's own scaling
            # (lora_alpha / r) over every row of the padded batch (lorafusion/patch/patch_lora.py:90-117)
            sc = lin.scaling[f"lora_{info.lora_idx_list[0]}"]
            ye, _ = lora_ref.linear_lora_fwd_fp32(x, w, a_list[0], b_list[0], sc)
            dxe, da1, db1, _ = lora_ref.linear_lora_bwd_fp32(dy, x, w, a_list[0], b_list[0], sc)
            dae, dbe = [da1], [db1]
        else:
            ye, _ = lora_ref.linear_multi_lora_fwd_fp32(x, w, a_list, b_list, seq, padded, scales, p_list, None)
            dxe, dae, dbe, _ = lora_ref.linear_multi_lora_bwd_fp32(dy, x, w, a_list, b_list, seq, padded, scales, p_list, None)
        _close(y[0], ye, f"micro-batch {mb.micro_batch_idx}: y")
        _close(xd.grad[0], dxe, f"micro-batch {mb.micro_batch_idx}: dx")
        for j, i in enumerate(info.lora_idx_list):
            exp_da[i] += dae[j]
            exp_db[i] += dbe[j]
    for i in range(len(cfgs)):
        _close(lin.lora_A[f"lora_{i}"].weight.grad, exp_da[i], f"accumulated da[{i}]")
        _close(lin.lora_B[f"lora_{i}"].weight.grad, exp_db[i], f"accumulated db[{i}]")
    assert mgr.adapter_sample_counts == {0: 1, 1: 3, 2: 2}


def test_merged_projections_equal_the_separate_ones(manager):
    """qkv and gate/up as one GEMM each: the column slices are the separate projections' outputs (same base
    weights, no LoRA contribution with B = 0), bit for bit against the plain GEMM of each weight."""
    from lorafusion_amd.ops import hip_ops
    from lorafusion_amd.patch.patch_transformers import DecoderLayerLoRAProjections, merge_linears

    adapters = {"default": (16, 32.0, 0.0)}
    layer = DecoderLayerLoRAProjections.from_shapes(HIDDEN, KV, MLP, adapters, seed=5)
    assert layer.qkv_proj.proj.out_features == HIDDEN + 2 * KV and layer.gate_up_proj.proj.out_features == 2 * MLP
    x = torch.randn(384, HIDDEN, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16).cuda()
    q, k, v = layer.qkv_proj(x)
    assert q.shape == (384, HIDDEN) and k.shape == v.shape == (384, KV)
    w = layer.qkv_proj.proj.base_layer.weight
    for got, rows in ((q, slice(0, HIDDEN)), (k, slice(HIDDEN, HIDDEN + KV)), (v, slice(HIDDEN + KV, HIDDEN + 2 * KV))):
        exp = x.float().cpu() @ w[rows].float().cpu().T
        _close(got, exp, "merged qkv slice")
    # biases: a missing one among biased layers counts as zero
    a, b = torch.nn.Linear(8, 4, bias=True), torch.nn.Linear(8, 2, bias=False)
    m = merge_linears([a, b])
    assert torch.equal(m.weight[:4], a.weight) and torch.equal(m.weight[4:], b.weight)
    assert torch.equal(m.bias[:4], a.bias) and torch.count_nonzero(m.bias[4:]) == 0
    # the whole harness: shapes, and gradients reach every adapter of every linear
    layer.train()
    for lin in layer.linears().values():
        torch.nn.init.normal_(lin.lora_B["default"].weight, std=0.01)
    h = x.clone().requires_grad_(True)
    out = layer(h)
    assert out.shape == (384, HIDDEN) and torch.isfinite(out.float()).all()
    out.float().square().mean().backward()
    assert h.grad is not None and torch.isfinite(h.grad.float()).all()
    for name, lin in layer.linears().items():
        for t in (lin.lora_A["default"].weight, lin.lora_B["default"].weight):
            assert t.grad is not None and torch.count_nonzero(t.grad) > 0, name
    assert hip_ops is not None
