"""The patch layer on the GPU: a duck-typed PEFT LoRA linear routed through ``lora_forward``.

Mirrors how lorafusion/patch/patch_lora.py:11-184 is used: ``apply_lora`` swaps the layer's forward, a
single adapter goes to the fused single op, several adapters registered with the ``MultiLoRAManager`` go
to the packed multi-adapter op; results are compared with the CPU oracle.  An NF4-packed base layer (as
bitsandbytes' Linear4bit stores it) exercises the QLoRA route.
"""

from __future__ import annotations

import numpy as np
import pytest
import torch
from torch import nn

from oracle import lora_ref
from oracle import nf4 as onf4
from tests.util import multi_inputs, single_inputs

pytestmark = pytest.mark.gpu


class FakeLoRALinear(nn.Module):
    """The attributes of peft.tuners.lora.Linear that the patch reads."""

    def __init__(self, w, adapters, bias=None, quant_state=None):
        super().__init__()
        self.base_layer = nn.Module()
        if quant_state is None:
            self.base_layer.weight = nn.Parameter(w, requires_grad=False)
        else:
            w.quant_state = quant_state          # packed uint8 codes + state, as Params4bit carries them
            self.base_layer.weight = w
        self.base_layer.bias = None if bias is None else nn.Parameter(bias, requires_grad=False)
        self.lora_A, self.lora_B, self.lora_dropout, self.scaling = nn.ModuleDict(), nn.ModuleDict(), nn.ModuleDict(), {}
        for name, (a, b, p, scale) in adapters.items():
            la = nn.Linear(a.shape[1], a.shape[0], bias=False)
            lb = nn.Linear(b.shape[1], b.shape[0], bias=False)
            la.weight, lb.weight = nn.Parameter(a.clone()), nn.Parameter(b.clone())
            self.lora_A[name], self.lora_B[name] = la, lb
            self.lora_dropout[name] = nn.Dropout(p) if p > 0 else nn.Identity()
            self.scaling[name] = scale


def _close(got, exp, name):
    ok, rel, excess = lora_ref.check_close(got.detach().float().cpu(), exp, rtol=1e-2)
    assert ok, f"{name}: rel {rel:.3e} excess {excess:.3e}"


def _nf4(w):
    st = onf4.quantize_nf4(w.float().numpy())
    wq = torch.from_numpy(onf4.dequantize(st).view(np.int16)).view(torch.bfloat16).reshape(w.shape)
    from lorafusion_amd.ops.nf4 import QuantState, QuantState2

    qs = QuantState(torch.Size(w.shape), torch.bfloat16, st.blocksize, torch.from_numpy(st.absmax).cuda(),
                    torch.from_numpy(st.offset).cuda(),
                    QuantState2(torch.from_numpy(st.absmax2).cuda(), torch.from_numpy(st.code2).cuda(), st.blocksize2))
    packed = torch.from_numpy(st.packed).cuda().reshape(-1, 1)     # bitsandbytes keeps the codes as [n/2, 1]
    return packed, qs, wq


@pytest.mark.parametrize("nf4", [False, True])
def test_single_adapter_layer(nf4):
    from lorafusion_amd.ops import multi_lora as ml
    from lorafusion_amd.patch import patch_lora

    ml.reset_multi_lora_manager()
    M, K, N, r, scale = 256, 512, 384, 16, 2.0
    d = single_inputs(M, K, N, r, p=0.0, seed=21, bias=True)
    w_ref, qs = d["w"], None
    w_dev = d["w"].cuda()
    if nf4:
        w_dev, qs, w_ref = _nf4(d["w"])
    layer = FakeLoRALinear(w_dev, {"default": (d["a"].cuda(), d["b"].cuda(), 0.0, scale)}, bias=d["bias"].cuda(),
                           quant_state=qs).cuda()
    patch_lora.apply_lora(target_cls=FakeLoRALinear)
    x = d["x"].reshape(2, M // 2, K).cuda().requires_grad_(True)       # 3-D input, as a transformer layer passes it
    y = layer(x)
    assert y.shape == (2, M // 2, N) and y.dtype == x.dtype
    y.backward(d["dy"].reshape(2, M // 2, N).cuda())
    ye, _ = lora_ref.linear_lora_fwd_fp32(d["x"], w_ref, d["a"], d["b"], scale, None, 0.0, bias=d["bias"])
    dxe, dae, dbe, _ = lora_ref.linear_lora_bwd_fp32(d["dy"], d["x"], w_ref, d["a"], d["b"], scale, None, 0.0)
    _close(y.reshape(M, N), ye, "y")
    _close(x.grad.reshape(M, K), dxe, "dx")
    _close(layer.lora_A["default"].weight.grad, dae, "da")
    _close(layer.lora_B["default"].weight.grad, dbe, "db")
    # the unfused route of the same layer agrees with the fused one
    y_ref = patch_lora.lora_forward(layer, x.detach(), use_fused=False)
    _close(y_ref.reshape(M, N), ye, "unfused y")
    # training mode with dropout: the fused op draws a Bernoulli(1-p) mask, so only the no-LoRA limit is exact
    layer.lora_dropout["default"] = nn.Dropout(0.5)
    layer.train()
    with torch.no_grad():
        layer.lora_B["default"].weight.zero_()
    yb = layer(x.detach())
    yb_e, _ = lora_ref.linear_lora_fwd_fp32(d["x"], w_ref, d["a"], torch.zeros_like(d["b"]), scale, None, 0.0, bias=d["bias"])
    _close(yb.reshape(M, N), yb_e, "y with B = 0 under dropout")
    with pytest.raises(TypeError):
        patch_lora.lora_forward(nn.Linear(4, 4), x)


@pytest.mark.parametrize("nf4", [False, True])
def test_multi_adapter_layer_through_manager(nf4):
    from lorafusion_amd.ops import multi_lora as ml
    from lorafusion_amd.patch import patch_lora

    seq, ranks, p_list, scales = [130, 57, 300], [16, 32, 16], [0.0, 0.0, 0.0], [1.0, 2.0, 0.5]
    idx = [0, 2, 3]                                   # adapters of this micro-batch out of four configured
    K, N = 512, 640
    d = multi_inputs(seq, K, N, ranks, p_list, seed=5, bias=True)
    w_ref, qs, w_dev = d["w"], None, d["w"].cuda()
    if nf4:
        w_dev, qs, w_ref = _nf4(d["w"])
    adapters = {f"lora_{i}": (a.cuda(), b.cuda(), 0.0, s) for i, a, b, s in zip(idx, d["a_list"], d["b_list"], scales)}
    spare = single_inputs(8, K, N, 16, seed=99)
    adapters["lora_1"] = (spare["a"].cuda(), spare["b"].cuda(), 0.0, 1.0)      # configured, idle in this micro-batch
    layer = FakeLoRALinear(w_dev, adapters, bias=d["bias"].cuda(), quant_state=qs).cuda()

    ml.reset_multi_lora_manager()
    mgr = ml.init_multi_lora_manager([object()] * 4, 1, None, [1] * 4)
    try:
        info = ml.prepare_multi_lora_batch_info(seq, idx, ranks, p_list, scales, 128, allow_empty_micro_batch_info=True)
        assert info.padded_seq_len_list == d["padded"]
        mgr.add_batch_info(info)
        Mp = sum(d["padded"])
        x = d["x"].cuda().reshape(1, Mp, K).requires_grad_(True)
        y = patch_lora.lora_forward(layer, x)
        mgr.mark_backward_pass_started()
        y.backward(d["dy"].cuda().reshape(1, Mp, N))
        ye, _ = lora_ref.linear_multi_lora_fwd_fp32(d["x"], w_ref, d["a_list"], d["b_list"], seq, d["padded"], scales,
                                                    p_list, None, bias=d["bias"])
        dxe, dae, dbe, _ = lora_ref.linear_multi_lora_bwd_fp32(d["dy"], d["x"], w_ref, d["a_list"], d["b_list"], seq,
                                                               d["padded"], scales, p_list, None)
        _close(y[0], ye, "y")
        _close(x.grad[0], dxe, "dx")
        for k, i in enumerate(idx):
            _close(layer.lora_A[f"lora_{i}"].weight.grad, dae[k], f"da[{i}]")
            _close(layer.lora_B[f"lora_{i}"].weight.grad, dbe[k], f"db[{i}]")
        assert layer.lora_A["lora_1"].weight.grad is None      # the idle adapter is untouched
        mgr.mark_forward_pass_started()
        y_ref = patch_lora.lora_forward(layer, x.detach(), use_fused=False)
        _close(y_ref[0], ye, "unfused y")
    finally:
        ml.reset_multi_lora_manager()
