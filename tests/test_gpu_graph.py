"""The C entry points under HIP graph capture: they allocate nothing, record no memset and never
synchronise, so a forward + backward can be captured once and replayed.  Every replay is compared
with the eager result on fresh input values (replays 2 and 3 are where a stale node would show)."""

from __future__ import annotations

import pytest
import torch

from tests.util import multi_inputs

pytestmark = pytest.mark.gpu


def test_forward_backward_replay_matches_eager():
    from lorafusion_amd.ops import hip_ops
    from lorafusion_amd.ops.multi_lora import prepare_multi_lora_batch_info

    seq, ranks, p_list, scales = [300, 140, 77], [16, 32, 16], [0.1, 0.0, 0.05], [2.0, 1.0, 0.5]
    K, N = 512, 768
    d = multi_inputs(seq, K, N, ranks, p_list, seed=3)
    info = prepare_multi_lora_batch_info(seq, [0, 1, 2], ranks, p_list, scales, 128, output_dtype=torch.float32)
    routing = hip_ops.MultiRouting(info.padded_seq_len_list, ranks, info.block_to_lookup_table, info.block_to_alpha,
                                   info.block_to_dropout_p)
    x, w, dy, mask = d["x"].cuda(), d["w"].cuda(), d["dy"].cuda(), d["mask"].cuda()
    a_list, b_list = [a.cuda() for a in d["a_list"]], [b.cuda() for b in d["b_list"]]

    def run():
        y, s = hip_ops.lora_forward(x, w, a_list, b_list, routing.c, routing.R, mask, None)
        dx, da, db = hip_ops.lora_backward(dy, x, w, a_list, b_list, s, routing.c, routing.R, mask, ranks)
        return [y, dx, *da, *db]

    run()                                  # first call: kernel attributes are set outside the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        run()
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            outs = run()
    torch.cuda.synchronize()
    gen = torch.Generator(device="cuda").manual_seed(7)
    for replay in range(3):
        # new values in the captured input buffers, eager work and synchronisation between the replays
        x.copy_(torch.randn(x.shape, generator=gen, device="cuda").to(x.dtype))
        dy.copy_(torch.randn(dy.shape, generator=gen, device="cuda").to(dy.dtype))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        want = run()
        torch.cuda.synchronize()
        for k, (g, e) in enumerate(zip(got, want)):
            assert torch.equal(g, e), f"replay {replay}: output {k} differs from the eager call"


def test_split_contraction_and_seeded_forward_replay_matches_eager():
    """A short batch with long contractions: forward (mask drawn in the pass) and backward both split their K range
    into slices whose fp32 partial tiles live in the call's workspace, which torch allocates inside the capture; the
    second kernels read what the replay's own first kernels wrote."""
    from lorafusion_amd import _lib as L
    from lorafusion_amd.ops import hip_ops

    M, K, N, r = 128, 5120, 5120, 16
    routing = L.single_routing(r, 2.0, 0.1)
    assert L.lib().lf_workspace_bytes(L.LF_OP_FWD, M, N, K, r, routing) > 0          # the forward splits
    gen = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn((M, K), generator=gen, device="cuda").to(torch.bfloat16)
    dy = torch.randn((M, N), generator=gen, device="cuda").to(torch.bfloat16)
    w = (torch.randn((N, K), generator=gen, device="cuda") * 0.02).to(torch.bfloat16)
    a = (torch.randn((r, K), generator=gen, device="cuda") / 90.0).to(torch.bfloat16)
    b = (torch.randn((N, r), generator=gen, device="cuda") * 0.01).to(torch.bfloat16)

    def run():
        y, s, mask = hip_ops.lora_forward_seeded(x, w, [a], [b], routing, r, 1234, None)
        dx, da, db = hip_ops.lora_backward(dy, x, w, [a], [b], s, routing, r, mask, [r])
        return [y, dx, *da, *db, mask]

    run()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        run()
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            outs = run()
    torch.cuda.synchronize()
    for replay in range(3):
        x.copy_(torch.randn(x.shape, generator=gen, device="cuda").to(x.dtype))
        dy.copy_(torch.randn(dy.shape, generator=gen, device="cuda").to(dy.dtype))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        want = run()
        torch.cuda.synchronize()
        for k, (g, e) in enumerate(zip(got, want)):
            assert torch.equal(g, e), f"replay {replay}: output {k} differs from the eager call"


def test_norm_activation_and_prologue_replay_matches_eager():
    """RMSNorm forward / backward (with dw: two kernels and a workspace), SiLU-multiply, and the down projection with
    the activation as its prologue, captured once and replayed on fresh values."""
    from lorafusion_amd.ops import norm_act
    from lorafusion_amd.ops.swiglu_lora import fused_swiglu_linear_lora

    M, H, I, N, r = 300, 512, 768, 256, 16
    g = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn(M, H, device="cuda", generator=g).to(torch.bfloat16)
    dyn = torch.randn(M, H, device="cuda", generator=g).to(torch.bfloat16)
    wn = (1 + 0.1 * torch.randn(H, device="cuda", generator=g)).to(torch.bfloat16)
    gu = torch.randn(M, 2 * I, device="cuda", generator=g).to(torch.bfloat16)
    w = (torch.randn(N, I, device="cuda", generator=g) * 0.02).to(torch.bfloat16)
    a = (torch.randn(r, I, device="cuda", generator=g) * 0.03).to(torch.bfloat16)
    b = (torch.randn(N, r, device="cuda", generator=g) * 0.01).to(torch.bfloat16)
    dy = torch.randn(M, N, device="cuda", generator=g).to(torch.bfloat16)

    def run():
        xs, ws = x.detach().requires_grad_(True), wn.detach().requires_grad_(True)
        y = norm_act.rms_norm(xs, ws, 1e-5)
        y.backward(dyn)
        gs, a_, b_ = gu.detach().requires_grad_(True), a.detach().requires_grad_(True), b.detach().requires_grad_(True)
        z = fused_swiglu_linear_lora(gs, w, a_, b_, 2.0, seed=11, dropout_p=0.1)
        z.backward(dy)
        return [y.detach(), xs.grad, ws.grad, z.detach(), gs.grad, a_.grad, b_.grad]

    run()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        run()
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            outs = run()
    torch.cuda.synchronize()
    gen = torch.Generator(device="cuda").manual_seed(9)
    for replay in range(3):
        x.copy_(torch.randn(x.shape, generator=gen, device="cuda").to(x.dtype))
        gu.copy_(torch.randn(gu.shape, generator=gen, device="cuda").to(gu.dtype))
        dy.copy_(torch.randn(dy.shape, generator=gen, device="cuda").to(dy.dtype))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        want = run()
        torch.cuda.synchronize()
        for k, (g_, e_) in enumerate(zip(got, want)):
            assert torch.equal(g_, e_), f"replay {replay}: output {k} differs from the eager call"
