#!/usr/bin/env python3
"""Benchmark of the fused LoRA-linear hot path on one MI355X.

Workload (the configuration the headline metric is quoted on): the multi-LoRA packed batch --
4 adapters of rank 16, scales {16,32,32,64}/16, dropout {0,.05,.1,.1}, lognormal(6.5, 0.8) token
segments clipped to [64,4096] and packed to 8192 tokens, each adapter padded to 128 rows, shared
base W[4096,4096] bf16, explicit seeded Bernoulli keep-mask, forward + backward (dX, dA_i, dB_i).
One "step" = one fused forward + backward of that linear layer with all inputs resident in HBM.

Prints ONE JSON line.  `value` = algorithmic TFLOP/s of the whole step, counted on the 8192 real
tokens: 2*(2MKN) + 6*M*r*(K+N).  `roofline` describes the dominant kernel (the MFMA GEMM of the
backward, dX = dY W + LoRA term), timed live with HIP events on the launch stream.  `cpu_baseline`
is the unfused PyTorch expression (the oracle's bf16 op-by-op arithmetic with autograd backward) on
a bounded sample of the same workload on the host cores.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import numpy as np  # noqa: E402
import torch  # noqa: E402

BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
HBM_PEAK_GBS = 8000.0

K = N = 4096
RANK = 16
TOKENS = 8192
SCALES = [1.0, 2.0, 2.0, 4.0]
DROPOUT = [0.0, 0.05, 0.1, 0.1]
BLOCK = 128


def segments(total_tokens: int, n_adapters: int, seed: int = 0, longest: int = 4096):
    rng = np.random.default_rng(seed)
    lens, tot = [], 0
    while tot < total_tokens:
        n = int(np.clip(rng.lognormal(6.5, 0.8), 64, longest))
        n = min(n, total_tokens - tot)
        lens.append(n)
        tot += n
    per = [0] * n_adapters
    for i, n in enumerate(lens):
        per[i % n_adapters] += n
    return per


def build_inputs(device, seq, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(0)
    padded = [((n - 1) // BLOCK + 1) * BLOCK for n in seq]
    Mp = sum(padded)
    x = torch.randn(Mp, K, generator=g).to(dtype)
    w = (torch.randn(N, K, generator=g) * 0.02).to(dtype)
    dy = torch.randn(Mp, N, generator=g).to(dtype)
    a_list, b_list = [], []
    for i in range(len(seq)):
        ga = torch.Generator().manual_seed(10 + i)
        a_list.append(((torch.rand(RANK, K, generator=ga) * 2 - 1) / K ** 0.5).to(dtype))
        b_list.append((torch.randn(N, RANK, generator=ga) * 0.01).to(dtype))
    gm = torch.Generator().manual_seed(1)
    row_p = torch.cat([torch.full((pl,), p) for pl, p in zip(padded, DROPOUT)])
    mask = torch.rand(Mp, K, generator=gm) >= row_p[:, None]
    t = dict(x=x, w=w, dy=dy, a_list=a_list, b_list=b_list, mask=mask)
    if device is not None:
        t = {k: ([v.to(device) for v in val] if isinstance(val, list) else val.to(device)) for k, val in t.items()}
    t["padded"] = padded
    return t


def step_flops(tokens: int) -> float:
    return 2 * (2.0 * tokens * K * N) + 6.0 * tokens * RANK * (K + N)


def event_time_ms(fn, reps: int) -> float:
    """Average duration of `fn`'s launches: `reps` back-to-back calls between two HIP events
    recorded on the stream the kernels are launched on (torch's current stream)."""
    st = torch.cuda.current_stream()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    fn()
    torch.cuda.synchronize()
    e0.record(st)
    for _ in range(reps):
        fn()
    e1.record(st)
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps


def graph_time_ms(fn, reps: int, inner: int = 10) -> float:
    """Average duration of `fn`'s launches with no host work between them: `inner` calls captured once
    as a HIP graph, replayed between two HIP events.  For kernels of a few tens of microseconds, whose
    Python wrapper takes longer than the kernel runs (the GPU would otherwise wait for the host)."""
    side, graph = torch.cuda.Stream(), torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        fn()
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            keep = [fn() for _ in range(inner)]
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    n = max(1, reps // inner)
    st = torch.cuda.current_stream()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(st)
    for _ in range(n):
        graph.replay()
    e1.record(st)
    torch.cuda.synchronize()
    del keep
    return e0.elapsed_time(e1) / (n * inner)


# The other benchmark configurations of the reference, as linear layers of the same fused path:
# (tokens, adapters, rank, scales, dropout, NF4 base weight, longest segment, [(projection, K, N)]).
LAYER_WORKLOADS = {
    "c1": (2048, 1, 16, [2.0], [0.1], False, 4096, [("linear", 4096, 4096)]),
    "c3": (4096, 1, 16, [2.0], [0.0], True, 4096, [("linear", 4096, 14336)]),
    "c4": (16384, 4, 16, [1.0, 2.0, 2.0, 4.0], [0.0, 0.05, 0.1, 0.1], False, 8192,
           [("q", 4096, 4096), ("k", 4096, 1024), ("v", 4096, 1024), ("o", 4096, 4096),
            ("gate", 4096, 14336), ("up", 4096, 14336), ("down", 14336, 4096)]),
    "c5": (8192, 8, 64, [1.0, 2.0, 2.0, 4.0] * 2, [0.0, 0.05, 0.1, 0.1] * 2, True, 4096,
           [("q", 8192, 8192), ("k", 8192, 1024), ("v", 8192, 1024), ("o", 8192, 8192),
            ("gate", 8192, 28672), ("up", 8192, 28672), ("down", 28672, 8192)]),
}
LAYER_NAMES = {
    "c1": "single LoRA linear, 2048 tokens, K=N=4096, r=16, p=0.1, explicit mask, fwd+bwd",
    "c3": "NF4 QLoRA linear 4096 -> 14336, 4096 tokens, r=16, dequantisation inside the call, fwd+bwd",
    "c4": "the seven LoRA linears of an 8B-class decoder layer (hidden 4096, kv 1024, MLP 14336), 16384 packed "
          "tokens, 4 adapters r=16, fwd+bwd; attention, norms and activation are not part of the path",
    "c5": "the seven LoRA linears of a 70B-class decoder layer (hidden 8192, kv 1024, MLP 28672) with NF4 base "
          "weights, 8192 packed tokens, 8 adapters r=64, fwd+bwd; attention, norms and activation are not part of the path",
}


def layer_workload(args, name: str) -> None:
    """One of the reference's other configurations: every projection timed on its own (inputs of one
    projection resident at a time), `value` = algorithmic flops of all projections / the sum of their times."""
    from lorafusion_amd.ops import hip_ops
    from lorafusion_amd.ops.multi_lora import prepare_multi_lora_batch_info
    from lorafusion_amd.ops.nf4 import NF4WeightRef, quantize_nf4

    tokens, n_ad, rank, scales, drops, nf4, longest, projs = LAYER_WORKLOADS[name]
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    seq = segments(tokens, n_ad, longest=longest) if n_ad > 1 else [tokens]
    info = prepare_multi_lora_batch_info(seq, list(range(n_ad)), [rank] * n_ad, drops, scales, BLOCK)
    padded = info.padded_seq_len_list
    Mp = sum(padded)
    routing = hip_ops.MultiRouting(padded, [rank] * n_ad, info.block_to_lookup_table, info.block_to_alpha, info.block_to_dropout_p)
    row_p = torch.cat([torch.full((pl,), float(p)) for pl, p in zip(padded, drops)]).to(dev)
    g = torch.Generator(device=dev).manual_seed(0)
    per_proj, total_ms, total_flops = {}, 0.0, 0.0
    for pname, k, n in projs:
        x = torch.randn(Mp, k, generator=g, device=dev).to(torch.bfloat16)
        dy = torch.randn(Mp, n, generator=g, device=dev).to(torch.bfloat16)
        w = (torch.randn(n, k, generator=g, device=dev) * 0.02).to(torch.bfloat16)
        a_l = [((torch.rand(rank, k, generator=g, device=dev) * 2 - 1) / k ** 0.5).to(torch.bfloat16) for _ in range(n_ad)]
        b_l = [(torch.randn(n, rank, generator=g, device=dev) * 0.01).to(torch.bfloat16) for _ in range(n_ad)]
        mask = (torch.rand(Mp, k, generator=g, device=dev) >= row_p[:, None]) if any(p > 0 for p in drops) else None
        if nf4:
            packed, qs = quantize_nf4(w.float())
            wref = NF4WeightRef(packed, qs)
            del w

            def step():
                y, s_ = hip_ops.nf4_lora_forward(x, wref, a_l, b_l, routing.c, routing.R, mask, None)
                return y, hip_ops.nf4_lora_backward(dy, x, wref, a_l, b_l, s_, routing.c, routing.R, mask, [rank] * n_ad)
        else:
            def step():
                y, s_ = hip_ops.lora_forward(x, w, a_l, b_l, routing.c, routing.R, mask, None)
                return y, hip_ops.lora_backward(dy, x, w, a_l, b_l, s_, routing.c, routing.R, mask, [rank] * n_ad)
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / args.steps
        flops = 2 * (2.0 * tokens * k * n) + 6.0 * tokens * rank * (k + n)
        per_proj[pname] = {"K": k, "N": n, "ms": round(ms, 4), "TFLOP/s": round(flops / (ms * 1e-3) / 1e12, 1)}
        total_ms += ms
        total_flops += flops
        del x, dy, mask, a_l, b_l, step
        torch.cuda.empty_cache()
    print(json.dumps({
        "metric": "fused LoRA fwd+bwd TFLOP/s (8B layer, r=16); NF4 dequant GB/s; % roofline",
        "value": round(total_flops / (total_ms * 1e-3) / 1e12, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(total_ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": LAYER_NAMES[name], "tokens": tokens, "rows_launched": Mp, "rank": rank, "adapters": n_ad,
                   "nf4_base": nf4, "seq_len_list": seq},
        "projections": per_proj, "roofline": None, "cpu_baseline": None,
    }))


def cpu_baseline(seq, budget_s: float = 15.0):
    """Oracle (bf16 op-by-op, autograd backward) on the host cores: the whole 8192-token batch when one
    run takes under a second (it does on the GPU box's host), else the first 256 tokens of every
    adapter; as many runs as fit in about `budget_s` seconds (at least 3), median reported."""
    from oracle import lora_ref

    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    def make(sample):
        sseq = [min(n, sample) for n in seq]
        t = build_inputs(None, sseq)

        def one():
            x = t["x"].clone().requires_grad_(True)
            a = [v.clone().requires_grad_(True) for v in t["a_list"]]
            b = [v.clone().requires_grad_(True) for v in t["b_list"]]
            y = lora_ref.linear_multi_lora_bf16_opbyop(x, t["w"], a, b, sseq, t["padded"], SCALES, DROPOUT, t["mask"])
            y.backward(t["dy"])

        return sseq, one

    sseq, one = make(256)
    one()
    t0 = time.perf_counter()
    one()
    small = time.perf_counter() - t0
    what = "256 tokens per adapter"
    if small * (sum(seq) / sum(sseq)) < 1.0:  # the full batch fits the budget many times over
        sseq, one = make(max(seq))
        one()
        what = "the whole batch"
    times = []
    t_start = time.perf_counter()
    while len(times) < 3 or time.perf_counter() - t_start < budget_s:
        t0 = time.perf_counter()
        one()
        times.append(time.perf_counter() - t0)
        if len(times) >= 200:
            break
    med = sorted(times)[len(times) // 2]
    return {
        "value": step_flops(sum(sseq)) / med / 1e12,
        "unit": "TFLOP/s",
        "cores": cores,
        "kind": "port",
        "sample": f"{sum(sseq)} tokens ({what}) of the same multi-LoRA batch, bf16 op-by-op + autograd, "
                  f"median of {len(times)} runs over {time.perf_counter() - t_start:.0f} s, {med * 1e3:.1f} ms/run",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--workload", choices=["c2", *LAYER_WORKLOADS], default="c2",
                    help="c2 (default): the multi-LoRA packed batch the metric is quoted on; c1, c3, c4, c5: the "
                         "reference's other configurations, one line with a per-projection breakdown and no roofline entry")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run one 256 MiB device-to-device copy (reference point for FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1).")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU (MI355X); none is visible.")

    if args.workload != "c2":
        return layer_workload(args, args.workload)

    from lorafusion_amd.ops import hip_ops
    from lorafusion_amd.ops.multi_lora import fused_linear_multi_lora, prepare_multi_lora_batch_info
    from lorafusion_amd.ops.nf4 import dequantize_nf4_triton, quantize_nf4

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    seq = segments(TOKENS, 4)
    t = build_inputs(dev, seq)
    info = prepare_multi_lora_batch_info(seq, [0, 1, 2, 3], [RANK] * 4, DROPOUT, SCALES, BLOCK)
    x = t["x"].requires_grad_(True)
    a_list = [a.requires_grad_(True) for a in t["a_list"]]
    b_list = [b.requires_grad_(True) for b in t["b_list"]]
    x3, dy3 = x.unsqueeze(0), t["dy"].unsqueeze(0)

    def step():
        y = fused_linear_multi_lora(
            x3, t["w"], lora_a_list=a_list, lora_b_list=b_list, seq_len_list=seq,
            padded_seq_len_list=info.padded_seq_len_list, block_to_lookup_table=info.block_to_lookup_table,
            block_to_dropout_p=info.block_to_dropout_p, block_to_alpha=info.block_to_alpha,
            enable_dropout=True, same_dropout_p_value=None, max_r=RANK, dropout_mask=t["mask"])
        y.backward(dy3)
        x.grad = None
        for p in a_list + b_list:
            p.grad = None

    if args.calibration_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    value = step_flops(TOKENS) / (ms * 1e-3) / 1e12

    # ---- the same forward + backward captured once as a HIP graph and replayed (what a training loop
    # that captures its step gets: no host launch work, shorter gaps between the kernels)
    routing_g = hip_ops.MultiRouting(info.padded_seq_len_list, [RANK] * 4, info.block_to_lookup_table,
                                     info.block_to_alpha, info.block_to_dropout_p)
    xg, ag, bg = x.detach(), [a.detach() for a in a_list], [b.detach() for b in b_list]

    def raw_step():
        y, s_ = hip_ops.lora_forward(xg, t["w"], ag, bg, routing_g.c, routing_g.R, t["mask"], None)
        return y, hip_ops.lora_backward(t["dy"], xg, t["w"], ag, bg, s_, routing_g.c, routing_g.R, t["mask"], [RANK] * 4)

    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        raw_step()
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            graph_out = raw_step()
    torch.cuda.synchronize()
    for _ in range(args.warmup):
        graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        graph.replay()
    torch.cuda.synchronize()
    ms_graph = (time.perf_counter() - t0) * 1e3 / args.steps
    del graph_out

    # ---- per-kernel timings with HIP events: the GEMMs as plain back-to-back launches, the short rank-r,
    # mask and dequant kernels replayed from a graph (their wrappers take longer than they run)
    routing = hip_ops.MultiRouting(info.padded_seq_len_list, [RANK] * 4, info.block_to_lookup_table,
                                   info.block_to_alpha, info.block_to_dropout_p)
    xd, wd, dyd, mask = x.detach(), t["w"], t["dy"], t["mask"]
    ad = [a.detach() for a in a_list]
    bd = [b.detach() for b in b_list]
    s = hip_ops.fused_multi_lora_xa(xd, ad, routing, mask)
    _, ds = hip_ops.fused_multi_lora_dys_dyb(dyd, s, bd, routing)
    Mp = xd.shape[0]
    reps = 20
    t_fwd = event_time_ms(lambda: hip_ops.fused_multi_lora_xw_sb(xd, wd, s, bd, routing), reps)
    t_bwd = event_time_ms(lambda: hip_ops.fused_multi_lora_dyw_dsa(dyd, wd, ds, ad, routing, mask), reps)
    t_plain_nt = event_time_ms(lambda: hip_ops.gemm(xd, wd, trans_b=True), reps)
    t_plain_nn = event_time_ms(lambda: hip_ops.gemm(dyd, wd, trans_b=False), reps)
    t_xa = graph_time_ms(lambda: hip_ops.fused_multi_lora_xa(xd, ad, routing, mask), reps)
    t_dys = graph_time_ms(lambda: hip_ops.fused_multi_lora_dys_dyb(dyd, s, bd, routing), reps)
    t_da = graph_time_ms(lambda: hip_ops.fused_multi_lora_da(xd, ds, routing, mask), reps)
    t_mask = graph_time_ms(lambda: hip_ops.make_dropout_mask(xd.shape, None, 1234, dev, routing=routing), reps)
    t_fwd_seeded = event_time_ms(lambda: hip_ops.lora_forward_seeded(xd, wd, ad, bd, routing.c, routing.R, 1234, None), reps)
    # ---- dominant kernel: the 256x256-tile MFMA GEMM of the dX path.  The library runs rows
    # [0, 8192) of the 8448 in whole rounds of that tile and the last 256 rows as a second, small
    # launch; the roofline entry times the big launch alone (same grid, same data: the first 64
    # routing blocks) so that its duration is one kernel's, comparable with a kernel trace.
    main_rows = (Mp // 4096) * 4096
    nbm = main_rows // BLOCK
    pad_main, left = [], main_rows
    for pl in info.padded_seq_len_list:
        take = min(pl, left)
        if take > 0:
            pad_main.append(take)
        left -= take
    routing_main = hip_ops.MultiRouting(pad_main, [RANK] * len(pad_main), info.block_to_lookup_table[:nbm].contiguous(),
                                        info.block_to_alpha[:nbm].contiguous(), info.block_to_dropout_p[:nbm].contiguous())
    dy_m, ds_m, mask_m = dyd[:main_rows], ds[:main_rows], mask[:main_rows]
    ad_m = ad[:len(pad_main)]
    dom_ms = event_time_ms(lambda: hip_ops.fused_multi_lora_dyw_dsa(dy_m, wd, ds_m, ad_m, routing_main, mask_m), reps)
    dom_name = "gemm_lora_kernel<256x256 tile, NN> (dX = dY W + mask*(dS A)/(1-p)), rows [0, %d)" % main_rows
    # algorithmic flops of that launch: 2*M*K*N dense + 2*M*r*N LoRA seed
    gemm_flops = 2.0 * main_rows * K * N + 2.0 * main_rows * RANK * N
    achieved = gemm_flops / (dom_ms * 1e-3) / 1e12

    # ---- NF4 dequant (W[14336,4096], blocksize 64, double quantised): 2.516 B/element
    wq = torch.randn(14336, 4096, device=dev) * 0.02
    packed, qs = quantize_nf4(wq)
    out = torch.empty(14336 * 4096, dtype=torch.bfloat16, device=dev)
    t_nf4_op = event_time_ms(lambda: dequantize_nf4_triton(packed, qs, out=out), reps)   # as called from Python
    t_nf4 = graph_time_ms(lambda: dequantize_nf4_triton(packed, qs, out=out), 5 * reps)   # the kernel alone
    n = 14336 * 4096
    nf4_bytes = n / 2 + n / 64 + 4 * n / 16384 + 1028 + 2 * n
    nf4_gbs = nf4_bytes / (t_nf4 * 1e-3) / 1e9

    # HBM-side bytes per launch of the dominant kernel: the figure of the committed counter summary
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "bench_c2_hbm_traffic.txt")
    if os.path.exists(tpath):
        with open(tpath) as f:
            for line in f:
                if line.startswith("dominant_kernel_bytes_per_launch"):
                    traffic = int(line.split()[1])

    res = {
        "metric": "fused LoRA fwd+bwd TFLOP/s (8B layer, r=16); NF4 dequant GB/s; % roofline",
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "multi-LoRA packed batch: 4 adapters r=16, 8192 tokens (lognormal segments, seed 0) "
                        f"padded to {Mp} rows, K=N=4096, fwd+bwd, explicit dropout mask",
            "tokens": TOKENS, "rows_launched": Mp, "K": K, "N": N, "rank": RANK, "adapters": 4,
            "seq_len_list": seq,
        },
        "roofline": {
            "bound": "mfma", "achieved": round(achieved, 2), "peak": BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": round(achieved / BF16_PEAK_TFLOPS, 4), "traffic": traffic,
            "kernel": dom_name, "launch_ms": round(dom_ms, 4), "flops_per_launch": gemm_flops,
        },
        "kernels_ms": {
            "xa": round(t_xa, 4), "gemm_fwd": round(t_fwd, 4), "dys_dyb": round(t_dys, 4), "da": round(t_da, 4),
            "gemm_bwd": round(t_bwd, 4), "seeded_mask": round(t_mask, 4), "fwd_seeded_xa_plus_gemm": round(t_fwd_seeded, 4), "plain_gemm_nt": round(t_plain_nt, 4), "plain_gemm_nn": round(t_plain_nn, 4),
        },
        "hipgraph_replay": {"ms_per_step": round(ms_graph, 4),
                            "TFLOP/s": round(step_flops(TOKENS) / (ms_graph * 1e-3) / 1e12, 2)},
        "lora_overhead_vs_plain_gemms": round((t_xa + t_fwd + t_dys + t_da + t_bwd) / (t_plain_nt + t_plain_nn) - 1.0, 4),
        "nf4_dequant": {
            "GB/s": round(nf4_gbs, 1), "frac_of_hbm_peak": round(nf4_gbs / HBM_PEAK_GBS, 4),
            "launch_ms": round(t_nf4, 4), "op_ms_from_python": round(t_nf4_op, 4), "bytes_per_launch": nf4_bytes,
            "shape": [14336, 4096],
        },
    }
    if not args.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline(seq)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
