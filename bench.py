#!/usr/bin/env python3
"""Benchmark of the fused LoRA-linear hot path on one MI355X.

Headline workload (the configuration the metric names: "8B layer, r=16"): the seven LoRA projections of a
Llama-3-8B-shaped decoder layer -- hidden 4096, kv 1024, MLP 14336 -- as four LoRA linears: q/k/v merged into one
N=6144 linear, which is what the reference's layer does (lorafusion/patch/patch_transformers.py:50-163, 278-287), and
gate/up merged likewise into one N=28672 linear, which the reference does not do (a merged gate/up adapter shares one
A between the two halves).  The same layer with only q/k/v merged (`workloads.c4_qkv_merged`, the reference's own
layer: five linears) and as seven separate linears (`workloads.c4_separate`, BASELINE's wording) is measured next to
it.  16384 packed tokens of 4 adapters (rank 16, multipliers
{1,2,2,4}, dropout {0,.05,.1,.1}, lognormal segment lengths up to 8192), each adapter padded to 128 rows,
bf16, training mode (dropout masks drawn in the rank-r pass), forward + backward (dX, dA_i, dB_i).  The
micro-batch comes in as a scheduler descriptor, goes through the MultiLoRAManager, and every linear is
called through the patched layer's forward.  Attention, rotary embedding, norms and the activation are not
part of the path and not run.  One "step" = forward + backward of the four linears, inputs resident in HBM.

Prints ONE JSON line.  `value` = algorithmic TFLOP/s of the step, counted on the 16384 real tokens:
per linear 2*(2*M*K*N) + 6*M*r*(K+N).  `roofline` describes the dominant kernel of the step -- the persistent
256x256-tile MFMA GEMM of the backward (dX = dY W + mask*(dS A)/(1-p)) -- over its four launches per step,
each timed live with HIP events on the launch stream.  `cpu_baseline` is the unfused PyTorch expression
(the oracle's bf16 op-by-op arithmetic with autograd backward) on the host cores.  `workloads` holds the
reference's other configurations (c1 single linear, c2 packed multi-LoRA linear, c3 NF4 linear, c5 70B-class
NF4 layer), each with its own roofline entry, `nf4_dequant` the standalone dequant kernel against HBM peak, and
`norm_act` the RMSNorm and SiLU-multiply kernels (the steps either side of the layer's linears) at the layer's
shapes, each against HBM peak; they are measured on their own and are not part of `value`.
"""

from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time
from types import SimpleNamespace

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import numpy as np  # noqa: E402
import torch  # noqa: E402

BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
HBM_PEAK_GBS = 8000.0
BLOCK = 128
METRIC = "fused LoRA fwd+bwd TFLOP/s (8B layer, r=16); NF4 dequant GB/s; % roofline"

# (tokens, adapters, rank, multipliers, dropout, NF4 base weight, longest segment, [(linear, K, N)])
WORKLOADS = {
    "c1": (2048, 1, 16, [2.0], [0.1], False, 4096, [("linear", 4096, 4096)]),
    "c2": (8192, 4, 16, [1.0, 2.0, 2.0, 4.0], [0.0, 0.05, 0.1, 0.1], False, 4096, [("linear", 4096, 4096)]),
    "c3": (4096, 1, 16, [2.0], [0.0], True, 4096, [("linear", 4096, 14336)]),
    "c4": (16384, 4, 16, [1.0, 2.0, 2.0, 4.0], [0.0, 0.05, 0.1, 0.1], False, 8192,
           [("qkv", 4096, 6144), ("o", 4096, 4096), ("gate_up", 4096, 28672), ("down", 14336, 4096)]),
    "c4_qkv_merged": (16384, 4, 16, [1.0, 2.0, 2.0, 4.0], [0.0, 0.05, 0.1, 0.1], False, 8192,
                      [("qkv", 4096, 6144), ("o", 4096, 4096), ("gate", 4096, 14336), ("up", 4096, 14336), ("down", 14336, 4096)]),
    "c4_separate": (16384, 4, 16, [1.0, 2.0, 2.0, 4.0], [0.0, 0.05, 0.1, 0.1], False, 8192,
                    [("q", 4096, 4096), ("k", 4096, 1024), ("v", 4096, 1024), ("o", 4096, 4096), ("gate", 4096, 14336),
                     ("up", 4096, 14336), ("down", 14336, 4096)]),
    "c5": (8192, 8, 64, [1.0, 2.0, 2.0, 4.0] * 2, [0.0, 0.05, 0.1, 0.1] * 2, True, 4096,
           [("qkv", 8192, 10240), ("o", 8192, 8192), ("gate_up", 8192, 57344), ("down", 28672, 8192)]),
    "c5_separate": (8192, 8, 64, [1.0, 2.0, 2.0, 4.0] * 2, [0.0, 0.05, 0.1, 0.1] * 2, True, 4096,
                    [("q", 8192, 8192), ("k", 8192, 1024), ("v", 8192, 1024), ("o", 8192, 8192),
                     ("gate", 8192, 28672), ("up", 8192, 28672), ("down", 28672, 8192)]),
}
NAMES = {
    "c1": "single LoRA linear, 2048 tokens, K=N=4096, r=16, p=0.1, explicit mask, fwd+bwd",
    "c2": "multi-LoRA packed batch: 4 adapters r=16, 8192 tokens (lognormal segments, seed 0), K=N=4096, fwd+bwd, "
          "explicit dropout mask",
    "c3": "NF4 QLoRA linear 4096 -> 14336, 4096 tokens, r=16, dequantisation inside the call, fwd+bwd",
    "c4": "the seven LoRA projections of an 8B-class decoder layer (hidden 4096, kv 1024, MLP 14336) as the four LoRA "
          "linears of the merged layer (qkv N=6144, o, gate+up N=28672, down), 16384 packed tokens, 4 adapters r=16, "
          "training-mode dropout drawn in the rank-r pass, fwd+bwd, driven by a micro-batch descriptor through the "
          "patched layer; attention, rotary embedding, norms and activation are not part of the path and not run",
    "c4_qkv_merged": "the same 8B-class layer the way the reference's patched layer runs it: q/k/v merged into one N=6144 "
                     "linear, o, gate, up and down on their own (five LoRA linears), 16384 packed tokens, 4 adapters r=16, "
                     "explicit bit-packed masks through the raw ops, fwd+bwd",
    "c4_separate": "the same 8B-class layer as seven separate LoRA linears (q, k, v, o, gate, up, down), 16384 packed tokens, "
                   "4 adapters r=16, explicit bit-packed masks through the raw ops, fwd+bwd",
    "c5": "the seven LoRA projections of a 70B-class decoder layer (hidden 8192, kv 1024, MLP 28672) as the four LoRA "
          "linears of the merged layer (qkv N=10240, o, gate+up N=57344, down) with NF4 base weights (dequantised "
          "inside every call), 8192 packed tokens, 8 adapters r=64, explicit masks, fwd+bwd; attention, norms and "
          "activation are not part of the path",
    "c5_separate": "the same 70B-class layer as seven separate LoRA linears (q, k, v, o, gate, up, down), NF4 base weights, "
                   "8192 packed tokens, 8 adapters r=64, explicit masks, fwd+bwd",
}


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


def linear_flops(tokens: int, k: int, n: int, rank: int) -> float:
    return 2 * (2.0 * tokens * k * n) + 6.0 * tokens * rank * (k + n)


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


def wall_time_ms(fn, steps: int, warmup: int, min_ms: float = 0.0):
    """Wall clock per step over `steps` back-to-back steps between two synchronisations.  min_ms > 0 (the sub-millisecond
    workloads beside the headline): when the timed region came out shorter than that, it is timed again over as many
    steps as fill it -- the closing synchronisation and the first launch cost about half a millisecond, which 20 steps
    of 0.15 ms do not amortise.  Returns (ms per step, steps timed)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    while True:
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        total = (time.perf_counter() - t0) * 1e3
        if total >= min_ms:
            return total / steps, steps
        steps = int(steps * min_ms / max(total, 1e-3) * 1.1) + 1


class Batch:
    """Routing of one packed batch on the device (shared by all linears of a workload)."""

    def __init__(self, name: str, dev):
        from lorafusion_amd.ops import hip_ops
        from lorafusion_amd.ops.multi_lora import prepare_multi_lora_batch_info

        self.tokens, self.n_ad, self.rank, self.scales, self.drops, self.nf4, longest, self.projs = WORKLOADS[name]
        self.seq = segments(self.tokens, self.n_ad, longest=longest) if self.n_ad > 1 else [self.tokens]
        self.info = prepare_multi_lora_batch_info(self.seq, list(range(self.n_ad)), [self.rank] * self.n_ad, self.drops,
                                                  self.scales, BLOCK, output_dtype=torch.float32)
        self.padded = self.info.padded_seq_len_list
        self.Mp = sum(self.padded)
        self.routing = hip_ops.MultiRouting(self.padded, [self.rank] * self.n_ad, self.info.block_to_lookup_table,
                                            self.info.block_to_alpha, self.info.block_to_dropout_p)
        self.row_p = torch.cat([torch.full((pl,), float(p)) for pl, p in zip(self.padded, self.drops)]).to(dev)
        self.dropout = any(p > 0 for p in self.drops)

    def head(self, rows: int):
        """Routing of rows [0, rows) alone (rows is a multiple of the block size)."""
        from lorafusion_amd.ops import hip_ops

        nb = rows // BLOCK
        pad, left = [], rows
        for pl in self.padded:
            take = min(pl, left)
            if take > 0:
                pad.append(take)
            left -= take
        return hip_ops.MultiRouting(pad, [self.rank] * len(pad), self.info.block_to_lookup_table[:nb].contiguous(),
                                    self.info.block_to_alpha[:nb].contiguous(), self.info.block_to_dropout_p[:nb].contiguous())


class Linear:
    """Device tensors of one LoRA linear of a workload and its raw (autograd-free) forward + backward."""

    def __init__(self, batch: Batch, name: str, k: int, n: int, g, dev):
        from lorafusion_amd.ops import hip_ops
        from lorafusion_amd.ops.nf4 import NF4WeightRef, quantize_nf4

        b = self.batch = batch
        self.name, self.k, self.n = name, k, n
        self.x = torch.randn(b.Mp, k, generator=g, device=dev).to(torch.bfloat16)
        self.dy = torch.randn(b.Mp, n, generator=g, device=dev).to(torch.bfloat16)
        w = (torch.randn(n, k, generator=g, device=dev) * 0.02).to(torch.bfloat16)
        self.a = [((torch.rand(b.rank, k, generator=g, device=dev) * 2 - 1) / k ** 0.5).to(torch.bfloat16) for _ in range(b.n_ad)]
        self.b = [(torch.randn(n, b.rank, generator=g, device=dev) * 0.01).to(torch.bfloat16) for _ in range(b.n_ad)]
        # explicit keep-mask, bit-packed (the library's own format for masks it draws; lf_mask_pack converts a bool tensor)
        self.mask = hip_ops.pack_mask(torch.rand(b.Mp, k, generator=g, device=dev) >= b.row_p[:, None]) if b.dropout else None
        self.wref = None
        if b.nf4:
            self.packed, self.qs = quantize_nf4(w.float())
            self.wref = NF4WeightRef(self.packed, self.qs)
            self.w = None
        else:
            self.w = w
        self.flops = linear_flops(b.tokens, k, n, b.rank)

    def step(self, keep_dense: bool = False):
        from lorafusion_amd.ops import hip_ops

        r = self.batch.routing
        ranks = [self.batch.rank] * self.batch.n_ad
        if self.wref is not None and keep_dense:
            # the forward's dequantised weight handed to the backward: one dequantisation per step
            y, s_, dense = hip_ops.nf4_lora_forward(self.x, self.wref, self.a, self.b, r.c, r.R, self.mask, None, keep_dense=True)
            return y, hip_ops.nf4_lora_backward(self.dy, self.x, self.wref, self.a, self.b, s_, r.c, r.R, self.mask, ranks,
                                                dense=dense)
        if self.wref is not None:
            y, s_ = hip_ops.nf4_lora_forward(self.x, self.wref, self.a, self.b, r.c, r.R, self.mask, None)
            return y, hip_ops.nf4_lora_backward(self.dy, self.x, self.wref, self.a, self.b, s_, r.c, r.R, self.mask, ranks)
        y, s_ = hip_ops.lora_forward(self.x, self.w, self.a, self.b, r.c, r.R, self.mask, None)
        return y, hip_ops.lora_backward(self.dy, self.x, self.w, self.a, self.b, s_, r.c, r.R, self.mask, ranks)

    def dense_weight(self):
        from lorafusion_amd.ops.nf4 import dequantize_nf4_triton

        if self.w is not None:
            return self.w
        return dequantize_nf4_triton(self.packed, self.qs).reshape(self.n, self.k)


def gemm_plan(M: int, N: int, K: int, routed: bool):
    from lorafusion_amd import _lib as L

    rows, ch, ct = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    L.check(L.lib().lf_gemm_plan(M, N, K, BLOCK if routed else 0, ctypes.byref(rows), ctypes.byref(ch), ctypes.byref(ct)), "lf_gemm_plan")
    return rows.value, ch.value, ct.value


def kernel_breakdown(linears, reps: int):
    """Per-kernel times of a workload's linears (summed over them) and the roofline entry of the dominant
    kernel: the dX GEMM.  Where the library runs a row count as whole rounds of 256x256 tiles plus a short
    second launch, the dominant launch is timed alone on its own rows (same grid, same data), so the figure is
    one kernel's duration, comparable with a kernel trace."""
    from lorafusion_amd.ops import hip_ops

    t = dict(xa=0.0, gemm_fwd=0.0, dys_dyb=0.0, da=0.0, gemm_bwd=0.0, plain_gemm_nt=0.0, plain_gemm_nn=0.0)
    dom_ms, dom_flops, launches, kinds = 0.0, 0.0, [], set()
    for lin in linears:
        b = lin.batch
        r, w = b.routing, lin.dense_weight()
        s = hip_ops.fused_multi_lora_xa(lin.x, lin.a, r, lin.mask)
        _, ds = hip_ops.fused_multi_lora_dys_dyb(lin.dy, s, lin.b, r)
        t["gemm_fwd"] += event_time_ms(lambda: hip_ops.fused_multi_lora_xw_sb(lin.x, w, s, lin.b, r), reps)
        t["gemm_bwd"] += event_time_ms(lambda: hip_ops.fused_multi_lora_dyw_dsa(lin.dy, w, ds, lin.a, r, lin.mask), reps)
        t["plain_gemm_nt"] += event_time_ms(lambda: hip_ops.gemm(lin.x, w, trans_b=True), reps)
        t["plain_gemm_nn"] += event_time_ms(lambda: hip_ops.gemm(lin.dy, w, trans_b=False), reps)
        t["xa"] += graph_time_ms(lambda: hip_ops.fused_multi_lora_xa(lin.x, lin.a, r, lin.mask), reps)
        t["dys_dyb"] += graph_time_ms(lambda: hip_ops.fused_multi_lora_dys_dyb(lin.dy, s, lin.b, r), reps)
        t["da"] += graph_time_ms(lambda: hip_ops.fused_multi_lora_da(lin.x, ds, r, lin.mask), reps)
        # the dX GEMM's main launch: output [Mp, K], reduction over N
        rows, cfg, _ = gemm_plan(b.Mp, lin.k, lin.n, True)
        if cfg == 7 and r.R > 32:
            cfg = 1   # the persistent kernel forms the dX term from at most 32 rank columns: the library runs this launch on the eight-wave 256x256 tile
        if rows < b.Mp:
            rh = b.head(rows)
            nseg = len(rh.padded_seq_len_list)
            dy_h, ds_h = lin.dy[:rows], ds[:rows]
            mask_h = lin.mask[:rows] if lin.mask is not None else None
            ms = event_time_ms(lambda: hip_ops.fused_multi_lora_dyw_dsa(dy_h, w, ds_h, lin.a[:nseg], rh, mask_h), reps)
        else:
            ms = event_time_ms(lambda: hip_ops.fused_multi_lora_dyw_dsa(lin.dy, w, ds, lin.a, r, lin.mask), reps)
        fl = 2.0 * rows * lin.k * lin.n + 2.0 * rows * r.R * lin.k
        dom_ms += ms
        dom_flops += fl
        kinds.add(cfg)
        launches.append({"linear": lin.name, "rows": rows, "K_out": lin.k, "N_red": lin.n, "tile_cfg": cfg, "ms": round(ms, 4),
                         "TFLOP/s": round(fl / (ms * 1e-3) / 1e12, 1)})
        del w, s, ds
    kern = ("gemm_big_kernel<bf16, NN, LoRA> (persistent 256x256 tiles)" if kinds == {7} else
            "gemm_lora_kernel / gemm_big_kernel, NN (tile configurations %s)" % sorted(kinds))
    achieved = dom_flops / (dom_ms * 1e-3) / 1e12
    n = len(launches)
    roofline = {
        "bound": "mfma", "achieved": round(achieved, 2), "peak": BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
        "frac": round(achieved / BF16_PEAK_TFLOPS, 4), "traffic": None, "traffic_source": None,
        "kernel": kern + ": dX = dY W + mask*(dS A)/(1-p), main launch of each linear",
        "launches_per_step": n, "launch_ms": round(dom_ms / n, 4), "flops_per_launch": dom_flops / n, "launches": launches,
    }
    t = {k: round(v, 4) for k, v in t.items()}
    overhead = (t["xa"] + t["gemm_fwd"] + t["dys_dyb"] + t["da"] + t["gemm_bwd"]) / (t["plain_gemm_nt"] + t["plain_gemm_nn"]) - 1.0
    roofline["lora_overhead_vs_plain_gemms"] = round(overhead, 4)
    roofline["plain_gemm_same_shapes_frac"] = round(
        sum(2.0 * lin.batch.Mp * lin.k * lin.n for lin in linears) / (t["plain_gemm_nn"] * 1e-3) / 1e12 / BF16_PEAK_TFLOPS, 4)
    return t, roofline, round(overhead, 4)


def read_traffic(roofline: dict, fname: str) -> None:
    """HBM-side bytes per launch of the dominant kernel from the committed counter summary (FETCH_SIZE /
    WRITE_SIZE runs are separate rocprofv3 passes; the figure is not measured in this run)."""
    path = os.path.join(ROOT, "profiles", fname)
    if os.path.exists(path):
        with open(path) as f:
            for line in f:
                if line.startswith("dominant_kernel_bytes_per_launch"):
                    roofline["traffic"] = int(line.split()[1])
                    roofline["traffic_source"] = f"profiles/{fname} (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, separate runs)"


def raw_workload(name: str, args, dev, breakdown: bool = True) -> dict:
    """One of the reference's configurations through the raw ops: all linears resident, K steps of all of them."""
    batch = Batch(name, dev)
    g = torch.Generator(device=dev).manual_seed(0)
    linears = [Linear(batch, pn, k, n, g, dev) for pn, k, n in batch.projs]

    def step():
        for lin in linears:
            lin.step()

    ms, steps_timed = wall_time_ms(step, args.steps, args.warmup, min_ms=40.0)
    flops = sum(lin.flops for lin in linears)
    per = {}
    for lin in linears:
        pm = event_time_ms(lin.step, max(3, args.steps // 4))
        per[lin.name] = {"K": lin.k, "N": lin.n, "ms": round(pm, 4), "TFLOP/s": round(lin.flops / (pm * 1e-3) / 1e12, 1)}
    res = {
        "workload": NAMES[name], "value": round(flops / (ms * 1e-3) / 1e12, 2), "unit": "TFLOP/s", "ms_per_step": round(ms, 4),
        "steps_timed": steps_timed, "tokens": batch.tokens, "rows_launched": batch.Mp, "rank": batch.rank, "adapters": batch.n_ad, "nf4_base": batch.nf4,
        "seq_len_list": batch.seq, "linears": per,
    }
    if batch.nf4:
        def step_keep():
            for lin in linears:
                lin.step(keep_dense=True)

        mk, _ = wall_time_ms(step_keep, args.steps, args.warmup, min_ms=40.0)
        res["reuse_dequantized_weight"] = {
            "ms_per_step": round(mk, 4), "TFLOP/s": round(flops / (mk * 1e-3) / 1e12, 2),
            "note": "the forward's dequantised weight is kept for the backward that follows it: one NF4 dequantisation per "
                    "linear per step instead of two, 2*N*K bytes held in between (the headline figure of this entry "
                    "dequantises in both calls and holds only the packed weight)"}
    if breakdown:
        res["kernels_ms"], res["roofline"], res["lora_overhead_vs_plain_gemms"] = kernel_breakdown(linears, 10)
    if name == "c2" and breakdown:
        from lorafusion_amd.ops import hip_ops

        lin = linears[0]
        r = batch.routing
        read_traffic(res["roofline"], "bench_c2_hbm_traffic.txt")
        res["kernels_ms"]["seeded_mask"] = round(graph_time_ms(
            lambda: hip_ops.make_dropout_mask(lin.x.shape, None, 1234, dev, routing=r), 20), 4)
        res["kernels_ms"]["fwd_seeded_xa_plus_gemm"] = round(event_time_ms(
            lambda: hip_ops.lora_forward_seeded(lin.x, lin.w, lin.a, lin.b, r.c, r.R, 1234, None), 20), 4)
        # the same forward + backward captured once as a HIP graph and replayed
        side, graph = torch.cuda.Stream(), torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            lin.step()
            side.synchronize()
            with torch.cuda.graph(graph, stream=side):
                keep = lin.step()
        torch.cuda.synchronize()
        mg, _ = wall_time_ms(graph.replay, args.steps, args.warmup, min_ms=40.0)
        del keep
        res["hipgraph_replay"] = {"ms_per_step": round(mg, 4), "TFLOP/s": round(flops / (mg * 1e-3) / 1e12, 2)}
    del linears
    torch.cuda.empty_cache()
    return res


def nf4_cpu_baseline(packed, qs, shape, nbytes: float) -> dict:
    """The C restatement of the dequantisation (oracle/nf4_oracle.c, one thread) on the same packed weight, host
    memory to host memory: best of three runs of the whole weight, in the kernel's own unit."""
    import numpy as np

    from oracle import nf4 as onf4

    st = onf4.NF4State(packed=packed.cpu().numpy().reshape(-1), absmax=qs.absmax.cpu().numpy(), shape=tuple(shape),
                       blocksize=qs.blocksize, code2=qs.state2.code.cpu().numpy(), absmax2=qs.state2.absmax.cpu().numpy(),
                       offset=qs.offset.cpu().numpy().reshape(1).astype(np.float32), blocksize2=qs.state2.blocksize)
    best = float("inf")
    for _ in range(3):
        t0 = time.perf_counter()
        onf4.dequantize(st)
        best = min(best, time.perf_counter() - t0)
    return {"value": round(nbytes / best / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"the whole {list(shape)} weight, oracle/nf4_oracle.c on one host core, best of 3 runs, {best * 1e3:.0f} ms/run"}


def nf4_dequant_block(dev, shape=(14336, 4096), fill: bool = False, cpu: bool = False) -> dict:
    """Standalone NF4 dequant of W[shape], blocksize 64, double quantised: 2.516 B/element.  `fill`: also time a plain
    fill of the output tensor (torch's fill kernel: stores only), the reference point for what the write stream of
    this chip reaches at that size."""
    from lorafusion_amd.ops.nf4 import dequantize_nf4_triton, quantize_nf4

    rows, cols = shape
    wq = torch.randn(rows, cols, device=dev) * 0.02
    packed, qs = quantize_nf4(wq)
    del wq
    out = torch.empty(rows * cols, dtype=torch.bfloat16, device=dev)
    t_op = event_time_ms(lambda: dequantize_nf4_triton(packed, qs, out=out), 20)     # as called from Python
    t_k = graph_time_ms(lambda: dequantize_nf4_triton(packed, qs, out=out), 100)     # the kernel alone
    n = rows * cols
    nbytes = n / 2 + n / 64 + 4 * n / 16384 + 1028 + 2 * n
    gbs = nbytes / (t_k * 1e-3) / 1e9
    res = {"GB/s": round(gbs, 1), "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4), "launch_ms": round(t_k, 4),
           "op_ms_from_python": round(t_op, 4), "bytes_per_launch": nbytes, "shape": [rows, cols],
           "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                        "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None, "kernel": "nf4_dequant_kernel"}}
    if cpu:
        res["cpu_baseline"] = nf4_cpu_baseline(packed, qs, (rows, cols), nbytes)
    if fill:
        t_f = graph_time_ms(lambda: out.fill_(1.0), 100)
        res["plain_fill_of_the_output"] = {"launch_ms": round(t_f, 4), "GB/s": round(2 * n / (t_f * 1e-3) / 1e9, 1),
                                           "bytes": 2 * n, "kernel": "torch fill_ (vectorized_elementwise_kernel)"}
    return res


def nf4_block(dev) -> dict:
    """`--only nf4`: the dequant kernel at the C3 weight and at the four weights of the 70B-class layer, each next to a
    plain fill of its output."""
    shapes = {"c3 [14336, 4096]": (14336, 4096), "c5 qkv [10240, 8192]": (10240, 8192), "c5 o [8192, 8192]": (8192, 8192),
              "c5 gate_up [57344, 8192]": (57344, 8192), "c5 down [8192, 28672]": (8192, 28672)}
    return {name: nf4_dequant_block(dev, shp, fill=True) for name, shp in shapes.items()}


def gemm_ref_block(dev, reps: int = 20, zero: bool = False) -> dict:
    """`--only gemm_ref`: the plain GEMMs of the 8B layer's largest shapes through this library (lf_gemm: the persistent
    kernel without a LoRA term) and through torch.matmul (hipBLASLt), same tensors, same process -- the run the
    counter comparison in profiles/ is taken from.  `--only gemm_ref_zero`: the same launches on all-zero operands:
    identical instruction streams and memory traffic, no switching in the multipliers.  What the two kernels gain
    there is what the chip's power management takes from them on real data; it says nothing about throughput on real
    data and is reported for that comparison only."""
    from lorafusion_amd.ops import hip_ops

    out = {}
    for name, (M, N, K, trans_b) in {"16384x4096x4096 NT": (16384, 4096, 4096, True), "16384x4096x28672 NN": (16384, 4096, 28672, False),
                                     "16384x14336x4096 NT": (16384, 14336, 4096, True),
                                     # the single linear of workload c1 (one round of the persistent kernel's 128x256 tiles)
                                     "2048x4096x4096 NT": (2048, 4096, 4096, True), "2048x4096x4096 NN": (2048, 4096, 4096, False)}.items():
        g = torch.Generator(device=dev).manual_seed(0)
        a = torch.randn(M, K, generator=g, device=dev).to(torch.bfloat16)
        b = (torch.randn(N, K, generator=g, device=dev) if trans_b else torch.randn(K, N, generator=g, device=dev)).to(torch.bfloat16)
        if zero:
            a.zero_()
            b.zero_()
        fl = 2.0 * M * N * K
        t_lib = event_time_ms(lambda: hip_ops.gemm(a, b, trans_b=trans_b), reps)
        t_ref = event_time_ms(lambda: torch.matmul(a, b.T if trans_b else b), reps)
        out[name] = {"lf_gemm_ms": round(t_lib, 4), "lf_gemm_TFLOP/s": round(fl / t_lib / 1e9, 1), "lf_gemm_frac": round(fl / t_lib / 1e9 / BF16_PEAK_TFLOPS, 4),
                     "torch_matmul_ms": round(t_ref, 4), "torch_matmul_TFLOP/s": round(fl / t_ref / 1e9, 1),
                     "torch_matmul_frac": round(fl / t_ref / 1e9 / BF16_PEAK_TFLOPS, 4)}
        del a, b
        torch.cuda.empty_cache()
    return out


FIG5_M, FIG5_KN = (2048, 4096, 8192), (4096, 5120, 8192)


def fig5_block(args, dev) -> dict:
    """The shape grid of the reference's kernel benchmark (benchmarks_paper/scripts/kernel_perf/1_bench_kernel.sh:3-16,
    bench_lora_kernels.py:682-685): one LoRA linear, M rows, K = N, r = 16, p = 0.1, forward + backward."""
    out = {}
    for m in FIG5_M:
        for kn in FIG5_KN:
            name = f"fig5_M{m}_KN{kn}"
            WORKLOADS[name] = (m, 1, 16, [2.0], [0.1], False, 4096, [("linear", kn, kn)])
            NAMES[name] = f"single LoRA linear, {m} tokens, K=N={kn}, r=16, p=0.1, explicit bit-packed mask, fwd+bwd"
            r = raw_workload(name, args, dev)
            out[f"M={m},K=N={kn}"] = {"ms_per_step": r["ms_per_step"], "TFLOP/s": r["value"], "kernels_ms": r["kernels_ms"],
                                      "lora_overhead_vs_plain_gemms": r["lora_overhead_vs_plain_gemms"],
                                      "roofline": {k: r["roofline"][k] for k in ("bound", "achieved", "peak", "unit", "frac", "kernel", "launch_ms")}}
    return out


def norm_act_block(dev) -> dict:
    """The elementwise steps either side of the 8B layer's linears on its 16512 rows: RMSNorm (hidden 4096) forward
    and backward, SiLU(gate) * up on the merged [16512, 2 x 14336] projection output, forward and backward (which
    writes the merged gradient), and the activation folded into the down projection's rank-r pass.  Algorithmic bytes per
    element: 4 (norm forward: read x, write y), 6 (norm backward: read dy and x, write dx), 6 (activation forward),
    10 (activation backward)."""
    from lorafusion_amd import _lib as L

    lib = L.lib()
    M, H, I = 16512, 4096, 14336
    g = torch.Generator(device=dev).manual_seed(0)
    x = torch.randn(M, H, device=dev, generator=g).to(torch.bfloat16)
    dy = torch.randn(M, H, device=dev, generator=g).to(torch.bfloat16)
    w = torch.ones(H, device=dev, dtype=torch.bfloat16)
    y, dx, dw = torch.empty_like(x), torch.empty_like(x), torch.empty_like(w)
    rstd = torch.empty(M, device=dev)
    n_ws = lib.lf_rmsnorm_bwd_workspace(M, H)
    ws = torch.empty(n_ws, dtype=torch.uint8, device=dev)
    gu = torch.randn(M, 2 * I, device=dev, generator=g).to(torch.bfloat16)
    dc = torch.randn(M, I, device=dev, generator=g).to(torch.bfloat16)
    c, dgu = torch.empty(M, I, device=dev, dtype=torch.bfloat16), torch.empty_like(gu)
    st = L.stream_of(x)
    calls = {
        "rmsnorm_fwd": (4 * M * H + 4 * M, "rmsnorm_fwd_kernel", lambda: L.check(lib.lf_rmsnorm_fwd(
            x.data_ptr(), w.data_ptr(), y.data_ptr(), rstd.data_ptr(), M, H, 1e-6, 0, st), "lf_rmsnorm_fwd")),
        "rmsnorm_bwd_frozen_weight": (6 * M * H + 4 * M, "rmsnorm_bwd_kernel", lambda: L.check(lib.lf_rmsnorm_bwd(
            dy.data_ptr(), x.data_ptr(), w.data_ptr(), rstd.data_ptr(), dx.data_ptr(), None, M, H, 0, None, 0, st),
            "lf_rmsnorm_bwd")),
        "rmsnorm_bwd_with_dw": (6 * M * H + 4 * M, "rmsnorm_bwd_kernel", lambda: L.check(lib.lf_rmsnorm_bwd(
            dy.data_ptr(), x.data_ptr(), w.data_ptr(), rstd.data_ptr(), dx.data_ptr(), dw.data_ptr(), M, H, 0,
            ws.data_ptr(), n_ws, st), "lf_rmsnorm_bwd")),
        "silu_mul_fwd": (6 * M * I, "silu_mul_fwd_kernel", lambda: L.check(lib.lf_silu_mul_fwd(
            gu.data_ptr(), gu[:, I:].data_ptr(), c.data_ptr(), M, I, 2 * I, 2 * I, I, 0, st), "lf_silu_mul_fwd")),
        "silu_mul_bwd": (10 * M * I, "silu_mul_bwd_kernel", lambda: L.check(lib.lf_silu_mul_bwd(
            dc.data_ptr(), gu.data_ptr(), gu[:, I:].data_ptr(), dgu.data_ptr(), dgu[:, I:].data_ptr(), M, I, I, 2 * I,
            2 * I, 2 * I, 2 * I, 0, st), "lf_silu_mul_bwd")),
    }
    # the down projection's rank-r pass (4 adapters r=16, the layer's segments, keep-mask drawn in the kernel) with the
    # activation as its prologue, next to the activation kernel followed by the plain pass.  Algorithmic bytes per
    # element: 6.125 fused (read gate and up, write the product and the mask bit), 6 + 2.125 separate.
    from lorafusion_amd.ops import multi_lora as ml

    seq = segments(16384, 4, seed=0, longest=8192)
    info = ml.prepare_multi_lora_batch_info(seq, [0, 1, 2, 3], [16] * 4, [0.0, 0.05, 0.1, 0.1], [1.0, 2.0, 2.0, 4.0], 128)
    rt = info.routing(enable_dropout=True)
    assert rt.M == M
    a_list = [torch.randn(16, I, device=dev, generator=g).to(torch.bfloat16) * 0.01 for _ in range(4)]
    a_ptrs = L.ptr_array(a_list)
    s_out = torch.empty(M, 16, device=dev, dtype=torch.bfloat16)
    mask_out = torch.empty(M, I // 8, device=dev, dtype=torch.uint8)   # bit-packed, as the training path keeps it
    seed = ctypes.c_uint64(1234)
    bits = L.LF_BF16 | L.LF_MASK_BITS
    calls["down_xa_with_silu_mul_prologue"] = (6 * M * I + M * I // 8, "lora_xa_kernel<.., seeded, activation>", lambda: L.check(
        lib.lf_lora_xa_silu_mul(gu.data_ptr(), gu[:, I:].data_ptr(), 2 * I, c.data_ptr(), None, mask_out.data_ptr(), seed,
                                a_ptrs, s_out.data_ptr(), M, I, 16, rt.c, bits, st), "lf_lora_xa_silu_mul"))
    calls["down_xa_seeded_alone"] = (2 * M * I + M * I // 8, "lora_xa_kernel<.., seeded>", lambda: L.check(
        lib.lf_lora_xa_seeded(c.data_ptr(), mask_out.data_ptr(), a_ptrs, s_out.data_ptr(), M, I, 16, rt.c, seed, bits, st),
        "lf_lora_xa_seeded"))
    out = {"rows": M, "hidden": H, "intermediate": I}
    for name, (nbytes, kernel, fn) in calls.items():
        t = event_time_ms(fn, 50)
        gbs = nbytes / (t * 1e-3) / 1e9
        out[name] = {"launch_ms": round(t, 4), "bytes_per_launch": nbytes,
                     "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                  "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None, "kernel": kernel}}
    out["down_prologue_saving_ms"] = round(out["silu_mul_fwd"]["launch_ms"] + out["down_xa_seeded_alone"]["launch_ms"]
                                           - out["down_xa_with_silu_mul_prologue"]["launch_ms"], 4)
    return out


# --------------------------------------------------------------------------- the headline: the 8B layer

def layer_c4(args, dev):
    """The four merged LoRA linears of the 8B-class layer, called through the patched layer module with the
    micro-batch registered at the MultiLoRAManager from a scheduler descriptor."""
    from lorafusion_amd.ops import multi_lora as ml
    from lorafusion_amd.patch.patch_transformers import DecoderLayerLoRAProjections

    tokens, n_ad, rank, scales, drops, _, longest, projs = WORKLOADS["c4"]
    seq = segments(tokens, n_ad, longest=longest)
    # the reference's data provider hands lora_alpha to the kernels as the multiplier (training_utils.py:1323)
    cfgs = [SimpleNamespace(r=rank, lora_alpha=s, lora_dropout=p) for s, p in zip(scales, drops)]
    adapters = {f"lora_{i}": (c.r, c.lora_alpha, c.lora_dropout) for i, c in enumerate(cfgs)}
    layer = DecoderLayerLoRAProjections.from_shapes(4096, 1024, 14336, adapters, device=dev, seed=0)
    layer.train()
    g = torch.Generator(device=dev).manual_seed(1)
    with torch.no_grad():
        for lin in layer.linears().values():
            for nm in lin.lora_B:
                lin.lora_B[nm].weight.copy_(torch.randn(lin.lora_B[nm].weight.shape, generator=g, device=dev) * 0.01)
    mb = SimpleNamespace(
        adapter_group_info=set(range(n_ad)), adapter_num_tokens_pairs=dict(enumerate(seq)),
        padded_adapter_num_tokens_pairs={i: ((n - 1) // BLOCK + 1) * BLOCK for i, n in enumerate(seq)},
        adapter_num_samples_pairs={i: 1 for i in range(n_ad)}, adapter_padding_multiple=BLOCK, is_empty_marker=False)
    ml.reset_multi_lora_manager()
    mgr = ml.init_multi_lora_manager(cfgs, 1, None, [1] * n_ad)
    info = ml.batch_info_from_micro_batch(mb, cfgs)
    mgr.add_batch_info(info)
    Mp = sum(info.padded_seq_len_list)
    lins = layer.linears()
    io = {}
    for name, k, n in projs:
        x = torch.randn(1, Mp, k, generator=g, device=dev).to(torch.bfloat16).requires_grad_(True)
        dy = torch.randn(1, Mp, n, generator=g, device=dev).to(torch.bfloat16)
        io[name] = (x, dy)
    params = [p for lin in lins.values() for p in lin.parameters() if p.requires_grad]

    def step():
        for name, lin in lins.items():
            x, dy = io[name]
            mgr.mark_forward_pass_started()
            y = lin(x)
            mgr.mark_backward_pass_started()
            y.backward(dy)
            x.grad = None
        for p in params:
            p.grad = None

    ms, _ = wall_time_ms(step, args.steps, args.warmup)
    flops = sum(linear_flops(tokens, k, n, rank) for _, k, n in projs)
    per = {}
    for name, k, n in projs:
        x, dy = io[name]

        own = [p for p in lins[name].parameters() if p.requires_grad]

        def one(lin=lins[name], x=x, dy=dy, own=own):
            mgr.mark_forward_pass_started()
            y = lin(x)
            mgr.mark_backward_pass_started()
            y.backward(dy)
            x.grad = None
            for p in own:
                p.grad = None

        pm = event_time_ms(one, max(3, args.steps // 4))
        fl = linear_flops(tokens, k, n, rank)
        per[name] = {"K": k, "N": n, "ms": round(pm, 4), "TFLOP/s": round(fl / (pm * 1e-3) / 1e12, 1)}
    for p in params:
        p.grad = None
    ml.reset_multi_lora_manager()
    del layer, io, lins, params
    torch.cuda.empty_cache()
    return ms, flops, seq, Mp, per


def cpu_baseline_c4(budget_s: float = 20.0):
    """Oracle (bf16 op-by-op, autograd backward) of the four linears on the host cores: the whole 16384-token
    batch when three runs of it fit the budget (estimated from a 1024-token run), else 256 tokens per adapter;
    median of at least 3 runs."""
    from oracle import lora_ref

    tokens, n_ad, rank, scales, drops, _, longest, projs = WORKLOADS["c4"]
    seq = segments(tokens, n_ad, longest=longest)
    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)

    def make(sample):
        sseq = [min(n, sample) for n in seq]
        padded = [((n - 1) // BLOCK + 1) * BLOCK for n in sseq]
        Mp = sum(padded)
        g = torch.Generator().manual_seed(0)
        row_p = torch.cat([torch.full((pl,), float(p)) for pl, p in zip(padded, drops)])
        data = []
        for _, k, n in projs:
            x = torch.randn(Mp, k, generator=g).to(torch.bfloat16)
            w = (torch.randn(n, k, generator=g) * 0.02).to(torch.bfloat16)
            dy = torch.randn(Mp, n, generator=g).to(torch.bfloat16)
            a = [((torch.rand(rank, k, generator=g) * 2 - 1) / k ** 0.5).to(torch.bfloat16) for _ in range(n_ad)]
            b = [(torch.randn(n, rank, generator=g) * 0.01).to(torch.bfloat16) for _ in range(n_ad)]
            mask = torch.rand(Mp, k, generator=g) >= row_p[:, None]
            data.append((x, w, dy, a, b, mask))

        def one():
            for x, w, dy, a, b, mask in data:
                xr = x.clone().requires_grad_(True)
                ar = [v.clone().requires_grad_(True) for v in a]
                br = [v.clone().requires_grad_(True) for v in b]
                y = lora_ref.linear_multi_lora_bf16_opbyop(xr, w, ar, br, sseq, padded, scales, drops, mask)
                y.backward(dy)

        return sseq, one

    sseq, one = make(256)
    one()
    t0 = time.perf_counter()
    one()
    small = time.perf_counter() - t0
    what = "256 tokens per adapter"
    if 3 * small * (sum(seq) / sum(sseq)) < budget_s:
        sseq, one = make(max(seq))
        one()
        what = "the whole batch"
    times = []
    t_start = time.perf_counter()
    while len(times) < 3 or time.perf_counter() - t_start < budget_s:
        t0 = time.perf_counter()
        one()
        times.append(time.perf_counter() - t0)
        if len(times) >= 100:
            break
    med = sorted(times)[len(times) // 2]
    fl = sum(linear_flops(sum(sseq), k, n, rank) for _, k, n in projs)
    return {
        "value": fl / med / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port",
        "sample": f"{sum(sseq)} tokens ({what}) of the same four LoRA linears, bf16 op-by-op + autograd, "
                  f"median of {len(times)} runs over {time.perf_counter() - t_start:.0f} s, {med * 1e3:.1f} ms/run",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true", help="only the headline workload (c4), its roofline and the CPU baseline")
    ap.add_argument("--only", choices=sorted(WORKLOADS) + ["norm_act", "nf4", "gemm_ref", "gemm_ref_zero", "fig5"], default=None,
                    help="run one workload through the raw ops and print its entry alone (for profiling runs)")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run one 256 MiB device-to-device copy (reference point for FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1).")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU (MI355X); none is visible.")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.calibration_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    if args.only == "norm_act":
        print(json.dumps({"metric": "norm_act", **norm_act_block(dev)}))
        return
    if args.only == "nf4":
        print(json.dumps({"metric": "nf4_dequant", **nf4_block(dev)}))
        return
    if args.only in ("gemm_ref", "gemm_ref_zero"):
        zero = args.only == "gemm_ref_zero"
        print(json.dumps({"metric": "plain GEMM: lf_gemm vs torch.matmul (hipBLASLt)" + (", all-zero operands" if zero else ""),
                          **gemm_ref_block(dev, zero=zero)}))
        return
    if args.only == "fig5":
        print(json.dumps({"metric": "fig5 grid", **fig5_block(argparse.Namespace(steps=max(5, args.steps // 2), warmup=2), dev)}))
        return
    if args.only is not None:
        print(json.dumps({"metric": METRIC, **raw_workload(args.only, args, dev, breakdown=not args.no_extras)}))
        return

    ms, flops, seq, Mp, per = layer_c4(args, dev)
    raw = raw_workload("c4", args, dev)       # the same four linears through the raw ops, explicit masks: per-kernel times
    read_traffic(raw["roofline"], "bench_c4_hbm_traffic.txt")
    res = {
        "metric": METRIC,
        "value": round(flops / (ms * 1e-3) / 1e12, 2),
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
        "config": {"workload": NAMES["c4"], "tokens": 16384, "rows_launched": Mp, "rank": 16, "adapters": 4,
                   "seq_len_list": seq, "linears": per, "lora_overhead_vs_plain_gemms": raw["lora_overhead_vs_plain_gemms"]},
        "roofline": raw["roofline"],
        "kernels_ms": raw["kernels_ms"],
        "lora_overhead_vs_plain_gemms": raw["lora_overhead_vs_plain_gemms"],
        "raw_ops_explicit_mask": {"ms_per_step": raw["ms_per_step"], "TFLOP/s": raw["value"], "linears": raw["linears"]},
    }
    if not args.no_extras:
        res["nf4_dequant"] = nf4_dequant_block(dev, cpu=not args.no_cpu_baseline)
        res["norm_act"] = norm_act_block(dev)
        small = argparse.Namespace(steps=max(5, args.steps // 2), warmup=max(2, args.warmup // 2))
        res["workloads"] = {name: raw_workload(name, args if name == "c2" else small, dev)
                            for name in ("c1", "c2", "c3", "c4_qkv_merged", "c4_separate", "c5")}
        res["workloads"]["fig5"] = fig5_block(small, dev)
        res["gemm_ref"] = {"random_operands": gemm_ref_block(dev, reps=10), "all_zero_operands": gemm_ref_block(dev, reps=10, zero=True)}
    if not args.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline_c4()
    print(json.dumps(res))


if __name__ == "__main__":
    main()
