#!/usr/bin/env python3
"""Benchmark of the MoE-forward hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3_bf16|c4_fp8|c2_bf16|c5_bf16|c5_fp8]
                    [--tokens T] [--no-cpu-baseline] [--no-extra] [--sample-clock] [--dense-reference]
                    [--hbm-ceiling] [--tile-trace]

A step is one forward pass of the hot path over one batch of synthetic input that is
already resident in HBM: top-k routing from the gate probabilities, the gather +
grouped GEMM with its SiLU / SwiGLU epilogue, (fp8: the row-wise quantisations),
the down-projection GEMM and the weighted merge.  The gate Linear + softmax that
produce the probabilities stay torch calls and are outside the step, as they are
outside the FLOP count.  Prints ONE JSON line.

Timing: `value` / `ms_per_step` come from exactly K back-to-back steps between two device
synchronisations (hot caches, the steady state of a serving loop).  Beside it: per-step HIP-event
samples (median, p95), the same with a 512 MiB buffer rewritten before every step so that neither
L2 nor the 256 MB last-level cache holds anything of the previous step (`cold`), and per-kernel
durations from HIP events over max(K, 100) launches after 25 warm-up launches (the reference's
do_bench(warmup=25, rep=100), kernels/benchmarks/timer.py:174-198).
"""
from __future__ import annotations

import argparse
import json
import math
import os
import re
import subprocess
import sys
import threading
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK = {"bf16": 2500.0, "fp8": 5000.0}   # dense MFMA TFLOP/s, MI355X
HBM_PEAK_GBS = 8000.0
PROFILE_OF = {"c3_bf16": "moe_forward_c3_bf16_T16384_E64.txt", "c4_fp8": "moe_forward_c4_fp8_T16384_E64.txt"}


def measured_traffic_bytes(workload):
    """HBM-side bytes per GEMM1 launch from the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE sections of
    the workload's summary under profiles/ (KiB per dispatch of the epi=2 ring kernel), scaled by the
    copy-kernel factors that summary states (FETCH_SIZE x 2.0, WRITE_SIZE x 1.0).  None if the
    summary is missing or has no such lines."""
    name = PROFILE_OF.get(workload)
    path = os.path.join(ROOT, "profiles", name) if name else None
    if not path or not os.path.exists(path):
        return None
    text = open(path).read()
    vals = {}
    for counter in ("FETCH_SIZE", "WRITE_SIZE"):
        m = re.search(r"^\s*gemm_ring\S* fp8=\w+ epi=2(?: msc)?\s+" + counter + r"=([0-9.e+]+)\s*$", text, re.M)
        if not m:
            return None
        vals[counter] = float(m.group(1))
    return int((vals["FETCH_SIZE"] * 2.0 + vals["WRITE_SIZE"] * 1.0) * 1024)


WORKLOADS = {
    # name: (T, E, K, D, H, O, kind, dtype, routing)
    "c2_bf16": dict(T=8192, E=8, K=2, D=1024, H=4096, O=1024, kind="mlp", dtype="bf16", routing="gate"),
    "c3_bf16": dict(T=16384, E=64, K=8, D=2048, H=1408, O=2048, kind="swiglu", dtype="bf16", routing="zipf"),
    "c4_fp8": dict(T=16384, E=64, K=8, D=2048, H=1408, O=2048, kind="swiglu", dtype="fp8", routing="zipf"),
    "c5_bf16": dict(T=4096, E=128, K=8, D=4096, H=1536, O=4096, kind="swiglu", dtype="bf16", routing="uniform"),
    "c5_fp8": dict(T=4096, E=128, K=8, D=4096, H=1536, O=4096, kind="swiglu", dtype="fp8", routing="uniform"),
}


def flops_of(w):
    R = w["T"] * w["K"]
    hn = 2 * w["H"] if w["kind"] == "swiglu" else w["H"]
    return 2.0 * R * w["D"] * hn, 2.0 * R * w["H"] * w["O"]


def make_inputs(w, device, seed=0):
    """Synthetic tensors of the workload's shape, generated on `device`."""
    g = torch.Generator(device=device).manual_seed(seed)
    bf = torch.bfloat16
    T, E, K, D, H, O = (w[k] for k in "TEKDHO")
    rn = lambda *s: torch.randn(*s, generator=g, device=device)
    x = rn(T, D).to(bf)
    if w["dtype"] == "fp8":          # 1 % of the token rows scaled x100 as outliers
        rows = torch.randperm(T, generator=g, device=device)[: max(1, T // 100)]
        x[rows] = (x[rows].float() * 100).to(bf)
    inp = {"x": x}
    if w["kind"] == "swiglu":
        inp["w_gate"] = (rn(E, H, D) * D ** -0.5).to(bf)     # stored [E, N, K], passed as [E, K, N] views
        inp["w_up"] = (rn(E, H, D) * D ** -0.5).to(bf)
        inp["w_down"] = (rn(E, O, H) * H ** -0.5).to(bf)
    else:
        inp["w1"] = (rn(E, H, D) * D ** -0.5).to(bf)
        inp["b1"] = torch.zeros(E, H, dtype=bf, device=device)
        inp["w2"] = (rn(E, O, H) * H ** -0.5).to(bf)
        inp["b2"] = torch.zeros(E, O, dtype=bf, device=device)
    w_gate_net = rn(D, E) * D ** -0.5
    logits = x.float() @ w_gate_net
    if w["routing"] == "zipf":       # per-expert Zipf(1.1) bias; the last two experts get no token
        p = (torch.arange(E, device=device, dtype=torch.float32) + 1) ** -1.1
        logits = logits + torch.log(p / p.sum())
        logits[:, E - 2:] = -1e30
    elif w["routing"] == "uniform":  # uniform random distinct experts, gates 1/K after renormalisation
        logits = torch.rand(T, E, generator=g, device=device) * 1e-3
    scores = torch.softmax(logits, dim=1)
    inp["scores"] = scores if w["kind"] == "swiglu" else scores.to(bf)
    return inp


class GpuPath:
    """The hot path through the library, split into its kernels so that each can be timed."""

    def __init__(self, w, inp):
        from fast_moe_amd.kernels import moe_fp8
        from fast_moe_amd.kernels.hip import ops
        self.ops, self.w, self.inp = ops, w, inp
        self.fp8 = w["dtype"] == "fp8"
        v = lambda t: t.permute(0, 2, 1)
        if w["kind"] == "swiglu":
            self.wg, self.wu, self.wd = v(inp["w_gate"]), v(inp["w_up"]), v(inp["w_down"])
            if self.fp8:             # weights are quantised once, outside the step (the opt-in fp8_weight path)
                self.quant_weights()
        else:
            self.w1, self.w2 = v(inp["w1"]), v(inp["w2"])

    def quant_weights(self):
        """The three expert weight tensors to e4m3 + row scales.  The library's fp8 operators do this
        on every call unless the caller hands them the quantised pair (fp8_weight=), as the
        reference's do (kernels/pytorch/moe_fp8.py:111); a serving loop with fixed weights does it once."""
        from fast_moe_amd.kernels import moe_fp8
        self.qg, self.sg = moe_fp8.quantize_expert_weights(self.wg)
        self.qu, self.su = moe_fp8.quantize_expert_weights(self.wu)
        self.qd, self.sd = moe_fp8.quantize_expert_weights(self.wd)

    def step_with_weight_quant(self):
        """The step of the default operator path: weights re-quantised inside it."""
        self.quant_weights()
        return self.step()

    # --- the pieces
    def route(self):
        # (the routing tensors of the previous step are written in place: a serving loop keeps them)
        self.r = self.ops.route_topk(self.inp["scores"], self.w["K"], out=getattr(self, "r", None))
        return self.r

    def quant_tokens(self):
        self.qx, self.sx = self.ops.quant_rows_fp8(self.inp["x"])

    def gemm1(self):
        o, w, r, K = self.ops, self.w, self.r, self.w["K"]
        R = w["T"] * K
        if w["kind"] == "mlp":
            self.hidden = o.grouped_gemm(r["offsets"], self.inp["x"], self.w1, total_rows=R,
                                         row_index=r["gate_index"], index_div=K, bias=self.inp["b1"], epilogue=1)
        elif self.fp8:
            self.hidden = o.grouped_gemm(r["offsets"], self.qx, self.qg, total_rows=R, row_index=r["gate_index"],
                                         index_div=K, b2=self.qu, epilogue=2, scales_pow2=True, a_scale=self.sx, b_scale=self.sg,
                                         b2_scale=self.su)
        else:
            self.hidden = o.grouped_gemm(r["offsets"], self.inp["x"], self.wg, total_rows=R,
                                         row_index=r["gate_index"], index_div=K, b2=self.wu, epilogue=2)

    def quant_hidden(self):
        self.qh, self.sh = self.ops.quant_rows_fp8(self.hidden)

    def gemm2(self):
        o, r = self.ops, self.r
        R = self.w["T"] * self.w["K"]
        if self.w["kind"] == "mlp":
            self.rows = o.grouped_gemm(r["offsets"], self.hidden, self.w2, total_rows=R, bias=self.inp["b2"])
        elif self.fp8:
            self.rows = o.grouped_gemm(r["offsets"], self.qh, self.qd, total_rows=R, scales_pow2=True, a_scale=self.sh,
                                       b_scale=self.sd)
        else:
            self.rows = o.grouped_gemm(r["offsets"], self.hidden, self.wd, total_rows=R)

    def combine(self):
        r = self.r
        gates = r["gates"] if self.w["kind"] == "mlp" else r["gates"].to(torch.bfloat16)
        self.y = self.ops.combine(self.rows, r["reverse_index"], gates, r["gate_index"])
        return self.y

    def pieces(self):
        seq = [("route", self.route)]
        if self.fp8:
            seq.append(("quant_tokens", self.quant_tokens))
        seq.append(("gemm1", self.gemm1))
        if self.fp8:
            seq.append(("quant_hidden", self.quant_hidden))
        seq += [("gemm2", self.gemm2), ("combine", self.combine)]
        return seq

    def step(self):
        for _, fn in self.pieces():
            fn()
        return self.y


def time_region(fn, iters, stream):
    """Average milliseconds of `fn` over `iters` launches, HIP events on the launch stream."""
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record(stream)
    for _ in range(iters):
        fn()
    stop.record(stream)
    stop.synchronize()
    return start.elapsed_time(stop) / iters


def algorithmic_bytes(w, name):
    T, E, K, D, H, O = (w[k] for k in "TEKDHO")
    R = T * K
    if name == "route":
        sb = 2 if w["kind"] == "mlp" else 4
        return T * E * sb + 3 * R * 8 + T * K * (8 + sb) + (2 * E + 1) * 8
    if name == "quant_tokens":
        return T * D * 3 + T * 4
    if name == "quant_hidden":
        return R * H * 3 + R * 4
    if name == "combine":
        return R * O * 2 + T * O * 2 + R * (8 + 8 + 2)
    return None


def step_samples(fn, n, stream, flush=None):
    """Per-step milliseconds from one HIP-event pair per step.  `flush`: a tensor rewritten before
    every step, outside the event pair, so that the step starts with cold caches."""
    pairs = []
    for _ in range(n):
        if flush is not None:
            flush.add_(1)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record(stream)
        fn()
        b.record(stream)
        pairs.append((a, b))
    torch.cuda.synchronize()
    return sorted(a.elapsed_time(b) for a, b in pairs)


def quantiles(samples):
    n = len(samples)
    return {"median": round(samples[n // 2], 4), "p95": round(samples[min(n - 1, int(math.ceil(0.95 * n)) - 1)], 4),
            "min": round(samples[0], 4), "samples": n}


def run_gpu(w, steps, warmup, detail=True):
    dev = torch.device("cuda:0")
    inp = make_inputs(w, dev)
    path = GpuPath(w, inp)
    stream = torch.cuda.current_stream(dev)
    for _ in range(max(warmup, 1)):
        path.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        path.step()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / steps
    timing = {}
    if detail and path.fp8:
        # the default operator path quantises the weights on every call: the same step with that inside
        path.step_with_weight_quant()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            path.step_with_weight_quant()
        torch.cuda.synchronize()
        timing["ms_per_step_weights_quantised_in_step"] = (time.perf_counter() - t0) * 1e3 / steps
    if detail:
        n = max(steps, 100)
        timing["hot"] = quantiles(step_samples(path.step, n, stream))
        flush = torch.zeros(512 << 20, dtype=torch.uint8, device=dev)
        timing["cold"] = quantiles(step_samples(path.step, max(steps, 30), stream, flush))
        del flush
    # per-kernel launch durations, measured live with events: 25 warm-up launches, then max(K, 100)
    path.step()
    per = {}
    reps = max(steps, 100) if detail else steps
    for name, fn in path.pieces():
        for _ in range(25 if detail else 1):
            fn()
        torch.cuda.synchronize()
        per[name] = time_region(fn, reps, stream)
    f1, f2 = flops_of(w)
    kernels = {}
    for name, ms in per.items():
        entry = {"ms": round(ms, 4)}
        if name == "gemm1":
            entry["tflops"] = round(f1 / ms / 1e9, 1)
        elif name == "gemm2":
            entry["tflops"] = round(f2 / ms / 1e9, 1)
        else:
            b = algorithmic_bytes(w, name)
            if b:
                entry["gbs"] = round(b / ms / 1e6, 1)
        kernels[name] = entry
    lengths = path.r["lengths"]
    stats = {"rows_max": int(lengths.max()), "rows_min": int(lengths.min()),
             "empty_experts": int((lengths == 0).sum())}
    return ms_step, kernels, stats, (f1, f2), timing


def cpu_baseline(w, budget_s=12.0):
    """The oracle (CPU restatement of the reference's PyTorch path) on a bounded sample of the
    same workload: same dims and routing law, fewer tokens."""
    from oracle import layer as o_layer
    from oracle import moe as o_moe
    from oracle import moe_fp8 as o_fp8
    cores = torch.get_num_threads()           # the threads the oracle's torch calls actually use
    sample_T = 256
    result = None
    while True:
        ws = dict(w, T=sample_T)
        inp = make_inputs(ws, torch.device("cpu"), seed=1)
        K = w["K"]
        v = lambda t: t.permute(0, 2, 1)

        def run():
            r = o_layer.route_scores(inp["scores"], K)
            idx2 = r["gate_index"].view(-1, K)
            if w["kind"] == "mlp":
                h = o_moe.index_select_jagged_bmm(r["offsets"], idx2, inp["x"], v(inp["w1"]), inp["b1"])
                return o_moe.silu_jagged_bmm_combine(r["offsets"], h, v(inp["w2"]), inp["b2"], r["token_index"], K,
                                                     r["gates"], r["gate_index"])
            gates = r["gates"].to(torch.bfloat16)
            if w["dtype"] == "fp8":
                return o_fp8.swiglu_moe_fp8(r["offsets"], idx2, inp["x"], v(inp["w_gate"]), None, v(inp["w_up"]),
                                            None, v(inp["w_down"]), None, r["token_index"], K, gates,
                                            r["gate_index"])[0]
            return o_moe.fused_jagged_bmm_swiglu_combine(r["offsets"], idx2, inp["x"], v(inp["w_gate"]), None,
                                                         v(inp["w_up"]), None, v(inp["w_down"]), None, K, gates,
                                                         r["gate_index"])

        t0 = time.perf_counter()
        run()
        dt = time.perf_counter() - t0
        if dt * 4 > budget_s or sample_T * 4 > w["T"]:       # final size: median of three more passes
            reps = []
            for _ in range(3):
                t0 = time.perf_counter()
                run()
                reps.append(time.perf_counter() - t0)
            dt = sorted(reps)[1]
        f1, f2 = flops_of(ws)
        result = {"value": round((f1 + f2) / dt / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
                  "sample": f"oracle PyTorch-kernel path, {w['dtype']} emulation, T={sample_T} of {w['T']} tokens "
                            f"(same E/K/D/H, same routing law), median of 3 passes after 1 warm-up, {dt:.2f} s each",
                  "tokens_per_s": round(sample_T / dt, 1), "torch_num_threads": cores,
                  "host_logical_cpus": os.cpu_count()}
        if dt * 4 > budget_s or sample_T * 4 > w["T"]:
            return result
        sample_T *= 4


def run_train(w, steps, warmup):
    """Forward + backward of the SwiGLU MoE through the differentiable operators (bf16): the
    training step, reported beside the forward metric, never instead of it."""
    from fast_moe_amd.kernels import moe
    from fast_moe_amd.kernels.hip import ops
    dev = torch.device("cuda:0")
    inp = make_inputs(w, dev)
    T, K = w["T"], w["K"]
    leaf = lambda t: t.detach().clone().requires_grad_(True)
    x, wg, wu, wd = leaf(inp["x"]), leaf(inp["w_gate"]), leaf(inp["w_up"]), leaf(inp["w_down"])
    dy = torch.randn(T, w["O"], device=dev).to(torch.bfloat16) * 0.01
    stream = torch.cuda.current_stream(dev)

    def forward():
        r = ops.route_topk(inp["scores"], K)
        gates = r["gates"].to(torch.bfloat16).requires_grad_(True)
        h = moe.index_select_jagged_bmm_swiglu(0, r["offsets"], r["gate_index"].view(T, K), x,
                                               wg.permute(0, 2, 1), None, wu.permute(0, 2, 1), None)
        return moe.silu_jagged_bmm_combine(0, r["offsets"], h, wd.permute(0, 2, 1), None, r["token_index"],
                                           r["reverse_index"], gates, r["gate_index"], has_silu=False)

    def step():
        for t in (x, wg, wu, wd):
            t.grad = None
        forward().backward(dy)

    for _ in range(max(warmup, 1)):
        step()
    torch.cuda.synchronize()
    ms = time_region(step, steps, stream)
    ms_fwd = time_region(lambda: forward(), steps, stream)
    f1, f2 = flops_of(w)
    return ms, ms_fwd, 3.0 * (f1 + f2)


def run_sgmoe(steps, warmup, tokens):
    """The SGMoE layer with the MRN router front-end at the 64-expert top-8 size of
    the headline workload (SiLU MLP experts, as the layer has them): evaluation forward,
    training step, and the share of the router front-end (norm, normalised-logit gating,
    dispatch) in the forward.  Reported beside the forward metric, never instead of it."""
    from fast_moe_amd.modules.sgmoe import SGConfig, SGMoE
    dev = torch.device("cuda:0")
    T, D, H, E, K = tokens, 2048, 1408, 64, 8
    torch.manual_seed(0)
    layer = SGMoE(D, D, False, 1, SGConfig(model_d=H, num_experts=E, num_activated_experts=K)).to(dev).to(torch.bfloat16)
    x = torch.randn(T, D, device=dev).to(torch.bfloat16)
    dy = torch.randn(T, D, device=dev).to(torch.bfloat16) * 0.01
    stream = torch.cuda.current_stream(dev)

    def front_end():
        x_norm = torch.nn.functional.layer_norm(x, (D,), layer._norm_w, layer._norm_bias, layer.norm_eps).to(x.dtype)
        _, gates, idx, _ = layer._noisy_gating(x_norm, False, None)
        from fast_moe_amd.kernels.hip import ops
        return ops.route_from_topk(idx, E), gates

    def train_step():
        layer.zero_grad(set_to_none=True)
        out = layer(x)
        (out.x * dy).sum().add(out.loss.sum() if out.loss is not None else 0).backward()

    layer.eval()
    with torch.no_grad():
        for _ in range(max(warmup, 1)):
            layer(x)
        torch.cuda.synchronize()
        ms_eval = time_region(lambda: layer(x), steps, stream)
        ms_front = time_region(front_end, steps, stream)
    layer.train()
    for _ in range(max(warmup, 1)):
        train_step()
    torch.cuda.synchronize()
    ms_train = time_region(train_step, steps, stream)
    flops = 2.0 * T * K * (D * H + H * D) + 2.0 * T * D * D       # routed experts + shared-expert addmm
    return ms_eval, ms_front, ms_train, flops, (T, D, H, E, K)


def bench_workload(name, steps, warmup, tokens=None, detail=True):
    w = dict(WORKLOADS[name])
    if tokens:
        w["T"] = tokens
    ms, kernels, stats, (f1, f2), timing = run_gpu(w, steps, warmup, detail)
    return w, ms, kernels, stats, f1 + f2, timing


def weight_stream_bytes(w, lengths_nonzero):
    """Algorithmic HBM bytes of one forward in the weight-streaming regime (few rows per expert):
    the weights of the experts that have a row, the tokens in and the outputs out."""
    wb = 1 if w["dtype"] == "fp8" else 2
    hn = 2 * w["H"] if w["kind"] == "swiglu" else w["H"]
    return lengths_nonzero * (w["D"] * hn + w["H"] * w["O"]) * wb + w["T"] * w["D"] * 2 + w["T"] * w["O"] * 2


def extra_workloads(steps, warmup):
    """The other configurations of the baseline beside the headline pair, one short entry each:
    C2 (8 experts, top-2, SiLU MLP) and the 128-expert sweep in bf16 and e4m3 (GB/s of the weight
    stream up to 512 tokens, TFLOP/s above), plus the one-off weight quantisation of the
    64-expert configuration (not part of a step)."""
    out = {}
    w, ms, kern, stats, fl, _ = bench_workload("c2_bf16", steps, warmup, detail=False)
    out["c2_bf16"] = {"tokens": w["T"], "ms_per_step": round(ms, 4), "tflops": round(fl / ms / 1e9, 1),
                      "tokens_per_s": round(w["T"] / ms * 1e3, 1)}
    for name in ("c5_bf16", "c5_fp8"):
        sweep = {}
        for T in (64, 512, 4096, 32768):
            w, ms, kern, stats, fl, _ = bench_workload(name, steps, warmup, tokens=T, detail=False)
            entry = {"ms_per_step": round(ms, 4), "tokens_per_s": round(T / ms * 1e3, 1),
                     "gemm1_ms": kern["gemm1"]["ms"], "gemm2_ms": kern["gemm2"]["ms"]}
            if T <= 512:
                touched = w["E"] - stats["empty_experts"]
                entry["gbs"] = round(weight_stream_bytes(w, touched) / ms / 1e6, 1)
                entry["frac_hbm"] = round(entry["gbs"] / HBM_PEAK_GBS, 4)
            else:
                entry["tflops"] = round(fl / ms / 1e9, 1)
                entry["frac_mfma"] = round(entry["tflops"] / PEAK["fp8" if w["dtype"] == "fp8" else "bf16"], 4)
            sweep[str(T)] = entry
        out[name] = sweep
        torch.cuda.empty_cache()
    out["weight_quant_c4"] = weight_quant_rate(WORKLOADS["c4_fp8"], steps)
    return out


def weight_quant_rate(w, steps):
    """GB/s of the one-off e4m3 quantisation of the expert weights (3 B per element: bf16 in, e4m3 out)."""
    from fast_moe_amd.kernels import moe_fp8
    dev = torch.device("cuda:0")
    E, D, H, O = w["E"], w["D"], w["H"], w["O"]
    g = torch.Generator(device=dev).manual_seed(2)
    ws = [(torch.randn(E, H, D, generator=g, device=dev) * D ** -0.5).to(torch.bfloat16).permute(0, 2, 1) for _ in range(2)]
    ws.append((torch.randn(E, O, H, generator=g, device=dev) * H ** -0.5).to(torch.bfloat16).permute(0, 2, 1))
    stream = torch.cuda.current_stream(dev)

    def run():
        for t in ws:
            moe_fp8.quantize_expert_weights(t)

    run()
    torch.cuda.synchronize()
    ms = time_region(run, max(5, steps // 2), stream)
    nbytes = sum(t.numel() for t in ws) * 3 + sum(t.shape[0] * t.shape[2] for t in ws) * 4
    return {"ms": round(ms, 4), "gbs": round(nbytes / ms / 1e6, 1), "frac_hbm": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4)}


class ClockSampler:
    """Shader clock while the GPU works: `rocm-smi --showclocks` polled from a thread (a child
    process per sample; this process is not replaced).  The MFMA peak scales with this clock."""

    def __init__(self, period=0.25):
        self.samples, self.period, self._stop = [], period, threading.Event()
        self._thread = threading.Thread(target=self._run, daemon=True)

    def _run(self):
        while not self._stop.is_set():
            try:
                out = subprocess.run(["rocm-smi", "--showclocks"], capture_output=True, text=True, timeout=5).stdout
                m = re.search(r"sclk clock level: \d+: \((\d+)Mhz\)", out)
                if m:
                    self.samples.append(int(m.group(1)))
            except Exception:
                pass
            self._stop.wait(self.period)

    def __enter__(self):
        self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop.set()
        self._thread.join(timeout=10)


def sustained(fn, seconds, sampler_period=0.25):
    """Runs `fn` back to back for about `seconds` and samples the shader clock meanwhile."""
    stream = torch.cuda.current_stream()
    fn()
    torch.cuda.synchronize()
    with ClockSampler(sampler_period) as cs:
        t_end = time.perf_counter() + seconds
        n, t0 = 0, time.perf_counter()
        while time.perf_counter() < t_end:
            for _ in range(20):
                fn()
            torch.cuda.synchronize()
            n += 20
        ms = (time.perf_counter() - t0) * 1e3 / n
    s = sorted(cs.samples[1:] or cs.samples)
    clock = {"median_mhz": s[len(s) // 2], "min_mhz": s[0], "max_mhz": s[-1], "samples": len(s)} if s else None
    return ms, clock


def hbm_ceiling(gib=4, reps=20):
    """GB/s of kernels that do nothing but memory accesses over `gib` GiB (far beyond the 256 MB
    last-level cache): the library's probe kernel (16-byte accesses, one, two or eight per lane)
    and torch's own reduction, fill and copy.  The fraction-of-HBM figures of the
    quantisers and of the merge are to be read against these, not only against the 8 TB/s of the
    data sheet."""
    from fast_moe_amd.kernels.hip import _lib
    lib = _lib.load()
    dev = torch.device("cuda:0")
    nbytes = gib << 30
    buf = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    buf.view(torch.int32).random_(0, 1 << 20)
    stream = torch.cuda.current_stream(dev)
    out = {"bytes": nbytes, "launches": reps}

    def probe(mode, per_lane):
        _lib.check(lib.fmoe_hbm_probe(buf.data_ptr(), nbytes, mode, per_lane, stream.cuda_stream), "fmoe_hbm_probe")

    for name, mode in (("read", 0), ("write", 1), ("copy", 2)):
        for per_lane in (1, 2, 8):
            fn = lambda: probe(mode, per_lane)
            fn()
            torch.cuda.synchronize()
            ms = time_region(fn, reps, stream)
            out[f"probe_{name}_{per_lane}_per_lane"] = {"ms": round(ms, 4), "gbs": round(nbytes / ms / 1e6, 1),
                                                        "frac_hbm": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4)}
    as_f32, half = buf.view(torch.float32), nbytes // 2
    for name, fn, moved in (("torch_sum_fp32", lambda: as_f32.sum(), nbytes),
                            ("torch_fill", lambda: buf.fill_(1), nbytes),
                            ("torch_copy", lambda: buf[half:].copy_(buf[:half]), nbytes)):
        fn()
        torch.cuda.synchronize()
        ms = time_region(fn, reps, stream)
        out[name] = {"ms": round(ms, 4), "gbs": round(moved / ms / 1e6, 1),
                     "frac_hbm": round(moved / ms / 1e6 / HBM_PEAK_GBS, 4)}
    del buf
    torch.cuda.empty_cache()
    return out


def sustained_section(w, sample_clock, dense_reference, seconds=3.0):
    """Each GEMM of the workload run back to back for ~3 s: milliseconds per launch, TFLOP/s, and the
    shader clock rocm-smi reports meanwhile; with `dense_reference` the vendor's dense GEMM
    (torch.matmul) on one product of the same FLOPs (R x K x N with the experts' columns side by
    side) measured the same way.  bf16 workloads only for the dense reference."""
    dev = torch.device("cuda:0")
    inp = make_inputs(w, dev)
    path = GpuPath(w, inp)
    path.step()
    f1, f2 = flops_of(w)
    out = {}
    for name, fn, fl in (("gemm1", path.gemm1, f1), ("gemm2", path.gemm2, f2)):
        ms, clock = sustained(fn, seconds)
        peak = PEAK["fp8" if w["dtype"] == "fp8" else "bf16"]
        entry = {"ms": round(ms, 4), "tflops": round(fl / ms / 1e9, 1), "sclk": clock}
        if clock:
            entry["frac_of_peak_at_clock"] = round(fl / ms / 1e9 / (peak * clock["median_mhz"] / 2400.0), 4)
        out[name] = entry
    if dense_reference and w["dtype"] == "fp8":
        # the vendor's e4m3 GEMM with row-wise scales (torch._scaled_mm -> hipBLASLt), one product of
        # the same FLOPs per GEMM of the workload, operands quantised by the library's own quantiser
        from fast_moe_amd.kernels.hip import ops
        R = w["T"] * w["K"]
        hn = 2 * w["H"] if w["kind"] == "swiglu" else w["H"]
        for name, (m, k, n) in (("dense_gemm1", (R, w["D"], hn)), ("dense_gemm2", (R, w["H"], w["O"]))):
            try:
                qa, sa = ops.quant_rows_fp8(torch.randn(m, k, device=dev).to(torch.bfloat16))
                qb, sb = ops.quant_rows_fp8((torch.randn(n, k, device=dev) * k ** -0.5).to(torch.bfloat16))
                ra, rb = (1.0 / sa).view(m, 1).contiguous(), (1.0 / sb).view(1, n).contiguous()
                fn = lambda: torch._scaled_mm(qa, qb.t(), scale_a=ra, scale_b=rb, out_dtype=torch.bfloat16)
                fn()
                torch.cuda.synchronize()
                ms, clock = sustained(fn, seconds)
                fl = 2.0 * m * k * n
                entry = {"kernel": "torch._scaled_mm, e4m3fn x e4m3fn, row-wise fp32 scales, bf16 out",
                         "shape_mkn": [m, k, n], "ms": round(ms, 4), "tflops": round(fl / ms / 1e9, 1), "sclk": clock}
                if clock:
                    entry["frac_of_peak_at_clock"] = round(fl / ms / 1e9 / (PEAK["fp8"] * clock["median_mhz"] / 2400.0), 4)
            except Exception as exc:        # not every hipBLASLt build has the row-wise form
                entry = {"shape_mkn": [m, k, n], "unavailable": f"{type(exc).__name__}: {exc}"[:300]}
            out[name] = entry
    if dense_reference and w["dtype"] == "bf16":
        R = w["T"] * w["K"]
        hn = 2 * w["H"] if w["kind"] == "swiglu" else w["H"]
        for name, (m, k, n) in (("dense_gemm1", (R, w["D"], hn)), ("dense_gemm2", (R, w["H"], w["O"]))):
            a = torch.randn(m, k, device=dev).to(torch.bfloat16)
            b = (torch.randn(n, k, device=dev) * k ** -0.5).to(torch.bfloat16).t()
            ms, clock = sustained(lambda: torch.matmul(a, b), seconds)
            fl = 2.0 * m * k * n
            entry = {"shape_mkn": [m, k, n], "ms": round(ms, 4), "tflops": round(fl / ms / 1e9, 1), "sclk": clock}
            if clock:
                entry["frac_of_peak_at_clock"] = round(fl / ms / 1e9 / (PEAK["bf16"] * clock["median_mhz"] / 2400.0), 4)
            out[name] = entry
            del a, b
    return out


def tile_trace(w):
    """Where a tile's time goes inside the ring kernel, from a library built with -DFMOE_TRACE
    (`python -m fast_moe_amd.build --out fast_moe_amd/libfastmoe_hip_trace.so -DFMOE_TRACE`, run with
    FMOE_LIB_PATH=fast_moe_amd/libfastmoe_hip_trace.so): waves 0 and 4 of every block stamp the
    100 MHz real-time counter at a tile's start, the end of its main loop, after the next tile has
    been located and at the end of the epilogue (plus the row blocks inside the epilogue); the
    stamps of one launch of each GEMM are averaged over the tiles that have a predecessor and a
    successor in their block.  Stamped builds run slower than the product: the split is the result."""
    import numpy as np
    dev = torch.device("cuda:0")
    inp = make_inputs(w, dev)
    path = GpuPath(w, inp)
    path.step()
    path.step()
    torch.cuda.synchronize()
    grid = torch.cuda.get_device_properties(0).multi_processor_count // 8 * 8
    out = {}
    for which in ("gemm1", "gemm2"):
        buf = torch.zeros(3 * grid * 32 * 2 * 8, dtype=torch.int64, device=dev)
        fn = getattr(path, which)
        fn()
        torch.cuda.synchronize()
        os.environ["FMOE_TRACE_PTR"] = hex(buf.data_ptr())
        try:
            fn()
            torch.cuda.synchronize()
        finally:
            del os.environ["FMOE_TRACE_PTR"]
        full = buf.cpu().numpy().reshape(3, grid, 32, 2, 8).astype(np.float64)
        t, steps, inner = full[0], full[1], full[2]
        ntiles = (t[:, :, 0, 0] > 0).sum(1)
        if ntiles.max() == 0:
            return {"unavailable": "no stamps: the loaded library was not built with -DFMOE_TRACE"}
        groups = {}
        for g in (0, 1):
            rows = []
            for b in range(grid):
                for i in range(1, int(ntiles[b]) - 1):
                    r, q = t[b, i, g], inner[b, i, g]
                    d = steps[b, i, g]      # after double steps 0..3, before the second last, before the last
                    mid = r[6] / 2 - 6      # double steps between the fourth and the second last
                    rows.append([r[1] - r[0], r[2] - r[1], r[3] - r[2], t[b, i + 1, g, 0] - r[3],
                                 q[0] - r[2], q[4] - q[0], r[3] - q[4],
                                 d[0] - r[0], d[1] - d[0], d[2] - d[1], d[3] - d[2],
                                 (d[4] - d[3]) / mid if mid > 0 else 0.0, d[5] - d[4], r[1] - d[5]])
            m = np.mean(np.array(rows), axis=0) / 100.0       # 100 MHz ticks -> microseconds
            groups[f"waves_{'0_3' if g == 0 else '4_7'}"] = {
                "main_loop_us": round(m[0], 2), "locate_next_and_prefetch_us": round(m[1], 2),
                "epilogue_us": round(m[2], 2), "epilogue_end_to_next_tile_start_us": round(m[3], 2),
                "epilogue_before_first_row_block_us": round(m[4], 2), "epilogue_row_blocks_us": round(m[5], 2),
                "epilogue_after_last_row_block_us": round(m[6], 2),
                # the main loop by double step (a pair of K-slices): the first four, the average of
                # those in the middle, the last two (the last one ends with the wait for the tile's
                # own LDS-DMA stream)
                "double_steps_first_four_us": [round(v, 2) for v in m[7:11]],
                "double_step_middle_us": round(m[11], 3),
                "double_steps_last_two_us": [round(v, 2) for v in m[12:14]],
                "tiles_averaged": len(rows)}
        out[which] = dict(groups, k_slices=int(t[0, 0, 0, 6]), tiles_per_block_max=int(ntiles.max()))
    return out


def with_wq(entry, timing, flops):
    """fp8 workloads: the step of the default operator path (weight quantisation inside) beside the
    headline step (weights quantised once)."""
    ms = timing.pop("ms_per_step_weights_quantised_in_step", None)
    if ms:
        entry["ms_per_step_weights_quantised_in_step"] = round(ms, 4)
        entry["value_weights_quantised_in_step"] = round(flops / ms / 1e9, 2)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # (100 steps: the K-step figure then agrees with the per-step HIP-event median; with 20, the one
    # pipeline fill after the synchronisation and the final synchronisation weigh 2.5 % of the step)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c3_bf16", choices=sorted(WORKLOADS))
    ap.add_argument("--tokens", type=int, default=None, help="override the token count (C5 sweep)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary fp8 / bf16 workload")
    ap.add_argument("--backward", action="store_true",
                    help="time forward + backward of the bf16 SwiGLU workload instead of the forward metric")
    ap.add_argument("--sgmoe", action="store_true",
                    help="time the SGMoE layer (MRN router front-end + experts), forward and training step")
    ap.add_argument("--sample-clock", action="store_true",
                    help="run each GEMM of the workload back to back for ~3 s and report the shader clock "
                         "rocm-smi shows meanwhile (the MFMA peak scales with it)")
    ap.add_argument("--dense-reference", action="store_true",
                    help="also time the vendor's dense GEMM (torch.matmul) on the FLOP-equivalent single product "
                         "of each GEMM of the workload, with the shader clock, for scale")
    ap.add_argument("--hbm-ceiling", action="store_true",
                    help="also stream 4 GiB with kernels that only read, only write, and copy (fmoe_hbm_probe, and "
                         "torch's sum / fill_ / copy_ beside them): what the part gives a memory-bound kernel")
    ap.add_argument("--tile-trace", action="store_true",
                    help="per-tile split of the ring GEMMs (main loop / locate / epilogue) from a -DFMOE_TRACE build of "
                         "the library loaded through FMOE_LIB_PATH; see tile_trace()")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 512 MiB device copy, for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU with all experts local; expert parallelism is out of "
              "scope, so --gpus must be 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)

    if args.sgmoe:
        ms_eval, ms_front, ms_train, flops, (T, D, H, E, K) = run_sgmoe(args.steps, args.warmup, args.tokens or 16384)
        print(json.dumps({
            "metric": "sgmoe_forward_tflops", "value": round(flops / ms_eval / 1e9, 2), "unit": "TFLOP/s", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_eval, 4),
            "ms_router_front_end": round(ms_front, 4), "ms_training_step": round(ms_train, 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": f"SGMoE layer (layer norm, normalised-logit router, SiLU MLP experts, shared-expert "
                                   f"addmm), T={T}, E={E}, top-{K}, D={D}, H={H}"}}))
        return
    if args.backward:
        w = dict(WORKLOADS[args.workload])
        if w["kind"] != "swiglu" or w["dtype"] != "bf16":
            print("bench.py --backward: a bf16 swiglu workload is required", file=sys.stderr)
            sys.exit(2)
        if args.tokens:
            w["T"] = args.tokens
        ms, ms_fwd, flops = run_train(w, args.steps, args.warmup)
        print(json.dumps({
            "metric": "moe_fwd_bwd_tflops", "value": round(flops / ms / 1e9, 2), "unit": "TFLOP/s", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
            "ms_forward_with_saved_tensors": round(ms_fwd, 4), "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": f"{args.workload}: swiglu MoE forward + backward (input, weight and gate "
                                   f"gradients), T={w['T']}, E={w['E']}, top-{w['K']}, D={w['D']}, H={w['H']}",
                       "flops": "3 x forward GEMM FLOPs"}}))
        return
    w, ms, kernels, stats, flops, timing = bench_workload(args.workload, args.steps, args.warmup, args.tokens)
    dt = w["dtype"]
    g1 = kernels["gemm1"]
    line = {
        "metric": "moe_forward_tflops", "value": round(flops / ms / 1e9, 2), "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if dt == "bf16" else "fp8_e4m3", "data": "synthetic",
        "tokens_per_s": round(w["T"] / ms * 1e3, 1),
        "timing": {"method": "value: K back-to-back steps between two synchronisations; hot / cold: one HIP-event "
                             "pair per step, cold = a 512 MiB buffer rewritten before every step; kernels: HIP events "
                             "over max(K, 100) launches after 25 warm-up launches; the routing output tensors of the "
                             "previous step are reused (route_topk(out=)), every other output is allocated by its "
                             "operator; fp8: expert weights quantised once outside the step (fp8_weight= path), the "
                             "step with the weight quantisation inside it (the operators' default, as the reference "
                             "re-quantises per call) is reported as *_weights_quantised_in_step",
                   "hot_ms": timing.get("hot"), "cold_ms": timing.get("cold"),
                   "cold_value": round(flops / timing["cold"]["median"] / 1e9, 2) if timing.get("cold") else None},
        "config": {"workload": f"{args.workload}: {w['kind']} MoE forward, T={w['T']} tokens, E={w['E']} experts, "
                               f"top-{w['K']}, D={w['D']}, H={w['H']}, O={w['O']}, routing={w['routing']}",
                   "tokens": w["T"], "experts": w["E"], "top_k": w["K"], "d_model": w["D"], "hidden": w["H"],
                   "routing": stats},
        "kernels": kernels,
        "roofline": {"bound": "mfma", "kernel": "grouped_gemm (gemm1: gather + GEMM + " +
                     ("SwiGLU" if w["kind"] == "swiglu" else "SiLU") + " epilogue)",
                     "achieved": g1["tflops"], "peak": PEAK[dt], "unit": "TFLOP/s",
                     "frac": round(g1["tflops"] / PEAK[dt], 4),
                     "traffic": measured_traffic_bytes(args.workload) if not args.tokens else None},
    }
    with_wq(line, timing, flops)
    if not args.no_extra:
        other = {"c3_bf16": "c4_fp8", "c4_fp8": "c3_bf16"}.get(args.workload)
        if other:
            w2, ms2, k2, _, fl2, tm2 = bench_workload(other, args.steps, args.warmup)
            line["extra"] = {other: {"value": round(fl2 / ms2 / 1e9, 2), "unit": "TFLOP/s",
                                     "ms_per_step": round(ms2, 4), "tokens_per_s": round(w2["T"] / ms2 * 1e3, 1),
                                     "hot_ms": tm2.get("hot"), "cold_ms": tm2.get("cold"), "kernels": k2}}
            with_wq(line["extra"][other], tm2, fl2)
            line["extra"].update(extra_workloads(args.steps, args.warmup))
    if args.sample_clock or args.dense_reference:
        line["sustained"] = sustained_section(w, args.sample_clock, args.dense_reference)
    if args.hbm_ceiling:
        line["hbm_ceiling"] = hbm_ceiling()
    if args.tile_trace:
        line["tile_trace"] = tile_trace(w)
    if args.calibrate_copy:      # a kernel of known traffic: 512 MiB read + 512 MiB written
        src = torch.empty(512 << 20, dtype=torch.uint8, device="cuda:0").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        line["calibration"] = {"kernel": "torch Tensor.copy_ of 536870912 bytes (uint8)", "launches": 3}
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(w)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
