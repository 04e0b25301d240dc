#!/usr/bin/env python3
"""Benchmark of the block-INT8 fused-MoE path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--tokens M]
                    [--sweep {default,none,full}] [--no-cpu-baseline]

A step is one call of ``fused_experts_impl_int8`` on one batch of synthetic tokens with
every input already resident in HBM.  Between steps a 512 MiB buffer is read through so
that weights are streamed from HBM and not served from the 256 MB Infinity Cache (read, not
overwritten: an overwrite leaves the cache full of dirty lines whose write-back takes place
inside the timed step - 5 to 25 us of it, `--flush write` shows the difference); the
step time is taken with HIP events on the launching stream and excludes that flush.
ms_per_step is the median of the timed steps (mean and min are reported next to it).  The
headline is timed in the library's default arithmetic (acc = fma(f32(d) * a_s, b_s, acc) per K block, the
mode the GPU parity tests compare bit for bit with the CPU checker); ms_per_step_separate_order and
ms_per_step_fused_scale are the same call with LO_GEMM_SEPARATE_ORDER and LO_GEMM_FUSED_SCALE.  `roofline`
also carries, as flat scalars, the sweep's figures for the targets of the path (the DeepSeek-V3-shaped
layer at M >= 4096 against the int8 MFMA peak, M <= 64 against the HBM peak) and the ceiling the scale
arithmetic puts on the matrix pipe (fold_insts_per_elem; mfma_cap_frac = the rate lo_measure_mfma_issue_rate
reports for MFMAs with that many vector instructions between them over the published peak, measured in
this run; achieved_over_cap; issue_ceiling_tops holds the measured rates).  The last line printed is one JSON object (fields: metric, value, unit,
ms_per_step, roofline, cpu_baseline, stage_ms, routers, sweep).
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import statistics
import sys
import time

import torch

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
INT8_PEAK_TOPS = 5000.0        # MI355X dense INT8 MFMA, published (5.0 POP/s)

PROFILES = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles")


def profile_record(workload, tokens):
    """What the committed rocprofv3 summary under profiles/ says about the dominant kernel of
    (workload, tokens): a line `bench-key: workload=... tokens=... kernel=... avg_us=... median_us=...
    min_us=... traffic_bytes=...` in one of the .md files (traffic_bytes = FETCH_SIZE x 2.00 x 1024 +
    WRITE_SIZE x 1.00 x 1024 per dispatch, the factors calibrated in the same runs on kernels of known
    size).  None if that point was not profiled: nothing is made up here."""
    try:
        names = sorted(os.listdir(PROFILES))
    except OSError:
        return None
    for name in names:
        if not name.endswith(".md"):
            continue
        for line in open(os.path.join(PROFILES, name)):
            if not line.startswith("bench-key:"):
                continue
            kv = dict(tok.split("=", 1) for tok in line[len("bench-key:"):].split() if "=" in tok)
            if kv.get("workload") == workload and kv.get("tokens") == str(tokens):
                rec = {"file": f"profiles/{name}", "kernel": kv.get("kernel")}
                for k in ("avg_us", "median_us", "min_us"):
                    rec[k] = float(kv[k]) if k in kv else None
                rec["traffic_bytes"] = int(kv["traffic_bytes"]) if "traffic_bytes" in kv else None
                return rec
    return None


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=50)
    p.add_argument("--warmup", type=int, default=5)
    p.add_argument("--workload", default="qwen3-30b-a3b")
    p.add_argument("--tokens", type=int, default=8192)
    p.add_argument("--sweep", default="default", choices=["default", "none", "full"])
    p.add_argument("--no-cpu-baseline", action="store_true")
    p.add_argument("--flush", default="read", choices=["read", "write"],
                   help="how the Infinity Cache is evicted between steps: by reading 512 MiB or by overwriting them")
    p.add_argument("--block-size-m", type=int, default=0)
    p.add_argument("--row-major-weights", action="store_true",
                   help="keep w1/w2 row-major instead of the load-time pre-shuffled layout")
    p.add_argument("--scale-order", default="contract", choices=["contract", "separate", "fused"],
                   help="scale arithmetic per 128-wide K block.  contract: acc = fma(f32(d) * a_s, b_s, acc), the "
                        "library default, bit-exact against the CPU checker; separate: acc + (f32(d) * a_s) * b_s "
                        "(LO_GEMM_SEPARATE_ORDER, bit-exact against the checker in that order); fused: "
                        "fma(f32(d), a_s * b_s, acc) (LO_GEMM_FUSED_SCALE, tolerance-matched)")
    return p.parse_args()


class Flusher:
    """Evicts the Infinity Cache between steps: a max-reduction reads 512 MiB ("write": a fill overwrites them)."""

    def __init__(self, dev, mode="read"):
        self.buf = torch.zeros(512 * 1024 * 1024 // 4, dtype=torch.int32, device=dev)
        self.i = 0
        self.mode = mode

    def __call__(self):
        self.i += 1
        if self.mode == "read":
            self.buf.max()
        else:
            self.buf.fill_(self.i)


def time_steps(fn, steps, warmup, flush):
    """Mean / median / min of `steps` event-timed calls (ms), each after a cache flush."""
    for _ in range(warmup):
        flush()
        fn()
    torch.cuda.synchronize()
    evs = []
    for _ in range(steps):
        flush()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        evs.append((a, b))
    torch.cuda.synchronize()
    ts = [a.elapsed_time(b) for a, b in evs]
    return sum(ts) / len(ts), statistics.median(ts), min(ts)


class Point:
    """One (layer, M) measurement: whole path plus the two GEMM kernels on their own."""

    def __init__(self, layer, weights, M, dev, seed=0, emap=None, pool=None):
        from lightop_amd import workloads as wl

        self.layer, self.M, self.dev = layer, M, dev
        self.w1, self.w2, self.w1s, self.w2s = weights
        self.emap = wl.expert_map_for(layer, dev) if emap is None else emap
        # a pool of different batches so that consecutive steps hit different experts
        pool = pool or (8 if M <= 64 else 2)
        self.batches = [tuple(t.to(dev) for t in wl.make_inputs(layer, M, seed=seed + i)) for i in range(pool)]
        self.cache13 = torch.empty(M * layer.top_k * max(2 * layer.I, layer.H), dtype=torch.bfloat16, device=dev)
        self.i = 0
        ops = byts = sloc = eact = 0
        for (_, _, ids) in self.batches:
            o, b, s, e = wl.algorithmic_work(layer, ids, self.emap)
            ops, byts, sloc, eact = ops + o, byts + b, sloc + s, eact + e
        n = len(self.batches)
        self.ops, self.bytes, self.S_loc, self.E_act = ops / n, byts / n, sloc / n, eact / n

    def step(self, bs=0, flags=0):
        from lightop_amd.moe import fused_experts_impl_int8, fused_experts_impl_w4a8

        x, tw, ids = self.batches[self.i % len(self.batches)]
        self.i += 1
        L = self.layer
        if L.weight_bits == 4:
            return fused_experts_impl_w4a8(
                x, self.w1, self.w2, tw, ids, self.cache13, global_num_experts=L.E_global, expert_map=self.emap,
                w1_scale=self.w1s, w2_scale=self.w2s, block_shape=None if L.quant == "channel" else [1, 128],
                lightop_amd_block_size_m=bs, lightop_amd_flags=flags)
        if L.quant == "channel":
            return fused_experts_impl_int8(
                x, self.w1, self.w2, tw, ids, self.cache13, use_int8_w8a8=True, per_channel_quant=True,
                global_num_experts=L.E_global, expert_map=self.emap, w1_scale=self.w1s, w2_scale=self.w2s,
                block_shape=None, lightop_amd_block_size_m=bs)
        return fused_experts_impl_int8(
            x, self.w1, self.w2, tw, ids, self.cache13, use_int8_w8a8=True, global_num_experts=L.E_global,
            expert_map=self.emap, w1_scale=self.w1s, w2_scale=self.w2s, block_shape=[128, 128],
            lightop_amd_block_size_m=bs, lightop_amd_flags=flags)

    def stage_times(self, steps, warmup, flush, bs=0, order_flags=0):
        """Event-timed duration of each stage kernel launched on its own (ms, median)."""
        from lightop_amd import moe
        from lightop_amd.quant import per_token_group_quant_int8

        L = self.layer
        wflag = _lib_flags_w4(L)
        if bs == 0:
            shape = None if L.quant == "channel" else ([1, 128] if L.weight_bits == 4 else [128, 128])
            bs = moe.get_w8a8moe_json(self.M, L.E, 2 * L.I, L.H, L.I, True, shape, L.top_k, L.E_global,
                                      preshuffled=bool(getattr(self.w1, "lo_preshuffled", False)),
                                      int4=L.weight_bits == 4)[0]["BLOCK_SIZE_M"]
        cfg = {"BLOCK_SIZE_M": bs}
        S = self.M * L.top_k
        c3 = self.cache13[: S * L.H].view(self.M, L.top_k, L.H)
        out = torch.empty(self.M, L.H, dtype=torch.bfloat16, device=self.dev)
        if L.quant == "channel":
            return self.stage_times_channel(steps, warmup, flush, bs), bs
        names = ["quant", "align", "gemm1_silu_quant", "gemm2", "moe_sum"]
        acc = {n: [] for n in names}
        # With an expert_map the whole path leaves the rows of other ranks' slots untouched and
        # reduces over the slot mask of the alignment: the stages on their own do the same here.
        ep = self.emap is not None
        g2flag = wflag | (_lib_skip_nonlocal() if ep else 0)
        for it in range(warmup + steps):
            x, tw, ids = self.batches[it % len(self.batches)]
            flush()
            ev = [torch.cuda.Event(enable_timing=True) for _ in range(6)]
            ev[0].record()
            a1q, a1s = per_token_group_quant_int8(x, 128)
            ev[1].record()
            if ep:
                s, e, p = _align_buffers(ids, bs, L.E_global)
                mask = torch.empty(S, dtype=torch.bool, device=self.dev)
                moe.moe_align_block_size_out(ids, L.E_global, bs, s, e, p, self.emap, mask)
            else:
                mask = None
                s, e, p = moe.moe_align_block_size(ids, bs, L.E_global, self.emap)
            ev[2].record()
            a2q, a2s = moe.invoke_fused_moe_gemm1_silu_quant(a1q, self.w1, a1s, self.w1s, tw, s, e, p, False,
                                                             L.top_k, S, cfg,
                                                             flags=wflag | order_flags, global_num_experts=L.E_global)
            ev[3].record()
            moe.invoke_fused_moe_kernel_int8(a2q, self.w2, c3, a2s, self.w2s, tw, s, e, p, True, 1, cfg,
                                             flags=g2flag | order_flags, global_num_experts=L.E_global)
            ev[4].record()
            moe.moe_sum(c3, out, expert_mask=mask)
            ev[5].record()
            if it >= warmup:
                torch.cuda.synchronize()
                for i, n in enumerate(names):
                    acc[n].append(ev[i].elapsed_time(ev[i + 1]))
        return {n: statistics.median(v) for n, v in acc.items()}, bs

    def stage_times_channel(self, steps, warmup, flush, bs):
        """The six launches of the per-channel path, each on its own (ms, median)."""
        from lightop_amd import fuse_silu_mul_quant, moe
        from lightop_amd.quant import per_token_quant_int8

        L = self.layer
        cfg = {"BLOCK_SIZE_M": bs}
        S = self.M * L.top_k
        c1 = self.cache13[: S * 2 * L.I].view(S, 2 * L.I)
        c3 = self.cache13[: S * L.H].view(self.M, L.top_k, L.H)
        out = torch.empty(self.M, L.H, dtype=torch.bfloat16, device=self.dev)
        names = ["quant", "align", "gemm1", "silu_mul_quant", "gemm2", "moe_sum"]
        acc = {n: [] for n in names}
        for it in range(warmup + steps):
            x, tw, ids = self.batches[it % len(self.batches)]
            flush()
            ev = [torch.cuda.Event(enable_timing=True) for _ in range(7)]
            ev[0].record()
            a1q, a1s = per_token_quant_int8(x)
            ev[1].record()
            s, e, p = moe.moe_align_block_size(ids, bs, L.E_global, self.emap)
            ev[2].record()
            if L.weight_bits == 4:
                moe.invoke_fused_moe_kernel_w4a8(a1q, self.w1, c1, a1s, self.w1s, None, None, s, e, p, False, L.top_k,
                                                 cfg, global_num_experts=L.E_global)
            else:
                moe.moe_gemm_w8a8(a1q, self.w1, c1, a1s, self.w1s, None, s, e, p, L.top_k, cfg,
                                  global_num_experts=L.E_global)
            ev[3].record()
            a2q, a2s = fuse_silu_mul_quant(c1)
            ev[4].record()
            if L.weight_bits == 4:
                moe.invoke_fused_moe_kernel_w4a8(a2q, self.w2, c3, a2s, self.w2s, None, tw, s, e, p, True, 1, cfg,
                                                 global_num_experts=L.E_global)
            else:
                moe.moe_gemm_w8a8(a2q, self.w2, c3, a2s, self.w2s, tw, s, e, p, 1, cfg,
                                  global_num_experts=L.E_global)
            ev[5].record()
            moe.moe_sum(c3, out)
            ev[6].record()
            if it >= warmup:
                torch.cuda.synchronize()
                for i, n in enumerate(names):
                    acc[n].append(ev[i].elapsed_time(ev[i + 1]))
        return {n: statistics.median(v) for n, v in acc.items()}


def graph_ms(pt, steps, flush, bs, flags):
    """Mean time (ms) of one step replayed from a HIP graph: the five launches of the path
    without their host-side launch cost.  None if the capture is refused."""
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                pt.step(bs, flags)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            pt.step(bs, flags)
        mean_ms, _, _ = time_steps(g.replay, steps, 2, flush)
        del g
        return mean_ms
    except Exception as e:  # report, do not fail the benchmark
        print(f"[graph] capture failed for M={pt.M}: {e}", file=sys.stderr, flush=True)
        return None


def graph_launch_floor(steps, flush):
    """Event-timed cost (us) of one trivial kernel launched eagerly and replayed from a HIP graph: what a
    graph launch itself adds on this runtime, whatever the graph holds."""
    try:
        t = torch.zeros(64, device="cuda")
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            t.add_(1.0)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        _, eager, _ = time_steps(lambda: t.add_(1.0), steps, 3, flush)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            t.add_(1.0)
        _, replay, _ = time_steps(g.replay, steps, 3, flush)
        del g
        return {"eager_us": round(eager * 1e3, 2), "replay_us": round(replay * 1e3, 2)}
    except Exception as e:
        print(f"[graph] floor measurement failed: {e}", file=sys.stderr, flush=True)
        return None


def _lib_flags_w4(layer):
    from lightop_amd import _lib

    return _lib.LO_GEMM_W4 if layer.weight_bits == 4 else 0


def _lib_skip_nonlocal():
    from lightop_amd import _lib

    return _lib.LO_GEMM_SKIP_NONLOCAL


def _align_buffers(ids, bs, num_experts):
    """Output buffers of the alignment, sized as moe_align_block_size sizes them."""
    numel = ids.numel()
    cap = numel + num_experts * (bs - 1)
    if numel < num_experts:
        cap = min(numel * bs, cap)
    dev = ids.device
    return (torch.empty(cap, dtype=torch.int32, device=dev), torch.empty((cap + bs - 1) // bs, dtype=torch.int32, device=dev),
            torch.empty(1, dtype=torch.int32, device=dev))


def measure_point(pt, steps, warmup, flush, bs, flags):
    mean_ms, med_ms, min_ms = time_steps(lambda: pt.step(bs, flags), steps, warmup, flush)
    g_ms = graph_ms(pt, steps, flush, bs, flags) if pt.M <= 64 else None
    t = med_ms * 1e-3
    L = pt.layer
    hbm = pt.bytes / t / 1e9
    tops = pt.ops / t / 1e12
    t_hbm, t_mfma = pt.bytes / (HBM_PEAK_GBS * 1e9), pt.ops / (INT8_PEAK_TOPS * 1e12)
    bound = "mfma" if t_mfma > t_hbm else "hbm"
    return {
        "workload": L.name, "tokens": pt.M, "ms_per_step": round(med_ms, 4), "ms_mean": round(mean_ms, 4),
        "ms_min": round(min_ms, 4), "tokens_per_s": round(pt.M / t, 1), "int8_tops": round(tops, 2),
        "hbm_gbs": round(hbm, 1), "S_loc": pt.S_loc, "E_act": pt.E_act, "bound": bound,
        "roofline_frac": round((tops / INT8_PEAK_TOPS) if bound == "mfma" else (hbm / HBM_PEAK_GBS), 4),
        "frac_hbm": round(hbm / HBM_PEAK_GBS, 4), "frac_mfma": round(tops / INT8_PEAK_TOPS, 4),
        "ms_graph_replay": None if g_ms is None else round(g_ms, 4),
    }


def expert_buckets(layer, weights, M, dev, steps, warmup, flush, flags):
    """Skewed routing: the experts split into those whose share of the batch is compute-bound (more
    slots than half the ridge point, 2 * slots op/B >= 629 op/B) and those that stream their weights
    for a handful of tokens.  Each bucket is timed on its own by running the whole path with an
    expert_map that hides the other bucket (those slots become -1 blocks and are skipped), and set
    against its own roofline."""
    from lightop_amd import workloads as wl

    ridge_slots = INT8_PEAK_TOPS * 1e12 / (HBM_PEAK_GBS * 1e9) / 2.0
    ids = wl.make_inputs(layer, M, seed=0)[2]
    counts = torch.bincount(ids.reshape(-1).long(), minlength=layer.E_global)
    out = []
    for name, sel in (("compute-bound experts", counts >= ridge_slots), ("weight-streaming experts", counts < ridge_slots)):
        if not bool(sel.any()):
            continue
        emap = torch.where(sel, torch.arange(layer.E_global), torch.full((layer.E_global,), -1)).to(torch.int32)
        pt = Point(layer, weights, M, dev, emap=emap.to(dev), pool=1)
        mean_ms, med_ms, min_ms = time_steps(lambda: pt.step(0, flags), steps, warmup, flush)
        t = med_ms * 1e-3
        out.append({"bucket": name, "experts": int(sel.sum()), "slots": int(counts[sel].sum()),
                    "slots_per_expert_min": int(counts[sel].min()), "slots_per_expert_max": int(counts[sel].max()),
                    "ms": round(med_ms, 4), "int8_tops": round(pt.ops / t / 1e12, 1),
                    "hbm_gbs": round(pt.bytes / t / 1e9, 1), "frac_mfma": round(pt.ops / t / 1e12 / INT8_PEAK_TOPS, 4),
                    "frac_hbm": round(pt.bytes / t / 1e9 / HBM_PEAK_GBS, 4)})
        del pt
    return out


def router_times(layer, M, dev, steps, warmup):
    """Mean time (us) per call of the two routers that produce topk_ids/topk_weights, launched
    back to back on M rows of fp32 logits over the layer's global experts (events around the
    whole loop, so at small M this is the launch rate of the host; the kernels' own durations are
    in profiles/router_kernels.md)."""
    from lightop_amd.moe import moe_fused_gate, topk_softmax

    E, k = layer.E_global, layer.top_k
    logits = torch.randn(M, E, device=dev)
    bias = torch.zeros(E, device=dev)
    w = torch.empty(M, k, dtype=torch.float32, device=dev)
    idx = torch.empty(M, k, dtype=torch.int32, device=dev)
    n_group = layer.n_group if layer.routing.startswith("grouped") else 1
    tg = layer.topk_group if layer.routing.startswith("grouped") else 1
    fns = {"topk_softmax": lambda: topk_softmax(w, idx, None, logits, True),
           "moe_fused_gate": lambda: moe_fused_gate(logits, bias, n_group, tg, k, 0, 2.5)}
    out = []
    byts = M * E * 4 + M * k * 8
    for name, fn in fns.items():
        for _ in range(warmup):
            fn()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        a.record()
        for _ in range(steps):
            fn()
        b.record()
        torch.cuda.synchronize()
        us = a.elapsed_time(b) * 1e3 / steps
        out.append({"kernel": name, "tokens": M, "experts": E, "topk": k, "us_per_call": round(us, 2),
                    "hbm_gbs": round(byts / us / 1e3, 1)})
    return out


def cpu_baseline(layer, weights, M_sample, seed=0):
    """The torch-CPU restatement of the reference path on the host cores, on the first
    M_sample tokens of the benchmark's batch."""
    from lightop_amd import workloads as wl
    from oracle import torch_ref

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    w1, w2, w1s, w2s = weights
    x, tw, ids = wl.make_inputs(layer, M_sample, seed=seed)
    emap = wl.expert_map_for(layer)
    if layer.weight_bits == 4 and layer.quant == "channel":
        return None  # no torch restatement of this form is kept: the C oracle checks it in the tests
    ref = torch_ref.torch_w4a8_group_moe if layer.weight_bits == 4 else (
        torch_ref.torch_w8a8_per_column_moe if layer.quant == "channel" else torch_ref.torch_w8a8_block_int8_moe)
    runs = []
    for i in range(4):  # one warm-up, three timed
        t0 = time.perf_counter()
        ref(x, w1, w2, w1s, w2s, tw, ids, expert_map=emap)
        runs.append(time.perf_counter() - t0)
    dt = statistics.median(runs[1:])
    return {"value": round(M_sample / dt, 2), "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{layer.name}, first {M_sample} tokens of the same synthetic batch, median of three runs "
                      f"after one warm-up of oracle/torch_ref.py ({dt:.1f} s each), torch {torch.__version__} CPU"}


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU only (one process, one MI355X, no collectives); "
              f"--gpus {args.gpus} is not supported. Sharding by experts is a design note only.",
              file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    from lightop_amd import _lib, workloads as wl

    _lib.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    flush = Flusher(dev, args.flush)
    order_flag = {"contract": 0, "separate": _lib.LO_GEMM_SEPARATE_ORDER, "fused": _lib.LO_GEMM_FUSED_SCALE}
    flags_default = order_flag[args.scale_order]
    # Vector instructions the fold spends per accumulator element and K block, and the rate the matrix pipe
    # reaches at best under that load: measured live with a loop of nothing but int8 MFMAs, each followed by
    # its share of the fold (two elements per v_mfma_i32_16x16x64_i8) as independent v_fma_f32, two waves per
    # SIMD, on random operand bytes (the clock this chip holds depends on how many operand bits toggle; the
    # same loop on zeros and the MFMAs alone are reported next to it).
    fold_insts = {"contract": 3, "separate": 4, "fused": 2}[args.scale_order]

    def issue_rate(valu_per_mfma, random_operands):
        out = ctypes.c_double(0.0)
        _lib.check(_lib.lib().lo_measure_mfma_issue_rate(valu_per_mfma, int(random_operands), 40000,
                                                         ctypes.c_void_p(torch.cuda.current_stream().cuda_stream),
                                                         ctypes.byref(out)))
        return out.value / 1e12

    issue = {"mfma_only_zero_operands_tops": issue_rate(0, False), "mfma_only_tops": issue_rate(0, True),
             "mfma_with_fold_tops": issue_rate(2 * fold_insts, True)}
    mfma_cap = min(1.0, issue["mfma_with_fold_tops"] / INT8_PEAK_TOPS)

    from lightop_amd.moe import preshuffle_moe_scale_int4, preshuffle_moe_weight, preshuffle_moe_weight_int4

    cpu_weights = []

    def load_weights(lay, keep_cpu_copy=False):
        """Synthetic checkpoint -> device, then the one-time load-time layout change."""
        w1, w2, w1s, w2s = wl.make_weights(lay, seed=0, device=dev, gen_device="cuda")
        if keep_cpu_copy:
            cpu_weights.extend(t.cpu() for t in (w1, w2, w1s, w2s))
        if lay.weight_bits == 4:
            w1, w2 = preshuffle_moe_weight_int4(w1), preshuffle_moe_weight_int4(w2)
            if lay.quant != "channel":
                w1s, w2s = preshuffle_moe_scale_int4(w1s), preshuffle_moe_scale_int4(w2s)
        elif not args.row_major_weights:
            w1, w2 = preshuffle_moe_weight(w1), preshuffle_moe_weight(w2)
        return w1, w2, w1s, w2s

    layer = wl.LAYERS[args.workload]
    weights = load_weights(layer, keep_cpu_copy=not args.no_cpu_baseline and layer.weight_bytes < 8e9)
    pt = Point(layer, weights, args.tokens, dev)
    head = measure_point(pt, args.steps, args.warmup, flush, args.block_size_m, flags_default)
    # the other scale orders, for comparison (block form only: the per-channel form has one order)
    others = {}
    if layer.quant != "channel":
        for name, fl in order_flag.items():
            if name != args.scale_order:
                others[name] = time_steps(lambda: pt.step(args.block_size_m, fl), args.steps, args.warmup, flush)[1]
    stages, bs_used = pt.stage_times(args.steps, args.warmup, flush, args.block_size_m, order_flags=flags_default)
    # host time of one call at one token: launches and marshalling only, nothing waited for
    host_us = None
    if layer.quant != "channel":
        p1 = Point(layer, weights, 1, dev, pool=1)
        for _ in range(20):
            p1.step(0, flags_default)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(200):
            p1.step(0, flags_default)
        host_us = (time.perf_counter() - t0) / 200 * 1e6
        torch.cuda.synchronize()
        del p1
    shape = None if layer.quant == "channel" else ([1, 128] if layer.weight_bits == 4 else [128, 128])
    from lightop_amd import moe as _moe
    tile1, tile2 = _moe.get_w8a8moe_json(args.tokens, layer.E, 2 * layer.I, layer.H, layer.I, True, shape, layer.top_k,
                                         layer.E_global, preshuffled=not args.row_major_weights,
                                         int4=layer.weight_bits == 4)

    # dominant kernel: the first grouped GEMM with its fused SiLU*mul + re-quantisation
    L = layer
    g1_ops = 4.0 * pt.S_loc * L.I * L.H
    # weights and block scales of the active experts once, int8 activations and their
    # group scales in (M rows) and out (S_loc rows)
    g1_w = (L.I * L.H + 4 * 2 * L.I * (L.H // 128)) if L.weight_bits == 4 \
        else (2 * L.I * L.H + 4 * (2 * L.I // 128) * (L.H // 128))
    g1_bytes = pt.E_act * g1_w + args.tokens * (L.H + 4 * L.H // 128) + pt.S_loc * (L.I + 4 * L.I // 128)
    if L.quant == "channel":  # whole-row scales; bf16 [S, 2I] out instead of int8 [S, I]
        g1_w = 2 * L.I * L.H * L.weight_bits // 8 + 4 * 2 * L.I
        g1_bytes = pt.E_act * g1_w + args.tokens * (L.H + 4) + pt.S_loc * 2 * L.I * 2
    g1_name = "gemm1" if L.quant == "channel" else "gemm1_silu_quant"
    g1_t = stages[g1_name] * 1e-3
    if head["bound"] == "mfma":
        ach, peak, unit = g1_ops / g1_t / 1e12, INT8_PEAK_TOPS, "TFLOP/s"
    else:
        ach, peak, unit = g1_bytes / g1_t / 1e9, HBM_PEAK_GBS, "GB/s"
    prof = profile_record(layer.name, args.tokens)
    # the tile query names the kernel the stage call launched (unless the block size was forced)
    kname = tile1["kernel_name"] if args.block_size_m in (0, tile1["BLOCK_SIZE_M"]) else f"block_size_m={bs_used}"
    if kname.startswith("dec_gemm1"):  # a few tokens: the whole-path call runs its two-launch path, while
        kname = "moe_gemm_ws_kernel"   # stage_ms and this record time the stage entry points on their own
    roofline = {"bound": head["bound"], "achieved": round(ach, 2), "peak": peak, "unit": unit,
                "frac": round(ach / peak, 4), "traffic": None if prof is None else prof["traffic_bytes"],
                "algorithmic_bytes": int(g1_bytes), "algorithmic_ops": int(g1_ops),
                "kernel": kname + (" (GEMM1, per-channel scales in the epilogue)" if L.quant == "channel"
                                   else "<FUSED_ACT, 160-token blocks> (GEMM1 + SiLU*mul + 1x128 re-quant)" if bs_used == 160
                                   else "<FUSED_ACT> (GEMM1 + SiLU*mul + 1x128 re-quant)"),
                "kernel_ms": round(stages[g1_name], 4),
                "scale_order": args.scale_order,
                "fold_insts_per_elem": fold_insts if L.quant != "channel" else 0,
                "mfma_cap_frac": round(mfma_cap, 3) if L.quant != "channel" else 1.0,
                "issue_ceiling_tops": {k: round(v, 1) for k, v in issue.items()},
                "profile": None if prof is None else prof["file"],
                "profile_kernel_us": None if prof is None else {k: prof[k] for k in ("avg_us", "median_us", "min_us")},
                "note": "TFLOP/s stands for int8 TOP/s (multiply and add counted separately); kernel_ms is the "
                        "median of HIP-event timings of the stage launched on its own; traffic and "
                        "profile_kernel_us are read from the committed rocprofv3 summary named in `profile`"}

    sweep = []
    if args.sweep != "none":
        plan = [(wl.QWEN3_30B, [1, 8, 32, 128, 512, 2048, 8192]), (wl.DSV3_EP, [1, 16, 64, 256, 1024, 4096])]
        plan.append((wl.QWEN3_235B_W4, [1, 32, 256, 2048]))
        plan.append((wl.QWEN3_235B_W4_PC, [32, 2048, 8192]))  # the reference's own W4A8 form
        plan.append((wl.QWEN3_30B_PC, [32, 512, 8192]))
        plan.append((wl.DSV3_EP_PC, [64, 4096]))
        plan.append((wl.DSV3_FULL, [8192]))  # all 256 experts resident (11.3 GB), Zipf-skewed routing
        sw_steps, sw_warm = max(10, args.steps // 2), max(2, args.warmup // 2)
        for lay, Ms in plan:
            w = weights if lay.name == layer.name else load_weights(lay)
            for M in Ms:
                p2 = Point(lay, w, M, dev)
                sweep.append(measure_point(p2, sw_steps, sw_warm, flush, 0, flags_default))
                if lay.routing.endswith("zipf"):
                    sweep[-1]["expert_buckets"] = expert_buckets(lay, w, M, dev, sw_steps, sw_warm, flush, flags_default)
                print(f"[sweep] {json.dumps(sweep[-1])}", file=sys.stderr, flush=True)
                del p2
            if lay.name != layer.name:
                del w
                torch.cuda.empty_cache()

    cpu = None
    if cpu_weights:
        cpu = cpu_baseline(layer, cpu_weights, min(args.tokens, 8192))

    # The targets of the path, as flat scalars next to the dominant kernel's figures: the DeepSeek-V3-shaped
    # layer at M >= 4096 against the int8 MFMA peak, decode sizes against the HBM peak.
    def sw(workload, M, key, scale=1.0):
        for r in sweep:
            if r["workload"] == workload and r["tokens"] == M:
                return None if r.get(key) is None else round(r[key] * scale, 4)
        return None

    def hot_bucket():
        for r in sweep:
            if r["workload"] == "deepseek-v3-full":
                for b in r.get("expert_buckets", []):
                    if b["bucket"].startswith("compute-bound"):
                        return b["frac_mfma"]
        return None

    roofline.update({
        "achieved_over_cap": round(roofline["frac"] / roofline["mfma_cap_frac"], 4) if head["bound"] == "mfma" else None,
        "gemm2_ms": round(stages.get("gemm2", 0.0), 4), "moe_sum_ms": round(stages.get("moe_sum", 0.0), 4),
        "profile_avg_us": None if prof is None else prof["avg_us"],
        "profile_median_us": None if prof is None else prof["median_us"],
        "ms_per_step_fused_scale": None if "fused" not in others else round(others["fused"], 4),
        "dsv3_full_M8192_ms": sw("deepseek-v3-full", 8192, "ms_per_step"),
        "dsv3_full_M8192_frac_mfma": sw("deepseek-v3-full", 8192, "frac_mfma"),
        "dsv3_full_hot_bucket_frac_mfma": hot_bucket(),
        "dsv3_ep_M4096_ms": sw("deepseek-v3-ep8-share", 4096, "ms_per_step"),
        "dsv3_ep_M4096_frac_hbm": sw("deepseek-v3-ep8-share", 4096, "frac_hbm"),
        "dsv3_ep_M64_frac_hbm": sw("deepseek-v3-ep8-share", 64, "frac_hbm"),
        "dsv3_ep_M16_frac_hbm": sw("deepseek-v3-ep8-share", 16, "frac_hbm"),
        "dsv3_ep_M1_us": sw("deepseek-v3-ep8-share", 1, "ms_per_step", 1e3),
        "qwen3_M2048_ms": sw("qwen3-30b-a3b", 2048, "ms_per_step"),
        "qwen3_M32_frac_hbm": sw("qwen3-30b-a3b", 32, "frac_hbm"),
        "qwen3_M8_frac_hbm": sw("qwen3-30b-a3b", 8, "frac_hbm"),
        "qwen3_M1_us": sw("qwen3-30b-a3b", 1, "ms_per_step", 1e3),
        "w4a8_M2048_ms": sw("qwen3-235b-a22b-w4a8", 2048, "ms_per_step"),
        "w4a8_M256_frac_hbm": sw("qwen3-235b-a22b-w4a8", 256, "frac_hbm"),
    })

    t = head["ms_per_step"] * 1e-3
    line = {
        "metric": "block-INT8 fused-MoE tokens/s", "value": round(args.tokens / t, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": head["ms_per_step"],
        "ms_per_step_mean": head["ms_mean"], "ms_per_step_min": head["ms_min"],
        "scale_order": args.scale_order,
        **{f"ms_per_step_{'fused_scale' if n == 'fused' else n + '_order'}": round(v, 4) for n, v in others.items()},
        "host_us_per_call_M1": None if host_us is None else round(host_us, 1),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": f"{layer.name} E={L.E}/{L.E_global} top{L.top_k} H={L.H} I={L.I} "
                               + ("W4A8 int4[1,128]" if L.weight_bits == 4 else
                                  "per-channel INT8" if L.quant == "channel" else "block-INT8[128,128]")
                               + f", M={args.tokens}",
                   "tokens": args.tokens, "block_size_m": bs_used, "routing": L.routing,
                   "gemm1_kernel": tile1["kernel_name"], "gemm2_kernel": tile2["kernel_name"],
                   "cache_flush": f"512 MiB {args.flush} between steps, outside the timed region"},
        "int8_tops": head["int8_tops"], "hbm_gbs": head["hbm_gbs"], "frac_hbm": head["frac_hbm"],
        "frac_mfma": head["frac_mfma"], "stage_ms": {k: round(v, 4) for k, v in stages.items()},
        "roofline": roofline, "cpu_baseline": cpu, "routers": router_times(layer, args.tokens, dev, 50, 5),
        "graph_launch_floor": graph_launch_floor(args.steps, flush),
        "sweep": sweep,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
