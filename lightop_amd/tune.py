"""Tile-table tuning for the fused-MoE path (block-INT8, per-channel INT8, W4A8) on the GPU at hand.

    python -m lightop_amd.tune [--workload NAME | --shape E,E_global,topk,H,I] [--tokens 1,16,...]
                               [--out DIR] [--steps N]

For every token count the whole path is timed with each token-block size the kernels
offer (16, 32: weight-streaming; 64, 128: LDS-tiled), caches flushed between calls.  The
report shows the best size per token count next to what the compiled-in table
(``pick_block_m`` in csrc/api.hip, ``lo_moe_tile_query``) picks and how much slower that pick
is, so the table's thresholds (slots per expert at which the next larger block takes over) can be
re-derived after a kernel change.  With ``--out`` the winners are also written in the JSON
layout the reference keeps per device (reference: test/moe_w8a8/tune_int8.py writes, and
python/lightop/_lmslim_native/vllm_compat/w8a8_get_cache_json.py:12-174 reads,
``configs/w8a8/MOE_BLOCKINT8[128,128]_E=..._N1=..._N2=..._K=..._TOPK..._<device>.json`` with
one ``config1`` / ``config2`` pair per M).  ``TRITON_JSON_DIR=<that directory>`` then makes the
whole-path calls and ``get_w8a8moe_json`` take their block sizes from the file
(``lightop_amd/moe/tile_files.py``); the tuner itself always measures against the compiled-in table.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys

import torch

BLOCK_SIZES = (16, 32, 64, 128)


def time_ms(fn, steps, flush):
    for _ in range(2):
        flush()
        fn()
    torch.cuda.synchronize()
    ts = []
    for _ in range(steps):
        flush()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        torch.cuda.synchronize()
        ts.append(a.elapsed_time(b))
    return statistics.median(ts)


def main(argv=None):
    from lightop_amd import _lib, workloads as wl
    from lightop_amd.moe import tile_files
    from lightop_amd.moe import (fused_experts_impl_int8, fused_experts_impl_w4a8, get_w8a8moe_json,
                                 preshuffle_moe_scale_int4, preshuffle_moe_weight, preshuffle_moe_weight_int4)

    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--workload", default="deepseek-v3-ep8-share", help=f"one of {sorted(wl.LAYERS)}")
    ap.add_argument("--shape", default=None, help="E,E_global,topk,H,I (softmax routing) instead of --workload")
    ap.add_argument("--tokens", default="1,4,16,32,64,128,256,512,1024,2048,4096,8192")
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--out", default=None, help="directory for the JSON tile file")
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        print("lightop_amd.tune: needs a GPU", file=sys.stderr)
        return 1
    _lib.lib()
    os.environ.pop("TRITON_JSON_DIR", None)  # "table" below is the compiled-in one, whatever files exist
    tile_files.forget()
    dev = torch.device("cuda:0")
    if args.shape:
        E, Eg, k, H, I = (int(v) for v in args.shape.split(","))
        layer = wl.MoeLayer(f"custom-{args.shape}", E=E, E_global=Eg, top_k=k, H=H, I=I, routing="softmax")
    else:
        layer = wl.LAYERS[args.workload]
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=0, device=dev, gen_device="cuda")
    if layer.weight_bits == 4:
        w1, w2 = preshuffle_moe_weight_int4(w1), preshuffle_moe_weight_int4(w2)
        if layer.quant != "channel":  # K-group scales go K-group-major; per-channel scales stay [E, N, 1]
            w1s, w2s = preshuffle_moe_scale_int4(w1s), preshuffle_moe_scale_int4(w2s)
    else:
        w1, w2 = preshuffle_moe_weight(w1), preshuffle_moe_weight(w2)
    # which form of the path the layer asks for: block-INT8, per-channel INT8, W4A8 with K-group scales, or
    # W4A8 with per-token and per-channel scales
    if layer.quant == "channel":
        block_shape = None
    else:
        block_shape = [1, 128] if layer.weight_bits == 4 else [128, 128]

    def run(x, tw, ids, cache13, bs):
        if layer.weight_bits == 4:
            return fused_experts_impl_w4a8(x, w1, w2, tw, ids, cache13, global_num_experts=layer.E_global,
                                           expert_map=emap, w1_scale=w1s, w2_scale=w2s, block_shape=block_shape,
                                           lightop_amd_block_size_m=bs)
        return fused_experts_impl_int8(x, w1, w2, tw, ids, cache13, use_int8_w8a8=True,
                                       per_channel_quant=block_shape is None, global_num_experts=layer.E_global,
                                       expert_map=emap, w1_scale=w1s, w2_scale=w2s, block_shape=block_shape,
                                       lightop_amd_block_size_m=bs)

    emap = wl.expert_map_for(layer, dev)
    flush_buf = torch.empty(512 * 1024 * 1024 // 4, dtype=torch.int32, device=dev)
    counter = [0]

    def flush():
        counter[0] += 1
        flush_buf.fill_(counter[0])

    rows, table = [], {}
    print(f"{layer.name}: E={layer.E}/{layer.E_global} top{layer.top_k} H={layer.H} I={layer.I}")
    # 160-token blocks exist for the block form with int8 weights (bf16 rows with SiLU keep the fused first stage)
    # and for per-channel scales
    has160 = (layer.weight_bits == 8 and block_shape is not None) or block_shape is None
    sizes = BLOCK_SIZES + ((160,) if has160 else ())
    print(f"{'tokens':>7} {'slots/expert':>12} | " + " ".join(f"bs={b:<4}" for b in sizes) + " | best  table  loss")
    for M in (int(v) for v in args.tokens.split(",")):
        x, tw, ids = (t.to(dev) for t in wl.make_inputs(layer, M, seed=1))
        cache13 = torch.empty(M * layer.top_k * max(2 * layer.I, layer.H), dtype=torch.bfloat16, device=dev)
        ms = {}
        for bs in sizes:
            ms[bs] = time_ms(lambda: run(x, tw, ids, cache13, bs), args.steps, flush)
        best = min(ms, key=ms.get)
        c1, c2 = get_w8a8moe_json(M, layer.E, 2 * layer.I, layer.H, layer.I, True, block_shape, layer.top_k,
                                  layer.E_global, int4=layer.weight_bits == 4)
        pick = c1["BLOCK_SIZE_M"]
        # a few tokens: with the block size left to the library the call takes its two-launch path, which no
        # explicit block size reaches; it is timed as the table's pick
        two_launch = c1["kernel"] == _lib.LO_KERNEL_DEC
        ms_pick = time_ms(lambda: run(x, tw, ids, cache13, 0), args.steps, flush) if two_launch else ms[pick]
        loss = ms_pick / min(ms[best], ms_pick) - 1.0
        rows.append((M, best, pick, loss))
        print(f"{M:>7} {M * layer.top_k / layer.E_global:>12.1f} | " + " ".join(f"{ms[b]*1e3:7.1f}" for b in sizes)
              + f" | {best:>4}  {pick:>5}  {loss*100:4.1f}%   (us)"
              + (f"   two-launch path {ms_pick*1e3:.1f}" if two_launch else ""), flush=True)
        tile = dict(c1, BLOCK_SIZE_M=best), dict(c2, BLOCK_SIZE_M=best)
        if two_launch and ms_pick <= ms[best]:  # read back as "leave the block size to the library"
            tile = dict(c1, lightop_amd_two_launch=True), dict(c2, lightop_amd_two_launch=True)
        for t in tile:
            t.pop("source", None)
        table[str(M)] = {"config1": tile[0], "config2": tile[1]}
    worst = max(r[3] for r in rows)
    print(f"largest loss of the compiled-in table against the best block size: {worst*100:.1f}%")
    if args.out:
        os.makedirs(args.out, exist_ok=True)
        props = torch.cuda.get_device_properties(dev)
        devname = f"{props.gcnArchName.split(':')[0]}_{props.multi_processor_count}cu"
        # file names as the reference's reader builds them (w8a8_get_cache_json.py:133-149)
        if layer.weight_bits == 4:
            kind = "W4A8INT8" if block_shape is None else "W4A8INT8[1,128]"
        else:
            kind = "W8A8INT8" if block_shape is None else "BLOCKINT8[128,128]"
        name = (f"MOE_{kind}_E={layer.E}_N1={2 * layer.I}_N2={layer.H}_K={layer.I}_"
                f"TOPK{layer.top_k}_{devname}.json")
        with open(os.path.join(args.out, name), "w") as f:
            json.dump({f"{2 * layer.I}_{layer.H}_{layer.I}": table}, f, indent=4)
        print("wrote", os.path.join(args.out, name), "(read back when TRITON_JSON_DIR names that directory)")
        tile_files.forget()
    return 0


if __name__ == "__main__":
    sys.exit(main())
