#!/usr/bin/env python3
"""Writes the golden fixtures of tests/golden/ from the CPU oracle (oracle/moe_oracle.c).

    python tests/golden/make_golden.py

Nothing from the reference tree is imported or executed: the fixtures are the oracle's
outputs on seeded synthetic inputs, kept so that (a) a later change of the oracle or of
the workload generator shows up as a diff and (b) the GPU box, which has no reference
tree, checks the HIP path against fixed bytes as well as against the live oracle.

  small_layer.npz    every input and every intermediate of one small fused-MoE call
                     (E=4 of 8 global, top-2, H=256, I=128, M=9, block 16, expert_map,
                     shared_output, routed_scaling_factor 2.5); ref_* in the default (contracted)
                     scale order, ref_sep_* the stages that differ in the separate order
  tiny_config1.json  the tiny benchmark configuration (E=8, top-2, H=1024, I=512, M=64, seed 0):
                     routing outputs in full, sha256 of every other stage's bytes in both scale
                     orders ("sha256": the default, acc = fma(f32(d) * a_s, b_s, acc);
                     "sha256_separate_order": acc = acc + (f32(d) * a_s) * b_s)
  tiny_forms.json    the same tiny layer in the per-channel W8A8 form and in the W4A8 form with
                     K-group scales (M=64, seed 0, block 16): sha256 of the inputs and of every stage
  align_docstring.json  the one literal known answer the reference holds
                     (moe_align_block_size.py:66-81)
"""
import hashlib
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from lightop_amd import workloads as wl  # noqa: E402
from oracle import cpu_oracle  # noqa: E402


def raw(t: torch.Tensor) -> np.ndarray:
    if t.dtype == torch.bfloat16:
        return t.contiguous().view(torch.int16).numpy()
    return t.contiguous().numpy()


def sha(t: torch.Tensor) -> str:
    return hashlib.sha256(raw(t).tobytes()).hexdigest()


STAGES_AFTER_GEMM1 = ("c1", "act", "a2q", "a2s", "c3", "out")  # what the scale order can change


def small_layer():
    layer = wl.MoeLayer("golden-small", E=4, E_global=8, top_k=2, H=256, I=128, routing="softmax")
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=11)
    x, tw, ids = wl.make_inputs(layer, 9, seed=11)
    emap = wl.expert_map_for(layer)
    g = torch.Generator().manual_seed(12)
    shared = torch.randn(9, layer.H, generator=g).to(torch.bfloat16)
    r = cpu_oracle.fused_experts_block_int8(x, w1, w2, w1s, w2s, tw, ids, 16, global_num_experts=8,
                                            expert_map=emap, routed_scaling_factor=2.5,
                                            shared_output=shared, return_intermediates=True)
    arrays = dict(x=raw(x), w1=raw(w1), w2=raw(w2), w1_scale=raw(w1s), w2_scale=raw(w2s),
                  topk_weights=raw(tw), topk_ids=raw(ids), expert_map=raw(emap), shared_output=raw(shared))
    arrays.update({"ref_" + k: raw(v) for k, v in r.items()})
    with cpu_oracle.scale_order("separate"):
        rs = cpu_oracle.fused_experts_block_int8(x, w1, w2, w1s, w2s, tw, ids, 16, global_num_experts=8,
                                                 expert_map=emap, routed_scaling_factor=2.5,
                                                 shared_output=shared, return_intermediates=True)
    arrays.update({"ref_sep_" + k: raw(rs[k]) for k in STAGES_AFTER_GEMM1})
    np.savez_compressed(os.path.join(HERE, "small_layer.npz"), **arrays)


def tiny_config1():
    layer = wl.TINY
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=0)
    x, tw, ids = wl.make_inputs(layer, 64, seed=0)
    r = cpu_oracle.fused_experts_block_int8(x, w1, w2, w1s, w2s, tw, ids, 16, return_intermediates=True)
    with cpu_oracle.scale_order("separate"):
        rs = cpu_oracle.fused_experts_block_int8(x, w1, w2, w1s, w2s, tw, ids, 16, return_intermediates=True)
    P = int(r["num_tokens_post_pad"].item())
    doc = {
        "config": "E=8 top-2 H=1024 I=512 M=64 seed 0 block_size_m=16",
        "inputs_sha256": {"x": sha(x), "w1": sha(w1), "w2": sha(w2), "w1_scale": sha(w1s), "w2_scale": sha(w2s),
                          "topk_weights": sha(tw), "topk_ids": sha(ids)},
        "topk_ids": ids.tolist(),
        "num_tokens_post_pad": P,
        "sorted_token_ids": r["sorted_ids"][:P].tolist(),
        "expert_ids": r["expert_ids"][: P // 16].tolist(),
        "sha256": {k: sha(r[k]) for k in ("a1q", "a1s", "c1", "act", "a2q", "a2s", "c3", "out")},
        "out_first_row_bf16_bits": raw(r["out"])[0, :16].tolist(),
        "out_abs_max": float(r["out"].float().abs().max()),
        "sha256_separate_order": {k: sha(rs[k]) for k in STAGES_AFTER_GEMM1},
        "out_first_row_bf16_bits_separate_order": raw(rs["out"])[0, :16].tolist(),
    }
    with open(os.path.join(HERE, "tiny_config1.json"), "w") as f:
        json.dump(doc, f, indent=1)


def tiny_forms():
    doc = {}
    for name, layer, fn in (("channel", wl.TINY_PC, cpu_oracle.fused_experts_channel_int8),
                            ("w4a8", wl.TINY_W4, cpu_oracle.fused_experts_w4a8)):
        w1, w2, w1s, w2s = wl.make_weights(layer, seed=0)
        x, tw, ids = wl.make_inputs(layer, 64, seed=0)
        r = fn(x, w1, w2, w1s, w2s, tw, ids, 16, return_intermediates=True)
        doc[name] = {
            "config": f"{layer.name}: E=8 top-2 H=1024 I=512 M=64 seed 0 block_size_m=16",
            "inputs_sha256": {"x": sha(x), "w1": sha(w1), "w2": sha(w2), "w1_scale": sha(w1s), "w2_scale": sha(w2s),
                              "topk_weights": sha(tw), "topk_ids": sha(ids)},
            "sha256": {k: sha(r[k]) for k in ("a1q", "a1s", "c1", "a2q", "a2s", "c3", "out")},
            "out_first_row_bf16_bits": raw(r["out"])[0, :16].tolist(),
        }
        if name == "w4a8":  # K-group scales: the scale order matters (the per-channel form scales once, at the end)
            with cpu_oracle.scale_order("separate"):
                rs = fn(x, w1, w2, w1s, w2s, tw, ids, 16, return_intermediates=True)
            doc[name]["sha256_separate_order"] = {k: sha(rs[k]) for k in ("c1", "a2q", "a2s", "c3", "out")}
    with open(os.path.join(HERE, "tiny_forms.json"), "w") as f:
        json.dump(doc, f, indent=1)


def align_docstring():
    doc = {"source": "python/lightop/_lmslim_native/vllm_compat/moe_align_block_size.py:66-81",
           "topk_ids": [[2, 3, 4], [1, 2, 4], [1, 3, 4], [1, 2, 3]], "block_size": 4, "num_experts": 5,
           "sorted_token_ids": [3, 6, 9, 12, 0, 4, 10, 12, 1, 7, 11, 12, 2, 5, 8, 12],
           "expert_ids": [1, 2, 3, 4], "num_tokens_post_pad": 16}
    with open(os.path.join(HERE, "align_docstring.json"), "w") as f:
        json.dump(doc, f, indent=1)


if __name__ == "__main__":
    small_layer()
    tiny_config1()
    tiny_forms()
    align_docstring()
    print("wrote", sorted(f for f in os.listdir(HERE) if not f.endswith(".py")))
