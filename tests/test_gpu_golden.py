"""The HIP path against the committed golden fixtures (tests/golden/), stage by stage."""
import hashlib
import json
import os
import sys

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from lightop_amd import _lib

    _lib.lib()
    return torch.device("cuda:0")


def bits(t):
    return t.contiguous().view(torch.int16) if t.dtype == torch.bfloat16 else t.contiguous()


def sha(t):
    return hashlib.sha256(bits(t.cpu()).numpy().tobytes()).hexdigest()


def test_small_layer_every_stage(dev):
    from lightop_amd import moe
    from lightop_amd.quant import per_token_group_quant_int8
    from test_host_logic import load_small_layer

    print("[case] golden small layer, staged", flush=True)
    g = {k: v.to(dev) for k, v in load_small_layer().items()}
    M, k, bs, Eg = 9, 2, 16, 8
    S = M * k
    a1q, a1s = per_token_group_quant_int8(g["x"], 128)
    assert torch.equal(a1q, g["ref_a1q"]) and torch.equal(a1s, g["ref_a1s"])
    s, e, p = moe.moe_align_block_size(g["topk_ids"], bs, Eg, g["expert_map"])
    assert torch.equal(s, g["ref_sorted_ids"]) and torch.equal(e, g["ref_expert_ids"])
    assert torch.equal(p, g["ref_num_tokens_post_pad"])
    c1 = torch.zeros(M, k, 256, dtype=torch.bfloat16, device=dev)
    moe.invoke_fused_moe_kernel_int8(a1q, g["w1"], c1, a1s, g["w1_scale"], g["topk_weights"], s, e, p, False, k,
                                     {"BLOCK_SIZE_M": bs}, fused_scale=False)
    assert torch.equal(bits(c1.view(S, -1)), bits(g["ref_c1"]))
    act = torch.empty(S, 128, dtype=torch.bfloat16, device=dev)
    moe.silu_and_mul(act, c1.view(S, -1))
    assert torch.equal(bits(act), bits(g["ref_act"]))
    local = g["expert_map"].long()[g["topk_ids"].reshape(-1).long()] >= 0
    a2q, a2s = moe.invoke_fused_moe_gemm1_silu_quant(a1q, g["w1"], a1s, g["w1_scale"], g["topk_weights"], s, e, p,
                                                     False, k, S, {"BLOCK_SIZE_M": bs}, fused_scale=False)
    assert torch.equal(a2q[local], g["ref_a2q"][local]) and torch.equal(a2s[local], g["ref_a2s"][local])
    c3 = torch.empty(M, k, 256, dtype=torch.bfloat16, device=dev)
    moe.invoke_fused_moe_kernel_int8(g["ref_a2q"], g["w2"], c3, g["ref_a2s"], g["w2_scale"], g["topk_weights"], s, e,
                                     p, True, 1, {"BLOCK_SIZE_M": bs}, fused_scale=False)
    assert torch.equal(bits(c3.view(S, -1)), bits(g["ref_c3"]))
    out = torch.empty(M, 256, dtype=torch.bfloat16, device=dev)
    moe.moe_sum(c3, out, bias=g["shared_output"], factor=2.5)
    assert torch.equal(bits(out), bits(g["ref_out"]))


@pytest.mark.parametrize("preshuffle", [False, True])
def test_small_layer_whole_path(dev, preshuffle):
    from lightop_amd import moe
    from test_host_logic import load_small_layer

    print(f"[case] golden small layer, fused entry, preshuffle={preshuffle}", flush=True)
    g = {k: v.to(dev) for k, v in load_small_layer().items()}
    w1, w2 = g["w1"], g["w2"]
    if preshuffle:
        w1, w2 = moe.preshuffle_moe_weight(w1), moe.preshuffle_moe_weight(w2)
    cache13 = torch.empty(9 * 2 * 256, dtype=torch.bfloat16, device=dev)
    out = moe.fused_experts_impl_int8(g["x"], w1, w2, g["topk_weights"], g["topk_ids"], cache13, use_int8_w8a8=True,
                                      global_num_experts=8, expert_map=g["expert_map"], w1_scale=g["w1_scale"],
                                      w2_scale=g["w2_scale"], block_shape=[128, 128], routed_scaling_factor=2.5,
                                      shared_output=g["shared_output"], lightop_amd_block_size_m=16)
    torch.cuda.synchronize()
    assert torch.equal(bits(out), bits(g["ref_out"]))


def test_tiny_config1_digests(dev):
    """The tiny benchmark configuration end to end: routing outputs in full, every other stage by digest."""
    from lightop_amd import moe, workloads as wl
    from lightop_amd.quant import per_token_group_quant_int8

    print("[case] golden tiny config 1", flush=True)
    doc = json.load(open(os.path.join(GOLDEN, "tiny_config1.json")))
    w1, w2, w1s, w2s = (t.to(dev) for t in wl.make_weights(wl.TINY, seed=0))
    x, tw, ids = (t.to(dev) for t in wl.make_inputs(wl.TINY, 64, seed=0))
    for name, t in (("x", x), ("w1", w1), ("w2", w2), ("w1_scale", w1s), ("w2_scale", w2s), ("topk_weights", tw),
                    ("topk_ids", ids)):
        assert sha(t) == doc["inputs_sha256"][name], f"this host's workload generator does not reproduce {name}"
    a1q, a1s = per_token_group_quant_int8(x, 128)
    assert sha(a1q) == doc["sha256"]["a1q"] and sha(a1s) == doc["sha256"]["a1s"]
    s, e, p = moe.moe_align_block_size(ids, 16, 8)
    P = doc["num_tokens_post_pad"]
    assert p.item() == P and s[:P].tolist() == doc["sorted_token_ids"] and e[: P // 16].tolist() == doc["expert_ids"]
    a2q, a2s = moe.invoke_fused_moe_gemm1_silu_quant(a1q, w1, a1s, w1s, tw, s, e, p, False, 2, 128,
                                                     {"BLOCK_SIZE_M": 16}, fused_scale=False)
    assert sha(a2q) == doc["sha256"]["a2q"] and sha(a2s) == doc["sha256"]["a2s"]
    cache13 = torch.empty(64 * 2 * 1024, dtype=torch.bfloat16, device=dev)
    out = moe.fused_experts_impl_int8(x, w1, w2, tw, ids, cache13, use_int8_w8a8=True, w1_scale=w1s, w2_scale=w2s,
                                      block_shape=[128, 128], lightop_amd_block_size_m=16)
    torch.cuda.synchronize()
    assert sha(cache13[: 128 * 1024].view(128, 1024)) == doc["sha256"]["c3"]
    assert sha(out) == doc["sha256"]["out"]
    assert bits(out.cpu())[0, :16].tolist() == doc["out_first_row_bf16_bits"]
    # the order without fp fusion (its c1, act and c3 differ from the default's on this input)
    from lightop_amd import _lib

    sep = doc["sha256_separate_order"]
    c1 = torch.zeros(64, 2, 1024, dtype=torch.bfloat16, device=dev)
    moe.invoke_fused_moe_kernel_int8(a1q, w1, c1, a1s, w1s, tw, s, e, p, False, 2, {"BLOCK_SIZE_M": 16},
                                     flags=_lib.LO_GEMM_SEPARATE_ORDER)
    assert sha(c1) == sep["c1"] and sep["c1"] != doc["sha256"]["c1"]
    out = moe.fused_experts_impl_int8(x, w1, w2, tw, ids, cache13, use_int8_w8a8=True, w1_scale=w1s, w2_scale=w2s,
                                      block_shape=[128, 128], lightop_amd_block_size_m=16,
                                      lightop_amd_flags=_lib.LO_GEMM_SEPARATE_ORDER)
    torch.cuda.synchronize()
    assert sha(cache13[: 128 * 1024].view(128, 1024)) == sep["c3"] and sep["c3"] != doc["sha256"]["c3"]
    assert sha(out) == sep["out"]
    assert bits(out.cpu())[0, :16].tolist() == doc["out_first_row_bf16_bits_separate_order"]


@pytest.mark.parametrize("form", ["channel", "w4a8"])
def test_tiny_forms_digests(dev, form):
    """The tiny layer in the per-channel and W4A8 forms: whole path and second GEMM's output by digest."""
    from lightop_amd import _lib, moe, workloads as wl

    print(f"[case] golden tiny layer, {form}", flush=True)
    doc = json.load(open(os.path.join(GOLDEN, "tiny_forms.json")))[form]
    layer = {"channel": wl.TINY_PC, "w4a8": wl.TINY_W4}[form]
    w1, w2, w1s, w2s = (t.to(dev) for t in wl.make_weights(layer, seed=0))
    x, tw, ids = (t.to(dev) for t in wl.make_inputs(layer, 64, seed=0))
    for name, t in (("x", x), ("w1", w1), ("w2", w2), ("w1_scale", w1s), ("w2_scale", w2s), ("topk_weights", tw),
                    ("topk_ids", ids)):
        assert sha(t) == doc["inputs_sha256"][name], f"this host's workload generator does not reproduce {name}"
    cache13 = torch.empty(64 * 2 * 1024, dtype=torch.bfloat16, device=dev)
    if form == "channel":
        out = moe.fused_experts_impl_int8(x, w1, w2, tw, ids, cache13, use_int8_w8a8=True, per_channel_quant=True,
                                          w1_scale=w1s, w2_scale=w2s, block_shape=None, lightop_amd_block_size_m=16)
    else:
        out = moe.fused_experts_impl_w4a8(x, moe.preshuffle_moe_weight_int4(w1), moe.preshuffle_moe_weight_int4(w2), tw,
                                          ids, cache13, w1_scale=w1s, w2_scale=w2s, block_shape=[1, 128],
                                          lightop_amd_block_size_m=16, lightop_amd_flags=0)
    torch.cuda.synchronize()
    assert sha(cache13[: 128 * 1024].view(128, 1024)) == doc["sha256"]["c3"]
    assert sha(out) == doc["sha256"]["out"]
    assert bits(out.cpu())[0, :16].tolist() == doc["out_first_row_bf16_bits"]
    if form == "w4a8":  # K-group scales: the order without fp fusion has digests of its own
        out = moe.fused_experts_impl_w4a8(x, moe.preshuffle_moe_weight_int4(w1), moe.preshuffle_moe_weight_int4(w2), tw,
                                          ids, cache13, w1_scale=w1s, w2_scale=w2s, block_shape=[1, 128],
                                          lightop_amd_block_size_m=16, lightop_amd_flags=_lib.LO_GEMM_SEPARATE_ORDER)
        torch.cuda.synchronize()
        assert sha(cache13[: 128 * 1024].view(128, 1024)) == doc["sha256_separate_order"]["c3"]
        assert sha(out) == doc["sha256_separate_order"]["out"]
