"""The two-launch decode path of the whole-path call (block_size_m = 0, weights in the load-time
layout, at most 512 routed slots): bit-exact against the CPU oracle and against the five-launch
path, for every variant of the call, with one, two, four and eight waves splitting K in its first
kernel, for experts that receive more slots than one pass holds, and on repeated calls."""
import sys

import pytest
import torch

pytestmark = pytest.mark.gpu


def say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from lightop_amd import _lib

    _lib.lib()
    return torch.device("cuda:0")


def run(dev, layer, M, seed, flags=None, shared=False, on_input=False, ids64=False, weights=None, repeat=1):
    from lightop_amd import workloads as wl
    from lightop_amd.moe import fused_experts_impl_int8, preshuffle_moe_weight

    from lightop_amd import _lib

    flags = _lib.LO_FUSED_FORCE_DECODE_PATH if flags is None else flags
    w1, w2, w1s, w2s = weights if weights is not None else wl.make_weights(layer, seed=seed)
    x, tw, ids = wl.make_inputs(layer, M, seed=seed)
    emap = wl.expert_map_for(layer)
    g = torch.Generator().manual_seed(seed + 5)
    sh = torch.randn(M, layer.H, generator=g).to(torch.bfloat16) if shared else None
    w1d, w2d = preshuffle_moe_weight(w1.to(dev)), preshuffle_moe_weight(w2.to(dev))
    outs = []
    for _ in range(repeat):
        cache13 = torch.full((M * layer.top_k * max(2 * layer.I, layer.H),), float("nan"), dtype=torch.bfloat16,
                             device=dev)
        out = fused_experts_impl_int8(
            x.to(dev), w1d, w2d, tw.to(dev), (ids.long() if ids64 else ids).to(dev), cache13,
            apply_router_weight_on_input=on_input, use_int8_w8a8=True, global_num_experts=layer.E_global,
            expert_map=None if emap is None else emap.to(dev), w1_scale=w1s.to(dev), w2_scale=w2s.to(dev),
            block_shape=[128, 128], routed_scaling_factor=2.5 if shared else layer.routed_scaling,
            shared_output=None if sh is None else sh.to(dev), lightop_amd_flags=flags)
        torch.cuda.synchronize()
        outs.append(out.cpu())
    return (x, w1, w2, w1s, w2s, tw, ids, emap, sh), outs


def oracle_out(oracle, layer, data, on_input=False, shared=False, order="contract"):
    x, w1, w2, w1s, w2s, tw, ids, emap, sh = data
    with oracle.scale_order(order):
        return oracle.fused_experts_block_int8(
            x, w1, w2, w1s, w2s, tw, ids, 16, global_num_experts=layer.E_global, expert_map=emap,
            apply_router_weight_on_input=on_input, routed_scaling_factor=2.5 if shared else layer.routed_scaling,
            shared_output=sh)


def layers():
    from lightop_amd import workloads as wl

    return {
        "tiny": wl.TINY,                                                       # K/128 = 8: split by 2 at most
        "ep": wl.MoeLayer("ep", E=4, E_global=32, top_k=8, H=512, I=256, routing="grouped_sigmoid",
                          n_group=8, topk_group=4, routed_scaling=2.5),        # most slots on other ranks
        "longk": wl.MoeLayer("longk", E=4, E_global=32, top_k=8, H=3584, I=256, routing="grouped_sigmoid",
                             n_group=8, topk_group=4, routed_scaling=2.5),     # K/128 = 28: split up to 7
        "longk2": wl.MoeLayer("longk2", E=3, E_global=3, top_k=2, H=7168, I=128, routing="softmax"),  # K/128 = 56
        "few": wl.MoeLayer("few", E=2, E_global=2, top_k=1, H=256, I=128, routing="softmax"),  # > 16 slots per expert
    }


@pytest.mark.parametrize("name", ["tiny", "ep", "longk", "longk2", "few"])
@pytest.mark.parametrize("M", [1, 3, 16, 64])
@pytest.mark.parametrize("order", ["contract", "separate"])
def test_decode_path_bit_exact(dev, oracle, name, M, order):
    """Both scale orders the checker restates: the default (acc = fma(f32(d) * a_s, b_s, acc)) and the one without
    fp fusion (LO_GEMM_SEPARATE_ORDER)."""
    from lightop_amd import _lib

    layer = layers()[name]
    say(f"decode path {name} M={M} order={order}")
    oflag = _lib.LO_GEMM_SEPARATE_ORDER if order == "separate" else 0
    data, outs = run(dev, layer, M, 7, repeat=3, flags=_lib.LO_FUSED_FORCE_DECODE_PATH | oflag)
    ref = oracle_out(oracle, layer, data, order=order)
    for i, out in enumerate(outs):  # repeated calls: the counters of the kernels are back at zero each time
        assert torch.equal(out.view(torch.int16), ref.view(torch.int16)), f"call {i}"
    _, (plain,) = run(dev, layer, M, 7, flags=_lib.LO_FUSED_NO_DECODE_PATH | oflag)
    assert torch.equal(plain.view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("variant", ["shared", "on_input", "ids64"])
@pytest.mark.parametrize("name,M", [("tiny", 5), ("ep", 40), ("longk", 2), ("few", 300)])
def test_decode_path_variants(dev, oracle, name, M, variant):
    layer = layers()[name]
    say(f"decode path {name} M={M} {variant}")
    kw = dict(shared=variant == "shared", on_input=variant == "on_input", ids64=variant == "ids64")
    data, outs = run(dev, layer, M, 11, repeat=2, **kw)
    ref = oracle_out(oracle, layer, data, on_input=kw["on_input"], shared=kw["shared"])
    for out in outs:
        assert torch.equal(out.view(torch.int16), ref.view(torch.int16))


def test_decode_path_activations(dev, oracle):
    """The bf16 activations the first kernel leaves at the front of cache13, against the oracle's."""
    from lightop_amd import _lib, workloads as wl
    from lightop_amd.moe import fused_experts_impl_int8, preshuffle_moe_weight

    for name, M in (("longk", 2), ("tiny", 33), ("ep", 9), ("few", 40)):
        layer = layers()[name]
        say(f"decode path activations {name} M={M}")
        w1, w2, w1s, w2s = wl.make_weights(layer, seed=2)
        x, tw, ids = wl.make_inputs(layer, M, seed=2)
        emap = wl.expert_map_for(layer)
        k, H, I, Eg = layer.top_k, layer.H, layer.I, layer.E_global
        cache13 = torch.empty(M * k * max(2 * I, H), dtype=torch.bfloat16, device=dev)
        out = fused_experts_impl_int8(
            x.to(dev), preshuffle_moe_weight(w1.to(dev)), preshuffle_moe_weight(w2.to(dev)), tw.to(dev), ids.to(dev),
            cache13, use_int8_w8a8=True, global_num_experts=Eg, expert_map=None if emap is None else emap.to(dev),
            w1_scale=w1s.to(dev), w2_scale=w2s.to(dev), block_shape=[128, 128], routed_scaling_factor=layer.routed_scaling,
            lightop_amd_flags=_lib.LO_FUSED_FORCE_DECODE_PATH)
        torch.cuda.synchronize()
        ref = oracle.fused_experts_block_int8(x, w1, w2, w1s, w2s, tw, ids, 16, global_num_experts=Eg, expert_map=emap,
                                              routed_scaling_factor=layer.routed_scaling, return_intermediates=True)
        flat = ids.reshape(-1).long()
        loc = torch.ones_like(flat, dtype=torch.bool) if emap is None else emap.long()[flat] >= 0
        assert torch.equal(out.cpu().view(torch.int16), ref["out"].view(torch.int16))
        act = cache13[: M * k * I].view(M * k, I).cpu()
        assert torch.equal(act[loc].view(torch.int16), ref["act"][loc].view(torch.int16))


def test_decode_path_is_the_default_for_one_token(dev, oracle):
    """Without any flag a single token takes the two-launch path (nothing else leaves activations at
    the front of cache13) and equals the oracle."""
    from lightop_amd import workloads as wl
    from lightop_amd.moe import fused_experts_impl_int8, preshuffle_moe_weight

    layer = wl.TINY
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=4)
    x, tw, ids = wl.make_inputs(layer, 1, seed=4)
    k, H, I = layer.top_k, layer.H, layer.I
    cache13 = torch.full((k * max(2 * I, H),), float("nan"), dtype=torch.bfloat16, device=dev)
    out = fused_experts_impl_int8(
        x.to(dev), preshuffle_moe_weight(w1.to(dev)), preshuffle_moe_weight(w2.to(dev)), tw.to(dev), ids.to(dev),
        cache13, use_int8_w8a8=True, w1_scale=w1s.to(dev), w2_scale=w2s.to(dev), block_shape=[128, 128])
    torch.cuda.synchronize()
    ref = oracle.fused_experts_block_int8(x, w1, w2, w1s, w2s, tw, ids, 16, return_intermediates=True)
    assert torch.equal(out.cpu().view(torch.int16), ref["out"].view(torch.int16))
    act = cache13[: k * I].view(k, I).cpu()
    assert torch.equal(act.view(torch.int16), ref["act"].view(torch.int16))
