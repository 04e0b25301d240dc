"""GPU parity of activation="gelu" (int8.py:825-838, w4a8.py:602-605), through the C ABI, bit for bit
against the oracle: the lookup table itself, gelu_and_mul, and the whole path in its four forms (block
scales, per-channel scales, int4 with K-group scales, int4 with per-channel scales)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from lightop_amd import _lib

    _lib.lib()
    return torch.device("cuda:0")


def say(msg):
    print(f"[case] {msg}", flush=True)


def test_gelu_table_equals_the_oracles(dev, oracle):
    from lightop_amd import _lib

    say("gelu table, all 65536 entries")
    tab = torch.empty(65536, dtype=torch.int16, device=dev)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().lo_activation_table(_lib.LO_ACT_GELU, _lib.LO_BF16, _lib.ptr(tab), _lib.stream_of(tab)))
    torch.cuda.synchronize()
    ref = oracle.gelu_bf16_table()
    got = tab.cpu()
    nan = ref.view(torch.bfloat16).isnan()
    assert torch.equal(got.view(torch.bfloat16).isnan(), nan)
    assert torch.equal(got[~nan], ref[~nan])


def test_gelu_and_mul_every_bf16(dev, oracle):
    from lightop_amd.moe import gelu_and_mul

    say("gelu_and_mul over all bf16 gates")
    gate = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).view(512, 128)
    finite = torch.isfinite(gate.float())
    gate = torch.where(finite, gate, torch.zeros_like(gate))
    g = torch.Generator().manual_seed(4)
    up = torch.randn(512, 128, generator=g).to(torch.bfloat16)
    c1 = torch.cat([gate, up], dim=1).contiguous()
    ref = oracle.gelu_and_mul(c1)
    out = torch.empty(512, 128, dtype=torch.bfloat16, device=dev)
    gelu_and_mul(out, c1.to(dev))
    torch.cuda.synchronize()
    assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))


def _weights_dev(layer, w1, w2, w1s, w2s, dev, preshuffle):
    from lightop_amd.moe import preshuffle_moe_weight, preshuffle_moe_weight_int4

    if layer.weight_bits == 4:
        return preshuffle_moe_weight_int4(w1.to(dev)), preshuffle_moe_weight_int4(w2.to(dev)), w1s.to(dev), w2s.to(dev)
    if preshuffle:
        return preshuffle_moe_weight(w1.to(dev)), preshuffle_moe_weight(w2.to(dev)), w1s.to(dev), w2s.to(dev)
    return w1.to(dev), w2.to(dev), w1s.to(dev), w2s.to(dev)


def _run(layer, wd, x, tw, ids, emap, dev, bs, activation, **kw):
    from lightop_amd.moe import fused_experts_impl_int8, fused_experts_impl_w4a8

    w1, w2, w1s, w2s = wd
    M = x.shape[0]
    cache13 = torch.empty(M * layer.top_k * max(2 * layer.I, layer.H), dtype=torch.bfloat16, device=dev)
    common = dict(global_num_experts=layer.E_global, expert_map=emap, w1_scale=w1s, w2_scale=w2s,
                  activation=activation, lightop_amd_block_size_m=bs, **kw)
    if layer.weight_bits == 4:
        out = fused_experts_impl_w4a8(x, w1, w2, tw, ids, cache13,
                                      block_shape=None if layer.quant == "channel" else [1, 128], **common)
    elif layer.quant == "channel":
        out = fused_experts_impl_int8(x, w1, w2, tw, ids, cache13, use_int8_w8a8=True, per_channel_quant=True,
                                      block_shape=None, **common)
    else:
        out = fused_experts_impl_int8(x, w1, w2, tw, ids, cache13, use_int8_w8a8=True, block_shape=[128, 128],
                                      **common)
    torch.cuda.synchronize()
    return out


def _oracle_fn(oracle, layer):
    if layer.weight_bits == 4:
        return oracle.fused_experts_w4a8_channel if layer.quant == "channel" else oracle.fused_experts_w4a8
    return oracle.fused_experts_channel_int8 if layer.quant == "channel" else oracle.fused_experts_block_int8


@pytest.mark.parametrize("form", ["TINY", "TINY_PC", "TINY_W4", "TINY_W4_PC"])
@pytest.mark.parametrize("bs", [0, 16, 64, 128])
@pytest.mark.parametrize("with_map", [False, True])
def test_whole_path_gelu_bit_exact(dev, oracle, form, bs, with_map):
    from lightop_amd import workloads as wl

    layer = getattr(wl, form)
    say(f"gelu whole path {form} bs={bs} map={with_map}")
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=0)
    M = 80
    x, tw, ids = wl.make_inputs(layer, M, seed=4)
    emap = None
    if with_map:
        emap = torch.full((layer.E,), -1, dtype=torch.int32)
        emap[:5] = torch.arange(5, dtype=torch.int32)
        w1, w2, w1s, w2s = (t[:5].contiguous() for t in (w1, w2, w1s, w2s))
    wd = _weights_dev(layer, w1, w2, w1s, w2s, dev, preshuffle=True)
    shared = (torch.randn(M, layer.H, generator=torch.Generator().manual_seed(9)) * 0.1).to(torch.bfloat16)
    for so, rsf in ((None, 1.0), (shared, 2.5)):
        out = _run(layer, wd, x.to(dev), tw.to(dev), ids.to(dev), None if emap is None else emap.to(dev), dev, bs,
                   "gelu", shared_output=None if so is None else so.to(dev), routed_scaling_factor=rsf)
        ref = _oracle_fn(oracle, layer)(x, w1, w2, w1s, w2s, tw, ids, 16, global_num_experts=layer.E,
                                        expert_map=emap, shared_output=so, routed_scaling_factor=rsf,
                                        activation="gelu")
        assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))
    # and it is not the SiLU result
    silu = _run(layer, wd, x.to(dev), tw.to(dev), ids.to(dev), None if emap is None else emap.to(dev), dev, bs, "silu")
    assert not torch.equal(silu.cpu(), _run(layer, wd, x.to(dev), tw.to(dev), ids.to(dev),
                                            None if emap is None else emap.to(dev), dev, bs, "gelu").cpu())


@pytest.mark.parametrize("M", [1, 3, 40])
@pytest.mark.parametrize("variant", ["plain", "on_input", "inplace", "row_major"])
def test_gelu_ep_share_variants_bit_exact(dev, oracle, M, variant):
    """Block form on an expert-parallel share; one token goes the long way too (no two-launch path for GELU)."""
    from lightop_amd import workloads as wl

    say(f"gelu ep-share M={M} {variant}")
    layer = wl.MoeLayer("ep-gelu", E=4, E_global=32, top_k=8, H=512, I=256, routing="grouped_sigmoid", n_group=8,
                        topk_group=4, routed_scaling=2.5)
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=3)
    x, tw, ids = wl.make_inputs(layer, M, seed=3)
    emap = wl.expert_map_for(layer)
    wd = _weights_dev(layer, w1, w2, w1s, w2s, dev, preshuffle=variant != "row_major")
    xd = x.to(dev)
    out = _run(layer, wd, xd, tw.to(dev), ids.to(dev), emap.to(dev), dev, 0, "gelu", inplace=variant == "inplace",
               apply_router_weight_on_input=variant == "on_input")
    if variant == "inplace":
        assert out.data_ptr() == xd.data_ptr()
    ref = oracle.fused_experts_block_int8(x, w1, w2, w1s, w2s, tw, ids, 16, global_num_experts=32, expert_map=emap,
                                          apply_router_weight_on_input=variant == "on_input", activation="gelu")
    assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))


def test_gelu_qwen3_layer_sampled_tokens(dev, oracle):
    """Qwen3-30B-A3B-shaped layer at 512 tokens with GELU, sampled tokens against the oracle."""
    from lightop_amd import workloads as wl

    layer = wl.QWEN3_30B
    say(f"gelu {layer.name} M=512")
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=0, device=dev, gen_device="cuda")
    from lightop_amd.moe import preshuffle_moe_weight

    wd = (preshuffle_moe_weight(w1), preshuffle_moe_weight(w2), w1s, w2s)
    M = 512
    x, tw, ids = (t.to(dev) for t in wl.make_inputs(layer, M, seed=3))
    tokens = torch.randperm(M, generator=torch.Generator().manual_seed(M))[:4].sort().values.to(dev)
    sub_ids = ids[tokens].cpu().long()
    used = torch.unique(sub_ids)
    remap = torch.full((layer.E,), -1, dtype=torch.int64)
    remap[used] = torch.arange(used.numel())
    sel = used.to(dev)
    ref = oracle.fused_experts_block_int8(x[tokens].cpu(), w1[sel].cpu(), w2[sel].cpu(), w1s[sel].cpu(), w2s[sel].cpu(),
                                          tw[tokens].cpu(), remap[sub_ids].to(torch.int32), 16, activation="gelu")
    out = _run(layer, wd, x, tw, ids, None, dev, 0, "gelu")
    assert torch.equal(out[tokens].cpu().view(torch.int16), ref.view(torch.int16))
