"""GPU parity with float16 activations (hidden_states.dtype == torch.float16, int8.py:689-696), through the
C ABI, bit for bit against the oracle: the stage ops on half rows, the activation tables, and the whole
path in its four forms with SiLU and GELU."""
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


@pytest.mark.parametrize("activation", ["silu", "gelu"])
def test_half_activation_tables_equal_the_oracles(dev, oracle, activation):
    from lightop_amd import _lib

    say(f"fp16 {activation} table")
    tab = torch.empty(65536, dtype=torch.int16, device=dev)
    act = _lib.LO_ACT_GELU if activation == "gelu" else _lib.LO_ACT_SILU
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().lo_activation_table(act, _lib.LO_F16, _lib.ptr(tab), _lib.stream_of(tab)))
    torch.cuda.synchronize()
    ref = oracle.activation_table(activation, torch.float16)
    got = tab.cpu()
    nan = ref.view(torch.float16).isnan()
    assert torch.equal(got.view(torch.float16).isnan(), nan)
    assert torch.equal(got[~nan], ref[~nan])


def test_stage_ops_on_half_rows(dev, oracle):
    from lightop_amd import fuse_silu_mul_quant
    from lightop_amd.moe import gelu_and_mul, moe_sum, silu_and_mul
    from lightop_amd.quant import per_token_group_quant_int8, per_token_quant_int8

    say("fp16 stage ops")
    g = torch.Generator().manual_seed(11)
    x = (torch.randn(37, 1024, generator=g) * 3).to(torch.float16)
    x[2] = 0
    x[5, :8] = torch.tensor([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5]).to(torch.float16)
    # 1x128 group quant and per-token quant
    rq, rs = oracle.per_token_group_quant_int8(x)
    q, s = per_token_group_quant_int8(x.to(dev), 128)
    torch.cuda.synchronize()
    assert torch.equal(q.cpu(), rq) and torch.equal(s.cpu(), rs)
    rq, rs = oracle.per_token_quant_int8(x)
    q, s = per_token_quant_int8(x.to(dev))
    torch.cuda.synchronize()
    assert torch.equal(q.cpu(), rq) and torch.equal(s.cpu(), rs)
    # gated activations over every finite half gate
    gate = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.float16).view(512, 128)
    gate = torch.where(gate.float().isfinite(), gate, torch.zeros_like(gate))
    up = torch.randn(512, 128, generator=g).to(torch.float16)
    c1 = torch.cat([gate, up], dim=1).contiguous()
    for op, ref_fn in ((silu_and_mul, oracle.silu_and_mul), (gelu_and_mul, oracle.gelu_and_mul)):
        out = torch.empty(512, 128, dtype=torch.float16, device=dev)
        op(out, c1.to(dev))
        torch.cuda.synchronize()
        ref = ref_fn(c1)
        nan = ref.isnan()
        assert torch.equal(out.cpu().isnan(), nan)
        assert torch.equal(out.cpu().view(torch.int16)[~nan], ref.view(torch.int16)[~nan])
    # SiLU-and-mul with per-token quant (no floor under the row maximum)
    c1 = (torch.randn(33, 2 * 768, generator=g) * 3).to(torch.float16)
    c1[3] = 0
    rq, rs = oracle.fuse_silu_mul_quant(c1)
    q, s = fuse_silu_mul_quant(c1.to(dev))
    torch.cuda.synchronize()
    assert torch.equal(q.cpu(), rq) and torch.equal(s.cpu().view(torch.int32), rs.view(torch.int32))
    # top-k reduce, with and without bias
    c3 = torch.randn(9, 8, 512, generator=g).to(torch.float16)
    bias = torch.randn(9, 512, generator=g).to(torch.float16)
    for b, f in ((None, 1.0), (bias, 2.5)):
        out = torch.empty(9, 512, dtype=torch.float16, device=dev)
        moe_sum(c3.to(dev), out, None if b is None else b.to(dev), None, None, f)
        torch.cuda.synchronize()
        assert torch.equal(out.cpu().view(torch.int16), oracle.moe_sum(c3, b, f).view(torch.int16))


def _weights_dev(layer, w1, w2, w1s, w2s, dev, preshuffle=True):
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
    cache13 = torch.empty(M * layer.top_k * max(2 * layer.I, layer.H), dtype=x.dtype, device=dev)
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
@pytest.mark.parametrize("activation", ["silu", "gelu"])
@pytest.mark.parametrize("bs", [0, 16, 64, 128])
def test_whole_path_float16_bit_exact(dev, oracle, form, activation, bs):
    from lightop_amd import workloads as wl

    layer = getattr(wl, form)
    say(f"fp16 whole path {form} {activation} bs={bs}")
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=0)
    M = 80
    x, tw, ids = wl.make_inputs(layer, M, seed=4)
    x = x.to(torch.float16)
    wd = _weights_dev(layer, w1, w2, w1s, w2s, dev)
    shared = (torch.randn(M, layer.H, generator=torch.Generator().manual_seed(9)) * 0.1).to(torch.float16)
    for so, rsf in ((None, 1.0), (shared, 2.5)):
        out = _run(layer, wd, x.to(dev), tw.to(dev), ids.to(dev), None, dev, bs, activation,
                   shared_output=None if so is None else so.to(dev), routed_scaling_factor=rsf)
        assert out.dtype == torch.float16
        ref = _oracle_fn(oracle, layer)(x, w1, w2, w1s, w2s, tw, ids, 16, global_num_experts=layer.E,
                                        shared_output=so, routed_scaling_factor=rsf, activation=activation)
        assert ref.float().abs().max() > 0.05
        assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("M", [1, 3, 40])
@pytest.mark.parametrize("variant", ["plain", "on_input", "inplace", "row_major"])
def test_float16_ep_share_variants_bit_exact(dev, oracle, M, variant):
    """Block form on an expert-parallel share; one token goes the five-stage way (no two-launch path for half)."""
    from lightop_amd import workloads as wl

    say(f"fp16 ep-share M={M} {variant}")
    layer = wl.MoeLayer("ep-fp16", E=4, E_global=32, top_k=8, H=512, I=256, routing="grouped_sigmoid", n_group=8,
                        topk_group=4, routed_scaling=2.5)
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=3)
    x, tw, ids = wl.make_inputs(layer, M, seed=3)
    x = x.to(torch.float16)
    emap = wl.expert_map_for(layer)
    wd = _weights_dev(layer, w1, w2, w1s, w2s, dev, preshuffle=variant != "row_major")
    xd = x.to(dev)
    out = _run(layer, wd, xd, tw.to(dev), ids.to(dev), emap.to(dev), dev, 0, "silu", inplace=variant == "inplace",
               apply_router_weight_on_input=variant == "on_input")
    if variant == "inplace":
        assert out.data_ptr() == xd.data_ptr()
    ref = oracle.fused_experts_block_int8(x, w1, w2, w1s, w2s, tw, ids, 16, global_num_experts=32, expert_map=emap,
                                          apply_router_weight_on_input=variant == "on_input")
    assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))


def test_float16_qwen3_layer_sampled_tokens(dev, oracle):
    """Qwen3-30B-A3B-shaped layer at 2048 tokens in half precision, sampled tokens against the oracle."""
    from lightop_amd import workloads as wl
    from lightop_amd.moe import preshuffle_moe_weight

    layer = wl.QWEN3_30B
    say(f"fp16 {layer.name} M=2048")
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=0, device=dev, gen_device="cuda")
    wd = (preshuffle_moe_weight(w1), preshuffle_moe_weight(w2), w1s, w2s)
    M = 2048
    x, tw, ids = (t.to(dev) for t in wl.make_inputs(layer, M, seed=3))
    x = x.to(torch.float16)
    tokens = torch.randperm(M, generator=torch.Generator().manual_seed(M))[:4].sort().values.to(dev)
    sub_ids = ids[tokens].cpu().long()
    used = torch.unique(sub_ids)
    remap = torch.full((layer.E,), -1, dtype=torch.int64)
    remap[used] = torch.arange(used.numel())
    sel = used.to(dev)
    ref = oracle.fused_experts_block_int8(x[tokens].cpu(), w1[sel].cpu(), w2[sel].cpu(), w1s[sel].cpu(), w2s[sel].cpu(),
                                          tw[tokens].cpu(), remap[sub_ids].to(torch.int32), 16)
    out = _run(layer, wd, x, tw, ids, None, dev, 0, "silu")
    assert torch.equal(out[tokens].cpu().view(torch.int16), ref.view(torch.int16))


def test_float32_rows_with_per_channel_scales_raise(dev):
    from lightop_amd import workloads as wl
    from lightop_amd.moe import fused_experts_impl_int8

    layer = wl.TINY_PC
    w1, w2, w1s, w2s = (t.to(dev) for t in wl.make_weights(layer, seed=0))
    x, tw, ids = (t.to(dev) for t in wl.make_inputs(layer, 4, seed=0))
    cache13 = torch.empty(4 * 2 * 1024, dtype=torch.float32, device=dev)
    with pytest.raises(NotImplementedError):
        fused_experts_impl_int8(x.float(), w1, w2, tw, ids, cache13, use_int8_w8a8=True, per_channel_quant=True,
                                w1_scale=w1s, w2_scale=w2s, block_shape=None)
