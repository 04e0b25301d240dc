"""GPU parity with float32 activations (hidden_states.dtype == torch.float32: compute_type tl.float32,
int8.py:689-696), block form, through the C ABI, bit for bit against the oracle: the stage ops on fp32 rows
and the whole path with SiLU and GELU."""
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


def bits(t):
    return t.contiguous().view(torch.int32)


def test_stage_ops_on_float_rows(dev, oracle):
    from lightop_amd.moe import act_and_mul_group_quant, gelu_and_mul, moe_sum, silu_and_mul
    from lightop_amd.quant import per_token_group_quant_int8

    say("fp32 stage ops")
    g = torch.Generator().manual_seed(21)
    x = torch.randn(37, 1024, generator=g) * 3
    x[2] = 0
    x[5, :8] = torch.tensor([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5])
    rq, rs = oracle.per_token_group_quant_int8(x)
    q, s = per_token_group_quant_int8(x.to(dev), 128)
    torch.cuda.synchronize()
    assert torch.equal(q.cpu(), rq) and torch.equal(bits(s.cpu()), bits(rs))
    # gated activations: ordinary values, large and tiny gates, zeros of both signs
    c1 = torch.randn(130, 2 * 384, generator=g) * 4
    c1[0, :12] = torch.tensor([0.0, -0.0, 1e-30, -1e-30, 20.0, -20.0, 88.0, -88.0, 100.0, -100.0, 1e30, -1e30])
    c1[3] = 0
    for op, ref_fn, name in ((silu_and_mul, oracle.silu_and_mul, "silu"), (gelu_and_mul, oracle.gelu_and_mul, "gelu")):
        out = torch.empty(130, 384, dtype=torch.float32, device=dev)
        op(out, c1.to(dev))
        torch.cuda.synchronize()
        ref = ref_fn(c1)
        assert torch.equal(bits(out.cpu()), bits(ref)), name
        rq, rs = oracle.per_token_group_quant_int8(ref)
        mask = torch.rand(130, generator=g) > 0.3
        q = torch.full((130, 384), 77, dtype=torch.int8, device=dev)
        s = torch.full((130, 3), -5.0, dtype=torch.float32, device=dev)
        act_and_mul_group_quant(c1.to(dev), name, row_mask=mask.to(dev), out=(q, s))
        torch.cuda.synchronize()
        assert torch.equal(q.cpu()[mask], rq[mask]) and torch.equal(bits(s.cpu()[mask]), bits(rs[mask])), name
        assert (q.cpu()[~mask] == 77).all() and (s.cpu()[~mask] == -5.0).all()
    # top-k reduce: bias, factor, slot mask, padded batch
    c3 = torch.randn(9, 8, 512, generator=g)
    bias = torch.randn(9, 512, generator=g)
    for b, f in ((None, 1.0), (None, 2.5), (bias, 2.5)):
        out = torch.empty(9, 512, dtype=torch.float32, device=dev)
        moe_sum(c3.to(dev), out, None if b is None else b.to(dev), None, None, f)
        torch.cuda.synchronize()
        assert torch.equal(bits(out.cpu()), bits(oracle.moe_sum(c3, b, f)))
    smask = torch.rand(9, 8, generator=g) > 0.5
    ref = oracle.moe_sum(torch.where(smask[..., None], c3, torch.zeros_like(c3)), None, 2.5)
    out = torch.empty(9, 512, dtype=torch.float32, device=dev)
    moe_sum(torch.where(smask[..., None], c3, torch.full_like(c3, float("nan"))).to(dev), out,
            expert_mask=smask.reshape(-1).to(dev), factor=2.5)
    torch.cuda.synchronize()
    assert torch.equal(bits(out.cpu()), bits(ref))
    prev = torch.full((9, 512), 3.0)
    out = prev.clone().to(dev)
    moe_sum(c3.to(dev), out, num_local_tokens=torch.tensor([4], dtype=torch.int32, device=dev), factor=1.5)
    torch.cuda.synchronize()
    assert torch.equal(bits(out.cpu()), bits(oracle.moe_sum(c3, None, 1.5, num_local_tokens=4, out=prev)))


@pytest.mark.parametrize("bs", [16, 32, 64, 128])
@pytest.mark.parametrize("pre", [True, False])
def test_gemm_stage_float_output(dev, oracle, bs, pre):
    """The fp32 output is the sum itself: rounded to bf16 it is the bf16 stage's output."""
    import math

    from lightop_amd.moe import invoke_fused_moe_kernel_int8, moe_align_block_size, preshuffle_moe_weight

    say(f"fp32 gemm stage bs={bs} pre={pre}")
    g = torch.Generator().manual_seed(bs)
    M, k, E, Eg, N, K = 70, 2, 3, 6, 320, 384
    Aq = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8)
    W = torch.randint(-127, 128, (E, N, K), generator=g, dtype=torch.int8)
    As = torch.rand(M, K // 128, generator=g) * 0.05 + 0.005
    Ws = torch.exp(torch.randn(E, (N + 127) // 128, K // 128, generator=g) * 0.3 + math.log(1e-3))
    ids = torch.stack([torch.randperm(Eg, generator=g)[:k] for _ in range(M)]).to(torch.int32)
    tw = torch.rand(M, k, generator=g) + 0.1
    emap = torch.full((Eg,), -1, dtype=torch.int32)
    emap[:E] = torch.arange(E, dtype=torch.int32)
    rs, re, rp = oracle.moe_align_block_size(ids, bs, Eg, expert_map=emap)
    s, e, p = moe_align_block_size(ids.to(dev), bs, Eg, emap.to(dev))
    Wd = preshuffle_moe_weight(W.to(dev)) if pre else W.to(dev)
    for mul in (False, True):
        ref = oracle.moe_gemm_block_int8(Aq, As, W, Ws, rs, re, rp, tw, mul, k, M * k, bs,
                                         out=torch.zeros(M * k, N, dtype=torch.float32))
        ref16 = oracle.moe_gemm_block_int8(Aq, As, W, Ws, rs, re, rp, tw, mul, k, M * k, bs)
        assert torch.equal(ref.to(torch.bfloat16).view(torch.int16), ref16.view(torch.int16))
        C = torch.full((M, k, N), 9.0, dtype=torch.float32, device=dev)
        invoke_fused_moe_kernel_int8(Aq.to(dev), Wd, C, As.to(dev), Ws.to(dev), tw.to(dev), s, e, p, mul, k,
                                     {"BLOCK_SIZE_M": bs}, global_num_experts=Eg)
        torch.cuda.synchronize()
        assert torch.equal(bits(C.cpu().view(M * k, N)), bits(ref)), f"mul_routed={mul}"


def _run(layer, wd, x, tw, ids, emap, dev, bs, activation, **kw):
    from lightop_amd.moe import fused_experts_impl_int8

    w1, w2, w1s, w2s = wd
    M = x.shape[0]
    cache13 = torch.empty(M * layer.top_k * max(2 * layer.I, layer.H), dtype=torch.float32, device=dev)
    out = fused_experts_impl_int8(x, w1, w2, tw, ids, cache13, use_int8_w8a8=True, block_shape=[128, 128],
                                  global_num_experts=layer.E_global, expert_map=emap, w1_scale=w1s, w2_scale=w2s,
                                  activation=activation, lightop_amd_block_size_m=bs, **kw)
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("activation", ["silu", "gelu"])
@pytest.mark.parametrize("bs", [0, 16, 64, 128])
@pytest.mark.parametrize("pre", [True, False])
def test_whole_path_float32_bit_exact(dev, oracle, activation, bs, pre):
    from lightop_amd import workloads as wl
    from lightop_amd.moe import preshuffle_moe_weight

    layer = wl.TINY
    say(f"fp32 whole path {activation} bs={bs} pre={pre}")
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=0)
    M = 80
    x, tw, ids = wl.make_inputs(layer, M, seed=4)
    x = x.float() * 1.37
    prep = preshuffle_moe_weight if pre else (lambda t: t)
    wd = (prep(w1.to(dev)), prep(w2.to(dev)), w1s.to(dev), w2s.to(dev))
    shared = torch.randn(M, layer.H, generator=torch.Generator().manual_seed(9)) * 0.1
    for so, rsf in ((None, 1.0), (shared, 2.5)):
        out = _run(layer, wd, x.to(dev), tw.to(dev), ids.to(dev), None, dev, bs, activation,
                   shared_output=None if so is None else so.to(dev), routed_scaling_factor=rsf)
        assert out.dtype == torch.float32
        ref = oracle.fused_experts_block_int8(x, w1, w2, w1s, w2s, tw, ids, 16, global_num_experts=layer.E,
                                              shared_output=so, routed_scaling_factor=rsf, activation=activation)
        assert ref.abs().max() > 0.05
        assert torch.equal(bits(out.cpu()), bits(ref))


@pytest.mark.parametrize("M", [1, 3, 40])
@pytest.mark.parametrize("variant", ["plain", "on_input", "inplace"])
def test_float32_ep_share_variants_bit_exact(dev, oracle, M, variant):
    from lightop_amd import workloads as wl
    from lightop_amd.moe import preshuffle_moe_weight

    say(f"fp32 ep-share M={M} {variant}")
    layer = wl.MoeLayer("ep-fp32", E=4, E_global=32, top_k=8, H=512, I=256, routing="grouped_sigmoid", n_group=8,
                        topk_group=4, routed_scaling=2.5)
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=3)
    x, tw, ids = wl.make_inputs(layer, M, seed=3)
    x = x.float()
    emap = wl.expert_map_for(layer)
    wd = (preshuffle_moe_weight(w1.to(dev)), preshuffle_moe_weight(w2.to(dev)), w1s.to(dev), w2s.to(dev))
    xd = x.to(dev)
    out = _run(layer, wd, xd, tw.to(dev), ids.to(dev), emap.to(dev), dev, 0, "silu", inplace=variant == "inplace",
               apply_router_weight_on_input=variant == "on_input")
    if variant == "inplace":
        assert out.data_ptr() == xd.data_ptr()
    ref = oracle.fused_experts_block_int8(x, w1, w2, w1s, w2s, tw, ids, 16, global_num_experts=32, expert_map=emap,
                                          apply_router_weight_on_input=variant == "on_input")
    assert torch.equal(bits(out.cpu()), bits(ref))
