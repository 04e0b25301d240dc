"""GPU parity of the W4A8 (packed int4 weights, K-group scales) path, through the C ABI, bit for
bit against the oracle in both bit-exact scale orders; the benchmark's int4 configuration (Qwen3-235B-A22B-shaped
layer, M in {1, 32, 256, 2048}) on sampled tokens."""
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


def gemm_case(seed, M, k, E, Eg, N, K):
    g = torch.Generator().manual_seed(seed)
    Aq = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8)
    As = torch.rand(M, K // 128, generator=g) * 0.05 + 0.005
    W4 = torch.randint(0, 256, (E, N, K // 2), generator=g, dtype=torch.int16).to(torch.uint8)
    Ws = torch.exp(torch.randn(E, N, K // 128, generator=g) * 0.3 - 4.6)
    ids = torch.stack([torch.randperm(Eg, generator=g)[:k] for _ in range(M)]).to(torch.int32)
    tw = torch.rand(M, k, generator=g) + 0.1
    emap = None
    if Eg != E:
        emap = torch.full((Eg,), -1, dtype=torch.int32)
        emap[:E] = torch.arange(E, dtype=torch.int32)
    return Aq, As, W4, Ws, ids, tw, emap


@pytest.mark.parametrize("M,k,E,Eg,N,K", [(1, 2, 4, 4, 64, 128), (5, 2, 4, 4, 256, 512), (40, 4, 8, 8, 320, 1024),
                                          (100, 8, 4, 16, 512, 768), (300, 2, 3, 3, 128, 2048)])
@pytest.mark.parametrize("bs", [16, 32, 64, 128])
@pytest.mark.parametrize("order", ["contract", "separate"])
def test_gemm_w4a8_bit_exact(dev, oracle, M, k, E, Eg, N, K, bs, order):
    from lightop_amd import _lib
    from lightop_amd.moe import (invoke_fused_moe_kernel_int8, moe_align_block_size, preshuffle_moe_scale_int4,
                                 preshuffle_moe_weight_int4)

    say(f"w4a8 gemm M={M} k={k} E={E}/{Eg} N={N} K={K} bs={bs} order={order}")
    oflag = _lib.LO_GEMM_SEPARATE_ORDER if order == "separate" else 0
    Aq, As, W4, Ws, ids, tw, emap = gemm_case(M + N + bs, M, k, E, Eg, N, K)
    rs, re, rp = oracle.moe_align_block_size(ids, bs, Eg, expert_map=emap)
    s, e, p = moe_align_block_size(ids.to(dev), bs, Eg, None if emap is None else emap.to(dev))
    Wd = preshuffle_moe_weight_int4(W4.to(dev))
    for mul in (False, True):
        with oracle.scale_order(order):
            ref = oracle.moe_gemm_w4a8(Aq, As, W4, Ws, rs, re, rp, tw, mul, k, M * k, bs)
        C = torch.empty((M, k, N), dtype=torch.bfloat16, device=dev)
        invoke_fused_moe_kernel_int8(Aq.to(dev), Wd, C, As.to(dev), preshuffle_moe_scale_int4(Ws.to(dev)), tw.to(dev), s, e, p, mul, k,
                                     {"BLOCK_SIZE_M": bs}, flags=_lib.LO_GEMM_W4 | oflag)
        torch.cuda.synchronize()
        assert torch.equal(C.cpu().view(M * k, N).view(torch.int16), ref.view(torch.int16)), f"mul_routed={mul}"


@pytest.mark.parametrize("M,k,E,Eg,I,K", [(1, 2, 4, 4, 128, 256), (9, 2, 4, 4, 256, 512), (50, 8, 4, 16, 256, 768),
                                          (200, 4, 6, 6, 384, 1024)])
@pytest.mark.parametrize("bs", [16, 32, 64, 128])
def test_gemm1_silu_quant_w4a8_bit_exact(dev, oracle, M, k, E, Eg, I, K, bs):
    from lightop_amd import _lib
    from lightop_amd.moe import (invoke_fused_moe_gemm1_silu_quant, moe_align_block_size, preshuffle_moe_scale_int4,
                                 preshuffle_moe_weight_int4)

    say(f"w4a8 gemm1+silu+quant M={M} k={k} E={E}/{Eg} I={I} K={K} bs={bs}")
    Aq, As, W4, Ws, ids, tw, emap = gemm_case(M + I + bs + 1, M, k, E, Eg, 2 * I, K)
    Ws = Ws * 30  # bring the gate into the range where SiLU is neither 0 nor identity
    rs, re, rp = oracle.moe_align_block_size(ids, bs, Eg, expert_map=emap)
    S = M * k
    s, e, p = moe_align_block_size(ids.to(dev), bs, Eg, None if emap is None else emap.to(dev))
    Wd = preshuffle_moe_weight_int4(W4.to(dev))
    for mul in (False, True):
        c1 = oracle.moe_gemm_w4a8(Aq, As, W4, Ws, rs, re, rp, tw, mul, k, S, bs)
        rq, rsc = oracle.per_token_group_quant_int8(oracle.silu_and_mul(c1))
        q, sc = invoke_fused_moe_gemm1_silu_quant(Aq.to(dev), Wd, As.to(dev), preshuffle_moe_scale_int4(Ws.to(dev)), tw.to(dev), s, e, p, mul, k,
                                                  S, {"BLOCK_SIZE_M": bs}, fused_scale=False, flags=_lib.LO_GEMM_W4)
        torch.cuda.synchronize()
        local = torch.ones(S, dtype=torch.bool) if emap is None else emap.long()[ids.reshape(-1).long()] >= 0
        assert torch.equal(sc.cpu()[local], rsc[local]) and torch.equal(q.cpu()[local], rq[local]), f"mul={mul}"


def run_path(layer, weights_dev, x, tw, ids, emap, dev, bs, flags):
    from lightop_amd.moe import fused_experts_impl_w4a8

    w1, w2, w1s, w2s = weights_dev
    M = x.shape[0]
    cache13 = torch.empty(M * layer.top_k * max(2 * layer.I, layer.H), dtype=torch.bfloat16, device=dev)
    out = fused_experts_impl_w4a8(x, w1, w2, tw, ids, cache13, global_num_experts=layer.E_global, expert_map=emap,
                                  w1_scale=w1s, w2_scale=w2s, block_shape=[1, 128], lightop_amd_block_size_m=bs,
                                  lightop_amd_flags=flags)
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("bs", [0, 16, 64])
@pytest.mark.parametrize("with_map", [False, True])
def test_whole_path_tiny_bit_exact(dev, oracle, bs, with_map):
    from lightop_amd import _lib, workloads as wl
    from lightop_amd.moe import preshuffle_moe_weight_int4

    layer = wl.TINY_W4
    say(f"w4a8 whole path tiny bs={bs} map={with_map}")
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=0)
    x, tw, ids = wl.make_inputs(layer, 64, seed=4)
    emap = None
    if with_map:
        emap = torch.full((layer.E,), -1, dtype=torch.int32)
        emap[:5] = torch.arange(5, dtype=torch.int32)
    wd = (preshuffle_moe_weight_int4(w1.to(dev)), preshuffle_moe_weight_int4(w2.to(dev)), w1s.to(dev), w2s.to(dev))
    if with_map:  # the weight tensors hold the local experts only
        wd = (preshuffle_moe_weight_int4(w1[:5].contiguous().to(dev)),
              preshuffle_moe_weight_int4(w2[:5].contiguous().to(dev)), w1s[:5].contiguous().to(dev),
              w2s[:5].contiguous().to(dev))
    out = run_path(layer, wd, x.to(dev), tw.to(dev), ids.to(dev), None if emap is None else emap.to(dev), dev, bs,
                   0)
    ref = oracle.fused_experts_w4a8(x, w1[:5] if with_map else w1, w2[:5] if with_map else w2,
                                    w1s[:5] if with_map else w1s, w2s[:5] if with_map else w2s, tw, ids, 16,
                                    global_num_experts=layer.E, expert_map=emap)
    assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("bs", [16, 32, 64, 128])
def test_whole_path_long_k_bit_exact(dev, oracle, bs):
    """K = 4608 and 5120: more than 32 K groups, so the copy of the row scales into LDS takes a second pass
    (streaming kernel and 64-token kernel), and both K-block parities end the loop."""
    from lightop_amd import _lib, workloads as wl
    from lightop_amd.moe import preshuffle_moe_weight_int4

    for H, I in ((4608, 256), (256, 5120), (7168, 128)):  # 7168: more than 48 KB of scales in LDS
        layer = wl.MoeLayer("w4-long-k", E=2, E_global=2, top_k=2, H=H, I=I, routing="softmax", weight_bits=4)
        say(f"w4a8 whole path H={H} I={I} bs={bs}")
        w1, w2, w1s, w2s = wl.make_weights(layer, seed=H)
        x, tw, ids = wl.make_inputs(layer, 40, seed=H)
        wd = (preshuffle_moe_weight_int4(w1.to(dev)), preshuffle_moe_weight_int4(w2.to(dev)), w1s.to(dev), w2s.to(dev))
        out = run_path(layer, wd, x.to(dev), tw.to(dev), ids.to(dev), None, dev, bs,
                       _lib.LO_FUSED_NO_DECODE_PATH)
        ref = oracle.fused_experts_w4a8(x, w1, w2, w1s, w2s, tw, ids, 16, global_num_experts=layer.E)
        assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("M", [1, 5, 40, 200])
@pytest.mark.parametrize("with_map", [False, True])
@pytest.mark.parametrize("order", ["contract", "separate"])
def test_two_launch_path_w4a8_bit_exact(dev, oracle, M, with_map, order):
    """The two-launch path for a few tokens on packed int4 weights (forced beyond its default size)."""
    from lightop_amd import _lib, workloads as wl
    from lightop_amd.moe import preshuffle_moe_weight_int4

    layer = wl.TINY_W4
    say(f"w4a8 two-launch path M={M} map={with_map}")
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=1)
    x, tw, ids = wl.make_inputs(layer, M, seed=M)
    emap, n = None, layer.E
    if with_map:
        n = 5
        emap = torch.full((layer.E,), -1, dtype=torch.int32)
        emap[:n] = torch.arange(n, dtype=torch.int32)
    wd = (preshuffle_moe_weight_int4(w1[:n].contiguous().to(dev)), preshuffle_moe_weight_int4(w2[:n].contiguous().to(dev)),
          w1s[:n].contiguous().to(dev), w2s[:n].contiguous().to(dev))
    with oracle.scale_order(order):
        ref = oracle.fused_experts_w4a8(x, w1[:n], w2[:n], w1s[:n], w2s[:n], tw, ids, 16, global_num_experts=layer.E,
                                        expert_map=emap)
    oflag = _lib.LO_GEMM_SEPARATE_ORDER if order == "separate" else 0
    for _ in range(2):
        out = run_path(layer, wd, x.to(dev), tw.to(dev), ids.to(dev), None if emap is None else emap.to(dev), dev, 0,
                       _lib.LO_FUSED_FORCE_DECODE_PATH | oflag)
        assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))


def test_w4a8_rejects_what_is_not_built(dev):
    from lightop_amd import workloads as wl
    from lightop_amd.moe import fused_experts_impl_w4a8, preshuffle_moe_weight_int4

    layer = wl.TINY_W4
    w1, w2, w1s, w2s = (t.to(dev) for t in wl.make_weights(layer, seed=0))
    x, tw, ids = (t.to(dev) for t in wl.make_inputs(layer, 4, seed=0))
    cache13 = torch.empty(4 * 2 * 1024, dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError):  # weights not in the load-time layout
        fused_experts_impl_w4a8(x, w1, w2, tw, ids, cache13, w1_scale=w1s, w2_scale=w2s, block_shape=[1, 128])
    w1p, w2p = preshuffle_moe_weight_int4(w1), preshuffle_moe_weight_int4(w2)
    with pytest.raises(NotImplementedError):  # neither the reference's per-channel form nor K groups of 128
        fused_experts_impl_w4a8(x, w1p, w2p, tw, ids, cache13, w1_scale=w1s, w2_scale=w2s, block_shape=[128, 128])
    with pytest.raises(NotImplementedError):
        fused_experts_impl_w4a8(x, w1p, w2p, tw, ids, cache13, w1_scale=w1s, w2_scale=w2s, block_shape=[1, 128],
                                w1_zp=torch.zeros(1, device=dev))


@pytest.mark.parametrize("M", [1, 32, 256, 2048])
def test_baseline_int4_layer_sampled_tokens(dev, oracle, M):
    """Qwen3-235B-A22B-shaped layer: a token's output depends on that token only, so a sample of
    tokens goes through the oracle with just the experts it uses."""
    from lightop_amd import _lib, workloads as wl
    from lightop_amd.moe import preshuffle_moe_weight_int4

    layer = wl.QWEN3_235B_W4
    say(f"w4a8 {layer.name} M={M}")
    if not hasattr(test_baseline_int4_layer_sampled_tokens, "w"):
        w1, w2, w1s, w2s = wl.make_weights(layer, seed=0, device=dev, gen_device="cuda")
        from lightop_amd.moe import preshuffle_moe_scale_int4
        test_baseline_int4_layer_sampled_tokens.w = (w1, w2, w1s, w2s, preshuffle_moe_weight_int4(w1),
                                                     preshuffle_moe_weight_int4(w2), preshuffle_moe_scale_int4(w1s),
                                                     preshuffle_moe_scale_int4(w2s))
    w1, w2, w1s, w2s, w1p, w2p, w1sp, w2sp = test_baseline_int4_layer_sampled_tokens.w
    x, tw, ids = (t.to(dev) for t in wl.make_inputs(layer, M, seed=3))
    tokens = torch.randperm(M, generator=torch.Generator().manual_seed(M))[: min(M, 4)].sort().values.to(dev)
    sub_ids = ids[tokens].cpu().long()
    used = torch.unique(sub_ids)
    remap = torch.full((layer.E,), -1, dtype=torch.int64)
    remap[used] = torch.arange(used.numel())
    sel = used.to(dev)
    ref = oracle.fused_experts_w4a8(x[tokens].cpu(), w1[sel].cpu(), w2[sel].cpu(), w1s[sel].cpu(), w2s[sel].cpu(),
                                    tw[tokens].cpu(), remap[sub_ids].to(torch.int32), 16)
    out = run_path(layer, (w1p, w2p, w1sp, w2sp), x, tw, ids, None, dev, 0, 0)
    assert torch.equal(out[tokens].cpu().view(torch.int16), ref.view(torch.int16))
    with oracle.scale_order("separate"):
        ref_s = oracle.fused_experts_w4a8(x[tokens].cpu(), w1[sel].cpu(), w2[sel].cpu(), w1s[sel].cpu(), w2s[sel].cpu(),
                                          tw[tokens].cpu(), remap[sub_ids].to(torch.int32), 16)
    out_s = run_path(layer, (w1p, w2p, w1sp, w2sp), x, tw, ids, None, dev, 0, _lib.LO_GEMM_SEPARATE_ORDER)
    assert torch.equal(out_s[tokens].cpu().view(torch.int16), ref_s.view(torch.int16))
    out2 = run_path(layer, (w1p, w2p, w1sp, w2sp), x, tw, ids, None, dev, 0, _lib.LO_GEMM_FUSED_SCALE)  # within the tolerance
    err = (out2.float() - out.float()).abs()
    assert err.max() <= 1e-2 * out.float().abs().max() and err.sum() <= 2e-3 * out.float().abs().sum()


# ---- the reference's own form: block_shape=None, scales per token and per weight row ---------

def channel_gemm_case(seed, M, k, E, Eg, N, K):
    g = torch.Generator().manual_seed(seed)
    Aq = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int8)
    As = torch.rand(M, 1, generator=g) * 0.05 + 0.005
    W4 = torch.randint(0, 256, (E, N, K // 2), generator=g, dtype=torch.int16).to(torch.uint8)
    Ws = torch.randn(E, N, 1, generator=g) * 1e-3
    ids = torch.stack([torch.randperm(Eg, generator=g)[:k] for _ in range(M)]).to(torch.int32)
    tw = torch.rand(M, k, generator=g) + 0.1
    emap = None
    if Eg != E:
        emap = torch.full((Eg,), -1, dtype=torch.int32)
        emap[:E] = torch.arange(E, dtype=torch.int32)
    return Aq, As, W4, Ws, ids, tw, emap


@pytest.mark.parametrize("M,k,E,Eg,N,K", [(1, 2, 4, 4, 64, 128), (5, 2, 4, 4, 256, 512), (40, 4, 8, 8, 320, 1152),
                                          (100, 8, 4, 16, 512, 768), (300, 2, 3, 3, 128, 2048), (70, 2, 2, 2, 48, 384)])
@pytest.mark.parametrize("bs", [16, 32, 64, 128, 160])
def test_channel_form_gemm_bit_exact(dev, oracle, M, k, E, Eg, N, K, bs):
    from lightop_amd.moe import invoke_fused_moe_kernel_w4a8, moe_align_block_size, preshuffle_moe_weight_int4

    say(f"w4a8 channel gemm M={M} k={k} E={E}/{Eg} N={N} K={K} bs={bs}")
    if bs == 160 and N % 64:
        pytest.skip("160-token blocks need N a multiple of 64")
    Aq, As, W4, Ws, ids, tw, emap = channel_gemm_case(M + N + bs, M, k, E, Eg, N, K)
    rs, re, rp = oracle.moe_align_block_size(ids, bs, Eg, expert_map=emap)
    s, e, p = moe_align_block_size(ids.to(dev), bs, Eg, None if emap is None else emap.to(dev))
    Wd = preshuffle_moe_weight_int4(W4.to(dev))
    for mul in (False, True):
        ref = oracle.moe_gemm_w4a8_channel(Aq, As, W4, Ws, rs, re, rp, tw, mul, k, M * k, bs)
        C = torch.full((M, k, N), 9.0, dtype=torch.bfloat16, device=dev)
        invoke_fused_moe_kernel_w4a8(Aq.to(dev), Wd, C, As.to(dev), Ws.to(dev), None, tw.to(dev), s, e, p, mul, k,
                                     {"BLOCK_SIZE_M": bs}, global_num_experts=Eg)
        torch.cuda.synchronize()
        assert torch.equal(C.cpu().view(M * k, N).view(torch.int16), ref.view(torch.int16)), f"mul_routed={mul}"


def test_channel_form_extreme_sums(dev, oracle):
    """Every product at its extreme: |sum| = K * 128 * 128 is a multiple of 16 below 2^28, exact in fp32."""
    from lightop_amd.moe import invoke_fused_moe_kernel_w4a8, moe_align_block_size, preshuffle_moe_weight_int4

    say("w4a8 channel gemm extreme sums")
    M, E, N, K = 20, 1, 64, 7168
    Aq = torch.full((M, K), -128, dtype=torch.int8)
    W4 = torch.full((E, N, K // 2), 0x88, dtype=torch.uint8)  # every weight -8
    W4[0, 1::2] = 0x77                                        # odd rows: every weight 7
    As, Ws = torch.ones(M, 1), torch.ones(E, N, 1)
    ids = torch.zeros(M, 1, dtype=torch.int32)
    rs, re, rp = oracle.moe_align_block_size(ids, 16, E)
    ref, acc = oracle.moe_gemm_w4a8_channel(Aq, As, W4, Ws, rs, re, rp, None, False, 1, M, 16, dump_acc=True)
    assert int(acc[0, 0]) == K * 16384 and int(acc[0, 1]) == -K * 128 * 112
    s, e, p = moe_align_block_size(ids.to(dev), 16, E)
    C = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    invoke_fused_moe_kernel_w4a8(Aq.to(dev), preshuffle_moe_weight_int4(W4.to(dev)), C, As.to(dev), Ws.to(dev), None,
                                 None, s, e, p, False, 1, {"BLOCK_SIZE_M": 16})
    torch.cuda.synchronize()
    assert torch.equal(C.cpu().view(torch.int16), ref.view(torch.int16))


def run_channel_path(layer, weights_dev, x, tw, ids, emap, dev, bs, **kw):
    from lightop_amd.moe import fused_experts_impl_w4a8

    w1, w2, w1s, w2s = weights_dev
    M = x.shape[0]
    cache13 = torch.empty(M * layer.top_k * max(2 * layer.I, layer.H), dtype=torch.bfloat16, device=dev)
    out = fused_experts_impl_w4a8(x, w1, w2, tw, ids, cache13, global_num_experts=layer.E_global, expert_map=emap,
                                  w1_scale=w1s, w2_scale=w2s, block_shape=None, lightop_amd_block_size_m=bs, **kw)
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("bs", [0, 16, 32, 64, 128, 160])
@pytest.mark.parametrize("with_map", [False, True])
def test_channel_form_whole_path_tiny_bit_exact(dev, oracle, bs, with_map):
    from lightop_amd import workloads as wl
    from lightop_amd.moe import preshuffle_moe_weight_int4

    layer = wl.TINY_W4_PC
    say(f"w4a8 channel whole path tiny bs={bs} map={with_map}")
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=0)
    x, tw, ids = wl.make_inputs(layer, 96, seed=4)
    emap = None
    if with_map:
        emap = torch.full((layer.E,), -1, dtype=torch.int32)
        emap[:5] = torch.arange(5, dtype=torch.int32)
        w1, w2, w1s, w2s = (t[:5].contiguous() for t in (w1, w2, w1s, w2s))
    wd = (preshuffle_moe_weight_int4(w1.to(dev)), preshuffle_moe_weight_int4(w2.to(dev)), w1s.to(dev), w2s.to(dev))
    shared = (torch.randn(96, layer.H, generator=torch.Generator().manual_seed(9)) * 0.1).to(torch.bfloat16)
    for so, rsf in ((None, 1.0), (shared, 2.5)):
        out = run_channel_path(layer, wd, x.to(dev), tw.to(dev), ids.to(dev), None if emap is None else emap.to(dev),
                               dev, bs, shared_output=None if so is None else so.to(dev), routed_scaling_factor=rsf)
        ref = oracle.fused_experts_w4a8_channel(x, w1, w2, w1s, w2s, tw, ids, 16, global_num_experts=layer.E,
                                                expert_map=emap, shared_output=so, routed_scaling_factor=rsf)
        assert ref.float().abs().max() > 0.05
        assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))


def test_channel_form_blocks_of_160_filled(dev, oracle):
    """Two experts, every token on both: blocks of 160 tokens with 1 ... 160 valid rows, every K-loop variant."""
    from lightop_amd import workloads as wl
    from lightop_amd.moe import preshuffle_moe_weight_int4

    layer = wl.MoeLayer("w4pc-160", E=2, E_global=2, top_k=2, H=512, I=256, routing="softmax", weight_bits=4,
                        quant="channel")
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=2)
    wd = (preshuffle_moe_weight_int4(w1.to(dev)), preshuffle_moe_weight_int4(w2.to(dev)), w1s.to(dev), w2s.to(dev))
    for M in (1, 60, 65, 129, 150, 160, 161, 330):
        say(f"w4a8 channel whole path, 160-token blocks, M={M}")
        x, tw, ids = wl.make_inputs(layer, M, seed=M)
        out = run_channel_path(layer, wd, x.to(dev), tw.to(dev), ids.to(dev), None, dev, 160)
        ref = oracle.fused_experts_w4a8_channel(x, w1, w2, w1s, w2s, tw, ids, 16, global_num_experts=layer.E)
        assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("M", [1, 3, 16, 77])
@pytest.mark.parametrize("variant", ["plain", "on_input", "inplace"])
def test_channel_form_ep_share_variants_bit_exact(dev, oracle, M, variant):
    from lightop_amd import workloads as wl
    from lightop_amd.moe import fused_experts_impl_w4a8, preshuffle_moe_weight_int4

    say(f"w4a8 channel ep-share M={M} {variant}")
    layer = wl.MoeLayer("ep-w4pc", E=4, E_global=32, top_k=8, H=512, I=256, routing="grouped_sigmoid", n_group=8,
                        topk_group=4, routed_scaling=2.5, weight_bits=4, quant="channel")
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=3)
    x, tw, ids = wl.make_inputs(layer, M, seed=3)
    emap = wl.expert_map_for(layer)
    cache13 = torch.empty(M * layer.top_k * max(2 * layer.I, layer.H), dtype=torch.bfloat16, device=dev)
    xd = x.to(dev)
    out = fused_experts_impl_w4a8(
        xd, preshuffle_moe_weight_int4(w1.to(dev)), preshuffle_moe_weight_int4(w2.to(dev)), tw.to(dev), ids.to(dev),
        cache13, inplace=variant == "inplace", apply_router_weight_on_input=variant == "on_input",
        global_num_experts=32, expert_map=emap.to(dev), w1_scale=w1s.to(dev), w2_scale=w2s.to(dev), block_shape=None)
    torch.cuda.synchronize()
    if variant == "inplace":
        assert out.data_ptr() == xd.data_ptr()
    ref = oracle.fused_experts_w4a8_channel(x, w1, w2, w1s, w2s, tw, ids, 16, global_num_experts=32, expert_map=emap,
                                            apply_router_weight_on_input=variant == "on_input")
    assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("M", [1, 32, 512, 2048, 4096])
def test_channel_form_int4_layer_sampled_tokens(dev, oracle, M):
    """Qwen3-235B-A22B-shaped layer in the reference's own int4 form, sampled tokens against the oracle."""
    from lightop_amd import workloads as wl
    from lightop_amd.moe import preshuffle_moe_weight_int4

    layer = wl.QWEN3_235B_W4_PC
    say(f"w4a8 channel {layer.name} M={M}")
    me = test_channel_form_int4_layer_sampled_tokens
    if not hasattr(me, "w"):
        w1, w2, w1s, w2s = wl.make_weights(layer, seed=0, device=dev, gen_device="cuda")
        me.w = (w1, w2, w1s, w2s, preshuffle_moe_weight_int4(w1), preshuffle_moe_weight_int4(w2))
    w1, w2, w1s, w2s, w1p, w2p = me.w
    x, tw, ids = (t.to(dev) for t in wl.make_inputs(layer, M, seed=3))
    tokens = torch.randperm(M, generator=torch.Generator().manual_seed(M))[: min(M, 4)].sort().values.to(dev)
    sub_ids = ids[tokens].cpu().long()
    used = torch.unique(sub_ids)
    remap = torch.full((layer.E,), -1, dtype=torch.int64)
    remap[used] = torch.arange(used.numel())
    sel = used.to(dev)
    ref = oracle.fused_experts_w4a8_channel(x[tokens].cpu(), w1[sel].cpu(), w2[sel].cpu(), w1s[sel].cpu(),
                                            w2s[sel].cpu(), tw[tokens].cpu(), remap[sub_ids].to(torch.int32), 16)
    out = run_channel_path(layer, (w1p, w2p, w1s, w2s), x, tw, ids, None, dev, 0)
    assert torch.equal(out[tokens].cpu().view(torch.int16), ref.view(torch.int16))
