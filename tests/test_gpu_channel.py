"""GPU parity of the per-channel W8A8 path (per_channel_quant=True, block_shape=None), through the
C ABI, bit for bit against the oracle: per-token quant, the grouped GEMM with every kernel family
and block size, SiLU-and-mul with per-token quant, the whole path, and a Qwen3-30B-A3B-shaped layer
on sampled tokens."""
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


@pytest.mark.parametrize("rows,cols", [(1, 128), (3, 1024), (17, 2048), (5, 7168), (2, 8200), (64, 24), (9, 20480)])
def test_per_token_quant_bit_exact(dev, oracle, rows, cols):
    from lightop_amd.quant import per_token_quant_int8

    say(f"per_token_quant rows={rows} cols={cols}")
    g = torch.Generator().manual_seed(rows * 31 + cols)
    x = (torch.randn(rows, cols, generator=g) * 3).to(torch.bfloat16)
    x[0, : min(cols, 64)] = 0  # some exact zeros
    if rows > 2:
        x[2] = 0  # a zero row: the 1e-10 floor
    # ties: a row whose maximum is 127 makes the multiplier exactly 1
    x[-1, :8] = torch.tensor([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5]).to(torch.bfloat16)
    x[-1, 8:] = x[-1, 8:].clamp(-100, 100)
    rq, rs = oracle.per_token_quant_int8(x)
    q, s = per_token_quant_int8(x.to(dev))
    torch.cuda.synchronize()
    assert s.shape == (rows, 1) and torch.equal(s.cpu(), rs) and torch.equal(q.cpu(), rq)


@pytest.mark.parametrize("rows,I", [(1, 128), (7, 768), (33, 2048), (4, 4104), (130, 256)])
def test_fuse_silu_mul_quant_bit_exact(dev, oracle, rows, I):
    from lightop_amd import fuse_silu_mul_quant

    say(f"fuse_silu_mul_quant rows={rows} I={I}")
    g = torch.Generator().manual_seed(rows + I)
    c1 = (torch.randn(rows, 2 * I, generator=g) * 3).to(torch.bfloat16)
    if rows > 3:
        c1[3] = 0  # zero row: scale 0, multiplier 0
    # every finite bf16 gate below 1e18 appears somewhere when the tensor is large enough
    n = min(c1.numel() // 2, 65536)
    pats = torch.arange(65536, dtype=torch.int32)[:n].to(torch.int16).view(torch.bfloat16).float()
    pats = torch.where(pats.isfinite() & (pats.abs() < 1e18), pats, torch.zeros(())).to(torch.bfloat16)
    if rows >= 33:
        c1[:32, :I] = pats[: 32 * I].reshape(32, I)
        c1[:32, I:] = (torch.rand(32, I, generator=g) * 1e-3).to(torch.bfloat16)
    rq, rs = oracle.fuse_silu_mul_quant(c1)
    q, s = fuse_silu_mul_quant(c1.to(dev))
    torch.cuda.synchronize()
    assert torch.equal(s.cpu(), rs) and torch.equal(q.cpu(), rq)
    # num_local_tokens: only the first n * topk rows are written
    if rows >= 4:
        out = torch.full((rows, I), 77, dtype=torch.int8, device=dev)
        sc = torch.full((rows, 1), -1.0, dtype=torch.float32, device=dev)
        nlt = torch.tensor([1], dtype=torch.int32, device=dev)
        fuse_silu_mul_quant(c1.to(dev), nlt, 2, -1, out, sc)
        torch.cuda.synchronize()
        assert torch.equal(out.cpu()[:2], rq[:2]) and (out.cpu()[2:] == 77).all() and (sc.cpu()[2:] == -1).all()


def test_fuse_silu_mul_quant_skips_rows_of_other_ranks(dev, oracle):
    """expert_ids (fuse_silu_mul_quant.cu:269-283): rows marked -1 keep whatever output and scales held."""
    from lightop_amd import fuse_silu_mul_quant

    for rows, I in ((37, 768), (9, 4096)):  # one wavefront per row, one workgroup per row
        say(f"fuse_silu_mul_quant expert_ids rows={rows} I={I}")
        g = torch.Generator().manual_seed(rows)
        c1 = torch.randn(rows, 2 * I, generator=g).to(torch.bfloat16)
        eids = torch.randint(-1, 3, (rows,), generator=g, dtype=torch.int32)
        eids[1], eids[rows - 1], eids[0] = -1, -1, 2
        rq, rs = oracle.fuse_silu_mul_quant(c1)
        out = torch.full((rows, I), 77, dtype=torch.int8, device=dev)
        sc = torch.full((rows, 1), -5.0, dtype=torch.float32, device=dev)
        fuse_silu_mul_quant(c1.to(dev), None, 1, -1, out, sc, eids.to(dev))
        torch.cuda.synchronize()
        keep = eids != -1
        assert keep.any() and (~keep).any()
        assert torch.equal(out.cpu()[keep], rq[keep]) and torch.equal(sc.cpu()[keep].view(torch.int32), rs[keep].view(torch.int32).reshape(-1, 1))
        assert (out.cpu()[~keep] == 77).all() and (sc.cpu()[~keep] == -5.0).all()


def gemm_case(seed, M, k, E, Eg, N, K):
    g = torch.Generator().manual_seed(seed)
    Aq = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int8)
    As = torch.rand(M, 1, generator=g) * 0.05 + 0.005
    W = torch.randint(-128, 128, (E, N, K), generator=g, dtype=torch.int8)
    Ws = torch.randn(E, N, 1, generator=g) * 1e-2
    ids = torch.stack([torch.randperm(Eg, generator=g)[:k] for _ in range(M)]).to(torch.int32)
    tw = torch.rand(M, k, generator=g) + 0.1
    emap = None
    if Eg != E:
        emap = torch.full((Eg,), -1, dtype=torch.int32)
        emap[:E] = torch.arange(E, dtype=torch.int32)
    return Aq, As, W, Ws, ids, tw, emap


@pytest.mark.parametrize("M,k,E,Eg,N,K", [(1, 2, 4, 4, 64, 128), (5, 2, 4, 4, 256, 512), (40, 4, 8, 8, 320, 1152),
                                          (100, 8, 4, 16, 512, 768), (300, 2, 3, 3, 128, 2048), (70, 2, 2, 2, 48, 384)])
@pytest.mark.parametrize("bs", [16, 32, 64, 128, 160])
@pytest.mark.parametrize("shuf", [False, True])
def test_moe_gemm_w8a8_bit_exact(dev, oracle, M, k, E, Eg, N, K, bs, shuf):
    from lightop_amd import _lib
    from lightop_amd.gemmopt import moe_gemm_w8a8
    from lightop_amd.moe import moe_align_block_size, preshuffle_moe_weight

    say(f"channel gemm M={M} k={k} E={E}/{Eg} N={N} K={K} bs={bs} shuf={shuf}")
    if bs == 160 and (not shuf or N % 64):
        pytest.skip("160-token blocks: weights in the load-time layout, N a multiple of 64")
    Aq, As, W, Ws, ids, tw, emap = gemm_case(M + N + bs, M, k, E, Eg, N, K)
    rs, re, rp = oracle.moe_align_block_size(ids, bs, Eg, expert_map=emap)
    s, e, p = moe_align_block_size(ids.to(dev), bs, Eg, None if emap is None else emap.to(dev))
    Wd = preshuffle_moe_weight(W.to(dev)) if shuf else W.to(dev)
    for mul in (False, True):
        for flags in (0, _lib.LO_GEMM_FORCE_STREAMING):
            ref = oracle.moe_gemm_w8a8(Aq, As, W, Ws, rs, re, rp, tw, mul, k, M * k, bs)
            C = torch.full((M, k, N), 9.0, dtype=torch.bfloat16, device=dev)
            moe_gemm_w8a8(Aq.to(dev), Wd, C, As.to(dev), Ws.to(dev), tw.to(dev) if mul else None, s, e, p, k,
                          {"BLOCK_SIZE_M": bs, "MODE": 0, "DELTA": 0}, flags=flags)
            torch.cuda.synchronize()
            assert torch.equal(C.cpu().view(M * k, N).view(torch.int16), ref.view(torch.int16)), \
                f"mul_routed={mul} flags={flags}"


def test_moe_gemm_w8a8_extreme_sums(dev, oracle):
    """Every product at its extreme: |sum| = K * 128 * 128 stays exact in int32 and in the fp32 epilogue."""
    from lightop_amd.gemmopt import moe_gemm_w8a8
    from lightop_amd.moe import moe_align_block_size

    say("channel gemm extreme sums")
    M, k, E, N, K = 70, 1, 1, 64, 7168
    Aq = torch.full((M, K), -128, dtype=torch.int8)
    W = torch.full((E, N, K), -128, dtype=torch.int8)
    W[0, 1::2] = 127
    As = torch.ones(M, 1)
    Ws = torch.ones(E, N, 1)
    ids = torch.zeros(M, 1, dtype=torch.int32)
    for bs in (16, 64):
        rs, re, rp = oracle.moe_align_block_size(ids, bs, E)
        ref, acc = oracle.moe_gemm_w8a8(Aq, As, W, Ws, rs, re, rp, None, False, k, M, bs, dump_acc=True)
        assert int(acc[0, 0]) == K * 16384 and int(acc[0, 1]) == -K * 128 * 127
        s, e, p = moe_align_block_size(ids.to(dev), bs, E)
        C = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
        moe_gemm_w8a8(Aq.to(dev), W.to(dev), C, As.to(dev), Ws.to(dev), None, s, e, p, k, {"BLOCK_SIZE_M": bs})
        torch.cuda.synchronize()
        assert torch.equal(C.cpu().view(torch.int16), ref.view(torch.int16))


def run_path(layer, weights_dev, x, tw, ids, emap, dev, bs, **kw):
    from lightop_amd.moe import fused_experts_impl_int8

    w1, w2, w1s, w2s = weights_dev
    M = x.shape[0]
    cache13 = torch.empty(M * layer.top_k * max(2 * layer.I, layer.H), dtype=torch.bfloat16, device=dev)
    out = fused_experts_impl_int8(x, w1, w2, tw, ids, cache13, use_int8_w8a8=True, per_channel_quant=True,
                                  global_num_experts=layer.E_global, expert_map=emap, w1_scale=w1s, w2_scale=w2s,
                                  block_shape=None, lightop_amd_block_size_m=bs, **kw)
    torch.cuda.synchronize()
    return out


def test_whole_path_blocks_of_160_filled(dev, oracle):
    """Two experts, every token on both: blocks of 160 tokens with 1 ... 160 valid rows, every K-loop variant;
    the router weight in the second GEMM's epilogue (ts = w * a_s) and on the input."""
    from lightop_amd import workloads as wl
    from lightop_amd.moe import preshuffle_moe_weight

    layer = wl.MoeLayer("pc-160", E=2, E_global=2, top_k=2, H=512, I=256, routing="softmax", quant="channel")
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=2)
    wd = (preshuffle_moe_weight(w1.to(dev)), preshuffle_moe_weight(w2.to(dev)), w1s.to(dev), w2s.to(dev))
    for M in (1, 60, 65, 129, 150, 160, 161, 330):
        for on_input in (False, True):
            say(f"channel whole path, 160-token blocks, M={M} on_input={on_input}")
            x, tw, ids = wl.make_inputs(layer, M, seed=M)
            out = run_path(layer, wd, x.to(dev), tw.to(dev), ids.to(dev), None, dev, 160,
                           apply_router_weight_on_input=on_input)
            ref = oracle.fused_experts_channel_int8(x, w1, w2, w1s, w2s, tw, ids, 16, global_num_experts=layer.E,
                                                    apply_router_weight_on_input=on_input)
            assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("bs", [0, 16, 32, 64, 128, 160])
@pytest.mark.parametrize("with_map", [False, True])
@pytest.mark.parametrize("shuf", [False, True])
def test_whole_path_tiny_bit_exact(dev, oracle, bs, with_map, shuf):
    from lightop_amd import workloads as wl
    from lightop_amd.moe import preshuffle_moe_weight

    layer = wl.TINY_PC
    say(f"channel whole path tiny bs={bs} map={with_map} shuf={shuf}")
    if bs == 160 and not shuf:
        pytest.skip("160-token blocks: weights in the load-time layout")
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=0)
    x, tw, ids = wl.make_inputs(layer, 96, seed=4)
    emap = None
    if with_map:
        emap = torch.full((layer.E,), -1, dtype=torch.int32)
        emap[:5] = torch.arange(5, dtype=torch.int32)
        w1, w2, w1s, w2s = (t[:5].contiguous() for t in (w1, w2, w1s, w2s))
    prep = preshuffle_moe_weight if shuf else (lambda t: t)
    wd = (prep(w1.to(dev)), prep(w2.to(dev)), w1s.to(dev), w2s.to(dev))
    shared = (torch.randn(96, layer.H, generator=torch.Generator().manual_seed(9)) * 0.1).to(torch.bfloat16)
    for so, rsf in ((None, 1.0), (shared, 2.5)):
        out = run_path(layer, wd, x.to(dev), tw.to(dev), ids.to(dev), None if emap is None else emap.to(dev), dev,
                       bs, shared_output=None if so is None else so.to(dev), routed_scaling_factor=rsf)
        ref = oracle.fused_experts_channel_int8(x, w1, w2, w1s, w2s, tw, ids, 16, global_num_experts=layer.E,
                                                expert_map=emap, shared_output=so, routed_scaling_factor=rsf)
        assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("M", [1, 3, 16, 77])
@pytest.mark.parametrize("variant", ["plain", "shared", "on_input", "inplace"])
def test_whole_path_ep_share_variants_bit_exact(dev, oracle, M, variant):
    """An expert-parallel share (4 of 32 experts held here) with the optional arguments of the entry point."""
    from lightop_amd import workloads as wl
    from lightop_amd.moe import fused_experts_impl_int8

    say(f"channel ep-share M={M} {variant}")
    layer = wl.MoeLayer("ep-pc", E=4, E_global=32, top_k=8, H=512, I=256, routing="grouped_sigmoid", n_group=8,
                        topk_group=4, routed_scaling=2.5, quant="channel")
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=3)
    x, tw, ids = wl.make_inputs(layer, M, seed=3)
    emap = wl.expert_map_for(layer)
    sh = torch.randn(M, layer.H, generator=torch.Generator().manual_seed(8)).to(torch.bfloat16) \
        if variant == "shared" else None
    cache13 = torch.empty(M * layer.top_k * max(2 * layer.I, layer.H), dtype=torch.bfloat16, device=dev)
    xd = x.to(dev)
    out = fused_experts_impl_int8(
        xd, w1.to(dev), w2.to(dev), tw.to(dev), ids.to(dev), cache13, inplace=variant == "inplace",
        apply_router_weight_on_input=variant == "on_input", use_int8_w8a8=True, per_channel_quant=True,
        global_num_experts=32, expert_map=emap.to(dev), w1_scale=w1s.to(dev), w2_scale=w2s.to(dev), block_shape=None,
        routed_scaling_factor=2.5 if sh is not None else 1.0, shared_output=None if sh is None else sh.to(dev),
        lightop_amd_block_size_m=16)
    torch.cuda.synchronize()
    if variant == "inplace":
        assert out.data_ptr() == xd.data_ptr()
    ref = oracle.fused_experts_channel_int8(x, w1, w2, w1s, w2s, tw, ids, 16, global_num_experts=32, expert_map=emap,
                                            apply_router_weight_on_input=variant == "on_input",
                                            routed_scaling_factor=2.5 if sh is not None else 1.0, shared_output=sh)
    assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))


def test_whole_path_in_chunks(dev, oracle, monkeypatch):
    """More tokens than LMSLIM_FUSED_MOE_CHUNK_SIZE: the chunks (int8.py:703-722) give the same rows."""
    from lightop_amd import workloads as wl

    say("channel whole path in chunks")
    monkeypatch.setenv("LMSLIM_FUSED_MOE_CHUNK_SIZE", "40")
    layer = wl.TINY_PC
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=0)
    x, tw, ids = wl.make_inputs(layer, 100, seed=6)
    out = run_path(layer, (w1.to(dev), w2.to(dev), w1s.to(dev), w2s.to(dev)), x.to(dev), tw.to(dev), ids.to(dev),
                   None, dev, 16)
    ref = oracle.fused_experts_channel_int8(x, w1, w2, w1s, w2s, tw, ids, 16)
    assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))


def _staged_reference(oracle, layer, i_q, i_s, w, tw, ids, bs, emap=None, shared=None, factor=1.0, activation="silu"):
    """The per-channel path from its stages on the CPU, starting from a given quantised input."""
    w1, w2, w1s, w2s = w
    M, k = ids.shape
    S = M * k
    srt, eids, ntpp = oracle.moe_align_block_size(ids, bs, layer.E_global, expert_map=emap)
    c1 = oracle.moe_gemm_w8a8(i_q, i_s, w1, w1s, srt, eids, ntpp, None, False, k, S, bs)
    if activation == "gelu":  # gelu_and_mul, then per_token_quant_int8 with its floor (int8.py:826-838)
        a2q, a2s = oracle.per_token_quant_int8(oracle.gelu_and_mul(c1))
    else:
        a2q, a2s = oracle.fuse_silu_mul_quant(c1)
    c3 = oracle.moe_gemm_w8a8(a2q, a2s, w2, w2s, srt, eids, ntpp, tw, True, 1, S, bs)
    return oracle.moe_sum(c3.view(M, k, layer.H), shared, factor)


@pytest.mark.parametrize("bs", [0, 16, 64, 128])
@pytest.mark.parametrize("chunk", [None, 48])
def test_caller_quantised_input(dev, oracle, monkeypatch, bs, chunk):
    """i_q / i_s with LMSLIM_USE_FUSED_RMS_QUANT (int8.py:291-293): the path starts from the caller's int8 rows
    and per-token scales - here unrelated to hidden_states, which must not be read - and without the flag,
    or in the block form, they are ignored."""
    from lightop_amd import workloads as wl
    from lightop_amd.moe import fused_experts_impl_int8

    say(f"channel whole path from i_q / i_s, bs={bs} chunk={chunk}")
    layer = wl.TINY_PC
    w = wl.make_weights(layer, seed=0)
    wd = tuple(t.to(dev) for t in w)
    M = 100
    x, tw, ids = wl.make_inputs(layer, M, seed=8)
    g = torch.Generator().manual_seed(5)
    i_q = torch.randint(-127, 128, (M, layer.H), generator=g, dtype=torch.int8)
    i_s = (torch.rand(M, 1, generator=g) * 0.04 + 0.005).to(torch.float32)
    shared = (torch.randn(M, layer.H, generator=g) * 0.1).to(torch.bfloat16)
    ref = _staged_reference(oracle, layer, i_q, i_s, w, tw, ids, bs or 16, shared=shared, factor=2.0)
    assert ref.float().abs().max() > 0.05
    plain = oracle.fused_experts_channel_int8(x, *w, tw, ids, 16, shared_output=shared, routed_scaling_factor=2.0)
    assert not torch.equal(plain, ref)
    kw = dict(shared_output=shared.to(dev), routed_scaling_factor=2.0, i_q=i_q.to(dev), i_s=i_s.to(dev))
    if chunk:
        monkeypatch.setenv("LMSLIM_FUSED_MOE_CHUNK_SIZE", str(chunk))
    # without the flag the arguments are ignored
    monkeypatch.delenv("LMSLIM_USE_FUSED_RMS_QUANT", raising=False)
    monkeypatch.delenv("USE_FUSED_RMS_QUANT", raising=False)
    out = run_path(layer, wd, x.to(dev), tw.to(dev), ids.to(dev), None, dev, bs, **kw)
    assert torch.equal(out.cpu().view(torch.int16), plain.view(torch.int16))
    monkeypatch.setenv("LMSLIM_USE_FUSED_RMS_QUANT", "1")
    poison = torch.full_like(x, float("nan")).to(dev)  # any read of hidden_states would show
    out = run_path(layer, wd, poison, tw.to(dev), ids.to(dev), None, dev, bs, **kw)
    assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))
    # the block form quantises hidden_states itself whatever the flag says (int8.py:297-301)
    lb = wl.TINY
    wb = wl.make_weights(lb, seed=0)
    xb, twb, idsb = wl.make_inputs(lb, M, seed=8)
    cache13 = torch.empty(M * lb.top_k * max(2 * lb.I, lb.H), dtype=torch.bfloat16, device=dev)
    outb = fused_experts_impl_int8(xb.to(dev), wb[0].to(dev), wb[1].to(dev), twb.to(dev), idsb.to(dev), cache13,
                                   use_int8_w8a8=True, w1_scale=wb[2].to(dev), w2_scale=wb[3].to(dev),
                                   block_shape=[128, 128], i_q=i_q.to(dev), i_s=i_s.to(dev))
    torch.cuda.synchronize()
    refb = oracle.fused_experts_block_int8(xb, *wb, twb, idsb, 16)
    assert torch.equal(outb.cpu().view(torch.int16), refb.view(torch.int16))


def test_caller_quantised_input_with_gelu(dev, oracle, monkeypatch):
    from lightop_amd import workloads as wl

    say("channel whole path from i_q / i_s, GELU")
    monkeypatch.setenv("LMSLIM_USE_FUSED_RMS_QUANT", "1")
    layer = wl.TINY_PC
    w = wl.make_weights(layer, seed=1)
    M = 50
    x, tw, ids = wl.make_inputs(layer, M, seed=3)
    g = torch.Generator().manual_seed(13)
    i_q = torch.randint(-127, 128, (M, layer.H), generator=g, dtype=torch.int8)
    i_s = (torch.rand(M, 1, generator=g) * 0.04 + 0.005).to(torch.float32)
    ref = _staged_reference(oracle, layer, i_q, i_s, w, tw, ids, 16, activation="gelu")
    out = run_path(layer, tuple(t.to(dev) for t in w), x.to(dev), tw.to(dev), ids.to(dev), None, dev, 16,
                   i_q=i_q.to(dev), i_s=i_s.to(dev), activation="gelu")
    assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))


def test_caller_quantised_input_on_an_expert_parallel_share(dev, oracle, monkeypatch):
    from lightop_amd import workloads as wl

    say("channel whole path from i_q / i_s, expert-parallel share")
    monkeypatch.setenv("LMSLIM_USE_FUSED_RMS_QUANT", "1")
    layer = wl.MoeLayer("ep-pc-q", E=4, E_global=32, top_k=8, H=512, I=256, routing="grouped_sigmoid", n_group=8,
                        topk_group=4, routed_scaling=2.5, quant="channel")
    w = wl.make_weights(layer, seed=2)
    M = 77
    x, tw, ids = wl.make_inputs(layer, M, seed=2)
    emap = wl.expert_map_for(layer)
    g = torch.Generator().manual_seed(9)
    i_q = torch.randint(-127, 128, (M, layer.H), generator=g, dtype=torch.int8)
    i_s = (torch.rand(M, generator=g) * 0.04 + 0.005).to(torch.float32)
    ref = _staged_reference(oracle, layer, i_q, i_s, w, tw, ids, 16, emap=emap)
    out = run_path(layer, tuple(t.to(dev) for t in w), x.to(dev), tw.to(dev), ids.to(dev), emap.to(dev), dev, 0,
                   i_q=i_q.to(dev), i_s=i_s.to(dev))
    assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))


def test_channel_path_rejects_mixed_arguments(dev):
    from lightop_amd import workloads as wl
    from lightop_amd.moe import fused_experts_impl_int8

    layer = wl.TINY_PC
    w1, w2, w1s, w2s = (t.to(dev) for t in wl.make_weights(layer, seed=0))
    x, tw, ids = (t.to(dev) for t in wl.make_inputs(layer, 4, seed=0))
    cache13 = torch.empty(4 * 2 * 1024, dtype=torch.bfloat16, device=dev)
    with pytest.raises(NotImplementedError):  # per-channel scales with a block shape
        fused_experts_impl_int8(x, w1, w2, tw, ids, cache13, use_int8_w8a8=True, per_channel_quant=True,
                                w1_scale=w1s, w2_scale=w2s, block_shape=[128, 128])
    with pytest.raises(NotImplementedError):  # neither block nor channel
        fused_experts_impl_int8(x, w1, w2, tw, ids, cache13, use_int8_w8a8=True, w1_scale=w1s, w2_scale=w2s,
                                block_shape=None)


@pytest.mark.parametrize("M", [1, 32, 512, 2048, 8192])
def test_qwen3_channel_layer_sampled_tokens(dev, oracle, M):
    """A token's output depends on that token only: a sample of tokens goes through the oracle with
    just the experts it uses."""
    from lightop_amd import workloads as wl
    from lightop_amd.moe import preshuffle_moe_weight

    layer = wl.QWEN3_30B_PC
    say(f"channel {layer.name} M={M}")
    if not hasattr(test_qwen3_channel_layer_sampled_tokens, "w"):
        w1, w2, w1s, w2s = wl.make_weights(layer, seed=0, device=dev, gen_device="cuda")
        test_qwen3_channel_layer_sampled_tokens.w = (w1, w2, w1s, w2s, preshuffle_moe_weight(w1),
                                                     preshuffle_moe_weight(w2))
    w1, w2, w1s, w2s, w1p, w2p = test_qwen3_channel_layer_sampled_tokens.w
    x, tw, ids = (t.to(dev) for t in wl.make_inputs(layer, M, seed=3))
    tokens = torch.randperm(M, generator=torch.Generator().manual_seed(M))[: min(M, 6)].sort().values.to(dev)
    sub_ids = ids[tokens].cpu().long()
    used = torch.unique(sub_ids)
    remap = torch.full((layer.E,), -1, dtype=torch.int64)
    remap[used] = torch.arange(used.numel())
    sel = used.to(dev)
    ref = oracle.fused_experts_channel_int8(x[tokens].cpu(), w1[sel].cpu(), w2[sel].cpu(), w1s[sel].cpu(),
                                            w2s[sel].cpu(), tw[tokens].cpu(), remap[sub_ids].to(torch.int32), 16)
    for wa, wb in ((w1, w2), (w1p, w2p)):
        out = run_path(layer, (wa, wb, w1s, w2s), x, tw, ids, None, dev, 0)
        assert torch.equal(out[tokens].cpu().view(torch.int16), ref.view(torch.int16))
