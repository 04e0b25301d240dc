"""GPU parity of the 160-token form of the direct-to-LDS GEMM kernel (block size 160: chosen by the tile table
around 128 slots per expert, where a 128-token block would spill a few tokens into a second pass over the
expert's weights), through the C ABI, bit for bit against the oracle: the plain GEMM and the first stage with its
fused SiLU*mul + re-quantisation at every fill level of a block, the activation + group-quantisation launch that
follows the plain first GEMM with fp16 rows and GELU, and the whole path, explicitly and where the table picks it."""
import math

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
    W = torch.randint(-127, 128, (E, N, K), generator=g, dtype=torch.int8)
    As = torch.rand(M, K // 128, generator=g) * 0.05 + 0.005
    Ws = torch.exp(torch.randn(E, (N + 127) // 128, K // 128, generator=g) * 0.3 + math.log(3e-2))
    ids = torch.stack([torch.randperm(Eg, generator=g)[:k] for _ in range(M)]).to(torch.int32)
    tw = torch.rand(M, k, generator=g) + 0.1
    emap = None
    if Eg != E:
        emap = torch.full((Eg,), -1, dtype=torch.int32)
        emap[:E] = torch.arange(E, dtype=torch.int32)
    return Aq, As, W, Ws, ids, tw, emap


@pytest.mark.parametrize("count,K", [(c, 384) for c in (1, 32, 33, 127, 128, 129, 130, 144, 145, 159, 160, 161, 200, 330)] +
                         [(c, k) for k in (128, 256, 1024) for c in (40, 136, 160)])
def test_gemm_160_token_blocks_fill_levels(dev, oracle, count, K):
    """Blocks of 160 holding 1 ... 160 valid tokens (the K loop comes in variants for 64, 128 and 160 tokens
    in use) and experts that need a second and a third block; one, two, three and eight K blocks."""
    from lightop_amd.moe import invoke_fused_moe_kernel_int8, moe_align_block_size, preshuffle_moe_weight

    say(f"160-token blocks, {count} tokens on expert 0, K = {K}")
    bs, E, N = 160, 2, 256
    M = count + 3
    Aq, As, W, Ws, _, tw, _ = gemm_case(count, M, 1, E, E, N, K)
    ids = torch.ones(M, 1, dtype=torch.int32)
    ids[torch.randperm(M, generator=torch.Generator().manual_seed(count))[:count]] = 0
    rs, re, rp = oracle.moe_align_block_size(ids, bs, E)
    s, e, p = moe_align_block_size(ids.to(dev), bs, E)
    assert torch.equal(s.cpu()[: int(rp[0])], rs[: int(rp[0])]) and torch.equal(e.cpu()[: int(rp[0]) // bs], re[: int(rp[0]) // bs])
    Wsh = preshuffle_moe_weight(W.to(dev))
    from lightop_amd import _lib

    for mul in (False, True):
        # the default order, the order without fp fusion (both bit-exact) and the fused-scale order
        for order, flags in (("contract", 0), ("separate", _lib.LO_GEMM_SEPARATE_ORDER), ("fused", _lib.LO_GEMM_FUSED_SCALE)):
            with oracle.scale_order("contract" if order == "fused" else order):
                ref = oracle.moe_gemm_block_int8(Aq, As, W, Ws, rs, re, rp, tw, mul, 1, M, bs)
            C = torch.full((M, 1, N), 7.0, dtype=torch.bfloat16, device=dev)
            invoke_fused_moe_kernel_int8(Aq.to(dev), Wsh, C, As.to(dev), Ws.to(dev), tw.to(dev), s, e, p, mul, 1,
                                         {"BLOCK_SIZE_M": bs}, flags=flags)
            torch.cuda.synchronize()
            got = C.view(M, -1).cpu()
            if order == "fused":  # the optional order: last-ulp differences in fp32
                err = (got.float() - ref.float()).abs()
                assert err.max() <= 1e-2 * ref.float().abs().max()
            else:
                assert torch.equal(got.view(torch.int16), ref.view(torch.int16)), f"mul_routed={mul} order={order}"


@pytest.mark.parametrize("M,k,E,Eg,N,K", [(5, 2, 4, 4, 256, 512), (400, 4, 8, 8, 320, 1152), (900, 8, 4, 16, 512, 768),
                                          (700, 2, 3, 3, 128, 2048)])
def test_gemm_160_bit_exact(dev, oracle, M, k, E, Eg, N, K):
    from lightop_amd import _lib
    from lightop_amd.moe import invoke_fused_moe_kernel_int8, moe_align_block_size, preshuffle_moe_weight

    say(f"gemm bs=160 M={M} k={k} E={E}/{Eg} N={N} K={K}")
    bs = 160
    Aq, As, W, Ws, ids, tw, emap = gemm_case(M + N, M, k, E, Eg, N, K)
    rs, re, rp = oracle.moe_align_block_size(ids, bs, Eg, expert_map=emap)
    s, e, p = moe_align_block_size(ids.to(dev), bs, Eg, None if emap is None else emap.to(dev))
    Wsh = preshuffle_moe_weight(W.to(dev))
    for mul in (False, True):
        ref = oracle.moe_gemm_block_int8(Aq, As, W, Ws, rs, re, rp, tw, mul, k, M * k, bs)
        C = torch.full((M, k, N), 9.0, dtype=torch.bfloat16, device=dev)
        invoke_fused_moe_kernel_int8(Aq.to(dev), Wsh, C, As.to(dev), Ws.to(dev), tw.to(dev), s, e, p, mul, k,
                                     {"BLOCK_SIZE_M": bs}, fused_scale=False)
        torch.cuda.synchronize()
        assert torch.equal(C.cpu().view(M * k, N).view(torch.int16), ref.view(torch.int16)), f"mul_routed={mul}"
    # blocks of experts on other ranks left untouched on request
    if emap is not None:
        C = torch.full((M, k, N), 9.0, dtype=torch.bfloat16, device=dev)
        invoke_fused_moe_kernel_int8(Aq.to(dev), Wsh, C, As.to(dev), Ws.to(dev), tw.to(dev), s, e, p, False, k,
                                     {"BLOCK_SIZE_M": bs}, fused_scale=False, flags=_lib.LO_GEMM_SKIP_NONLOCAL)
        torch.cuda.synchronize()
        local = (emap[ids.reshape(-1).long()] >= 0)
        ref = oracle.moe_gemm_block_int8(Aq, As, W, Ws, rs, re, rp, tw, False, k, M * k, bs)
        got = C.cpu().view(M * k, N)
        assert torch.equal(got[local].view(torch.int16), ref[local].view(torch.int16)) and (got[~local] == 9.0).all()


def test_160_token_blocks_need_the_load_time_layout(dev):
    from lightop_amd.moe import invoke_fused_moe_gemm1_silu_quant, invoke_fused_moe_kernel_int8, moe_align_block_size

    Aq, As, W, Ws, ids, tw, _ = gemm_case(1, 8, 2, 4, 4, 256, 256)
    s, e, p = moe_align_block_size(ids.to(dev), 160, 4)
    C = torch.empty((8, 2, 256), dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError, match="160-token blocks"):  # row-major weights
        invoke_fused_moe_kernel_int8(Aq.to(dev), W.to(dev), C, As.to(dev), Ws.to(dev), tw.to(dev), s, e, p, False, 2,
                                     {"BLOCK_SIZE_M": 160})
    with pytest.raises(RuntimeError, match="160-token blocks"):  # the fused first stage as well
        invoke_fused_moe_gemm1_silu_quant(Aq.to(dev), W.to(dev), As.to(dev), Ws.to(dev), tw.to(dev), s, e, p, False, 2,
                                          16, {"BLOCK_SIZE_M": 160})


@pytest.mark.parametrize("count,K", [(c, 384) for c in (1, 32, 33, 64, 65, 127, 128, 129, 144, 145, 160, 161, 330)] +
                         [(c, k) for k in (128, 256, 1024) for c in (40, 136, 160)])
def test_gemm1_fused_160_token_blocks_fill_levels(dev, oracle, count, K):
    """The first stage with its fused epilogue on blocks of 160 holding 1 ... 160 valid tokens, in both bit-exact
    scale orders, with and without the router weight: int8 activations and group scales against the oracle.
    (The SiLU band and the amax exchange of this form live in the waves' weight stages after the K loop.)"""
    from lightop_amd import _lib
    from lightop_amd.moe import invoke_fused_moe_gemm1_silu_quant, moe_align_block_size, preshuffle_moe_weight

    say(f"fused first stage, 160-token blocks, {count} tokens on expert 0, K = {K}")
    bs, E, I = 160, 2, 256
    M = count + 3
    Aq, As, W, Ws, _, tw, _ = gemm_case(1000 + count, M, 1, E, E, 2 * I, K)
    Ws = Ws * 30  # gates where SiLU is neither 0 nor the identity
    ids = torch.ones(M, 1, dtype=torch.int32)
    ids[torch.randperm(M, generator=torch.Generator().manual_seed(count))[:count]] = 0
    rs, re, rp = oracle.moe_align_block_size(ids, bs, E)
    s, e, p = moe_align_block_size(ids.to(dev), bs, E)
    Wsh = preshuffle_moe_weight(W.to(dev))
    for mul in (False, True):
        for order, flags in (("contract", 0), ("separate", _lib.LO_GEMM_SEPARATE_ORDER)):
            with oracle.scale_order(order):
                c1 = oracle.moe_gemm_block_int8(Aq, As, W, Ws, rs, re, rp, tw, mul, 1, M, bs)
            rq, rsc = oracle.per_token_group_quant_int8(oracle.silu_and_mul(c1))
            q, sc = invoke_fused_moe_gemm1_silu_quant(Aq.to(dev), Wsh, As.to(dev), Ws.to(dev), tw.to(dev), s, e, p, mul,
                                                      1, M, {"BLOCK_SIZE_M": bs}, flags=flags)
            torch.cuda.synchronize()
            assert torch.equal(sc.cpu(), rsc), f"scales differ (mul_routed={mul}, order={order})"
            assert torch.equal(q.cpu(), rq), f"int8 activations differ (mul_routed={mul}, order={order})"


@pytest.mark.parametrize("M,k,E,Eg,I,K", [(9, 2, 4, 4, 256, 512), (400, 4, 8, 8, 384, 1152), (900, 8, 4, 16, 256, 768)])
def test_gemm1_fused_160_bit_exact_with_expert_map(dev, oracle, M, k, E, Eg, I, K):
    from lightop_amd.moe import invoke_fused_moe_gemm1_silu_quant, moe_align_block_size, preshuffle_moe_weight

    say(f"fused first stage bs=160 M={M} k={k} E={E}/{Eg} I={I} K={K}")
    bs = 160
    Aq, As, W, Ws, ids, tw, emap = gemm_case(M + I, M, k, E, Eg, 2 * I, K)
    Ws = Ws * 30
    rs, re, rp = oracle.moe_align_block_size(ids, bs, Eg, expert_map=emap)
    S = M * k
    s, e, p = moe_align_block_size(ids.to(dev), bs, Eg, None if emap is None else emap.to(dev))
    c1 = oracle.moe_gemm_block_int8(Aq, As, W, Ws, rs, re, rp, tw, False, k, S, bs)
    rq, rsc = oracle.per_token_group_quant_int8(oracle.silu_and_mul(c1))
    q, sc = invoke_fused_moe_gemm1_silu_quant(Aq.to(dev), preshuffle_moe_weight(W.to(dev)), As.to(dev), Ws.to(dev),
                                              tw.to(dev), s, e, p, False, k, S, {"BLOCK_SIZE_M": bs})
    torch.cuda.synchronize()
    local = torch.ones(S, dtype=torch.bool) if emap is None else emap.long()[ids.reshape(-1).long()] >= 0
    assert torch.equal(sc.cpu()[local], rsc[local]) and torch.equal(q.cpu()[local], rq[local])


def test_gemm1_fused_160_every_finite_bf16_gate_and_special_gates(dev, oracle):
    """Every bf16 value below 1e18 in magnitude as the gate of the 160-token form's fused epilogue, then rows with
    NaN and infinite gates next to ordinary rows (they leave the fast lookup by a wave-wide vote)."""
    from lightop_amd.moe import invoke_fused_moe_gemm1_silu_quant, moe_align_block_size, preshuffle_moe_weight

    say("fused first stage bs=160 over all bf16 gates")
    bs, I, K = 160, 128, 128
    pat = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()
    pat = pat[torch.isfinite(pat) & (pat.abs() < 1e18)]
    g = torch.Generator().manual_seed(3)
    special = torch.randn(200, generator=g) * 3
    special[5], special[70], special[71], special[150] = float("inf"), float("-inf"), float("nan"), float("-inf")
    W = torch.zeros(1, 2 * I, K, dtype=torch.int8)
    W[0, :, 0] = 1
    Wsh = preshuffle_moe_weight(W.to(dev))
    for vals in (pat, special):
        M = vals.numel()
        Aq = torch.zeros(M, K, dtype=torch.int8)
        Aq[:, 0] = 1
        As = vals.reshape(M, 1).contiguous()
        Ws = torch.ones(1, 2, 1)
        ids = torch.zeros(M, 1, dtype=torch.int32)
        tw = torch.ones(M, 1)
        rs, re, rp = oracle.moe_align_block_size(ids, bs, 1)
        c1 = oracle.moe_gemm_block_int8(Aq, As, W, Ws, rs, re, rp, tw, False, 1, M, bs)
        rq, rsc = oracle.per_token_group_quant_int8(oracle.silu_and_mul(c1))
        s, e, p = moe_align_block_size(ids.to(dev), bs, 1)
        q, sc = invoke_fused_moe_gemm1_silu_quant(Aq.to(dev), Wsh, As.to(dev), Ws.to(dev), tw.to(dev), s, e, p, False,
                                                  1, M, {"BLOCK_SIZE_M": bs})
        torch.cuda.synchronize()
        ordinary = torch.isfinite(vals)
        assert torch.equal(sc.cpu()[ordinary], rsc[ordinary]) and torch.equal(q.cpu()[ordinary], rq[ordinary])
        sp = ~ordinary
        assert ((torch.isnan(sc.cpu()[sp]) == torch.isnan(rsc[sp])) & (torch.isinf(sc.cpu()[sp]) == torch.isinf(rsc[sp]))).all()


@pytest.mark.parametrize("rows,I", [(1, 128), (7, 768), (33, 2048), (130, 256)])
@pytest.mark.parametrize("activation", ["silu", "gelu"])
def test_act_and_mul_group_quant_bit_exact(dev, oracle, rows, I, activation):
    from lightop_amd.moe import act_and_mul_group_quant

    say(f"act_and_mul_group_quant {activation} rows={rows} I={I}")
    g = torch.Generator().manual_seed(rows + I)
    c1 = (torch.randn(rows, 2 * I, generator=g) * 3).to(torch.bfloat16)
    if rows > 3:
        c1[3] = 0  # zero row: the 1e-10 floor
    n = min(c1[:, :I].numel(), 65536)
    pats = torch.arange(65536, dtype=torch.int32)[:n].to(torch.int16).view(torch.bfloat16).float()
    pats = torch.where(pats.isfinite() & (pats.abs() < 1e18), pats, torch.zeros(())).to(torch.bfloat16)
    if rows >= 33:  # every finite gate below 1e18
        c1[:32, :I] = pats[: 32 * I].reshape(32, I)
        c1[:32, I:] = (torch.rand(32, I, generator=g) * 1e-3).to(torch.bfloat16)
    act = oracle.silu_and_mul(c1) if activation == "silu" else oracle.gelu_and_mul(c1)
    rq, rs = oracle.per_token_group_quant_int8(act)
    q, s = act_and_mul_group_quant(c1.to(dev), activation)
    torch.cuda.synchronize()
    assert torch.equal(s.cpu(), rs) and torch.equal(q.cpu(), rq)


def test_act_and_mul_group_quant_row_mask_and_out(dev, oracle):
    """Rows whose mask byte is 0 are neither read (NaN there must not matter) nor written."""
    from lightop_amd.moe import act_and_mul_group_quant

    say("act_and_mul_group_quant with a row mask")
    g = torch.Generator().manual_seed(5)
    rows, I = 77, 384
    c1 = (torch.randn(rows, 2 * I, generator=g) * 3).to(torch.bfloat16)
    mask = torch.rand(rows, generator=g) > 0.4
    mask[0], mask[1] = True, False
    c1[~mask] = float("nan")
    rq, rs = oracle.per_token_group_quant_int8(oracle.silu_and_mul(torch.where(mask[:, None], c1, torch.zeros_like(c1))))
    q = torch.full((rows, I), 77, dtype=torch.int8, device=dev)
    s = torch.full((rows, I // 128), -5.0, dtype=torch.float32, device=dev)
    q2, s2 = act_and_mul_group_quant(c1.to(dev), "silu", row_mask=mask.to(dev), out=(q, s))
    torch.cuda.synchronize()
    assert q2.data_ptr() == q.data_ptr() and s2.data_ptr() == s.data_ptr()
    assert torch.equal(q.cpu()[mask], rq[mask]) and torch.equal(s.cpu()[mask], rs[mask])
    assert (q.cpu()[~mask] == 77).all() and (s.cpu()[~mask] == -5.0).all()


def _run(layer, wd, x, tw, ids, emap, dev, bs, **kw):
    from lightop_amd.moe import fused_experts_impl_int8

    w1, w2, w1s, w2s = wd
    M = x.shape[0]
    cache13 = torch.empty(M * layer.top_k * max(2 * layer.I, layer.H), dtype=torch.bfloat16, device=dev)
    out = fused_experts_impl_int8(x, w1, w2, tw, ids, cache13, use_int8_w8a8=True, global_num_experts=layer.E_global,
                                  expert_map=emap, w1_scale=w1s, w2_scale=w2s, block_shape=[128, 128],
                                  lightop_amd_block_size_m=bs, **kw)
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("M", [3, 96, 700])
@pytest.mark.parametrize("with_map", [False, True])
def test_whole_path_tiny_bit_exact(dev, oracle, M, with_map):
    from lightop_amd import workloads as wl
    from lightop_amd.moe import preshuffle_moe_weight

    layer = wl.TINY
    say(f"whole path bs=160 tiny M={M} map={with_map}")
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=0)
    x, tw, ids = wl.make_inputs(layer, M, seed=4)
    emap = None
    if with_map:
        emap = torch.full((layer.E,), -1, dtype=torch.int32)
        emap[:5] = torch.arange(5, dtype=torch.int32)
        w1, w2, w1s, w2s = (t[:5].contiguous() for t in (w1, w2, w1s, w2s))
    wd = (preshuffle_moe_weight(w1.to(dev)), preshuffle_moe_weight(w2.to(dev)), w1s.to(dev), w2s.to(dev))
    shared = (torch.randn(M, layer.H, generator=torch.Generator().manual_seed(9)) * 0.1).to(torch.bfloat16)
    for so, rsf, on_input in ((None, 1.0, False), (shared, 2.5, False), (None, 1.0, True)):
        out = _run(layer, wd, x.to(dev), tw.to(dev), ids.to(dev), None if emap is None else emap.to(dev), dev, 160,
                   shared_output=None if so is None else so.to(dev), routed_scaling_factor=rsf,
                   apply_router_weight_on_input=on_input)
        ref = oracle.fused_experts_block_int8(x, w1, w2, w1s, w2s, tw, ids, 16, global_num_experts=layer.E,
                                              expert_map=emap, shared_output=so, routed_scaling_factor=rsf,
                                              apply_router_weight_on_input=on_input)
        assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))


def test_whole_path_rejects_160_where_it_does_not_apply(dev):
    from lightop_amd import workloads as wl

    layer = wl.TINY
    w1, w2, w1s, w2s = (t.to(dev) for t in wl.make_weights(layer, seed=0))
    x, tw, ids = (t.to(dev) for t in wl.make_inputs(layer, 8, seed=0))
    with pytest.raises(RuntimeError, match="160"):  # row-major weights
        _run(layer, (w1, w2, w1s, w2s), x, tw, ids, None, dev, 160)


@pytest.mark.parametrize("name,M", [("QWEN3_30B", 2048), ("DSV3_EP", 4096)])
def test_table_picks_160_and_sampled_tokens_bit_exact(dev, oracle, name, M):
    """Where the tile table picks 160-token blocks on the two benchmark layers: the query says so, and sampled
    tokens of the default call equal the oracle's (a token's output depends on that token only)."""
    from lightop_amd import workloads as wl
    from lightop_amd.moe import get_w8a8moe_json, preshuffle_moe_weight

    layer = getattr(wl, name)
    say(f"table pick on {layer.name} at M={M}")
    c1, c2 = get_w8a8moe_json(M, layer.E, 2 * layer.I, layer.H, layer.I, True, [128, 128], layer.top_k, layer.E_global)
    assert c1["BLOCK_SIZE_M"] == 160 == c2["BLOCK_SIZE_M"] and c1["kernel_name"] == "moe_gemm_t128_kernel"
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=0, device=dev, gen_device="cuda")
    wd = (preshuffle_moe_weight(w1), preshuffle_moe_weight(w2), w1s, w2s)
    x, tw, ids = (t.to(dev) for t in wl.make_inputs(layer, M, seed=3))
    emap = wl.expert_map_for(layer, dev)
    local_tok = torch.arange(M, device=dev)
    if emap is not None:  # sample tokens that have at least one local expert
        local_tok = ((emap[ids.long()] >= 0).sum(dim=1) > 0).nonzero().flatten()
    pick = torch.randperm(local_tok.numel(), generator=torch.Generator().manual_seed(M))[:4]
    tokens = local_tok[pick.to(dev)].sort().values
    sub_ids = ids[tokens].cpu().long()
    if emap is not None:
        loc = emap.cpu()[sub_ids].long()
        used = torch.unique(loc[loc >= 0])
        remap = torch.full((layer.E_global,), -1, dtype=torch.int32)
        gl = (emap.cpu() >= 0).nonzero().flatten()
        inv = torch.full((layer.E,), -1, dtype=torch.int32)
        inv[used] = torch.arange(used.numel(), dtype=torch.int32)
        remap[gl] = inv[emap.cpu()[gl].long()]
        sel = used.to(dev)
        ref = oracle.fused_experts_block_int8(x[tokens].cpu(), w1[sel].cpu(), w2[sel].cpu(), w1s[sel].cpu(), w2s[sel].cpu(),
                                              tw[tokens].cpu(), sub_ids.to(torch.int32), 16,
                                              global_num_experts=layer.E_global, expert_map=remap)
    else:
        used = torch.unique(sub_ids)
        remap = torch.full((layer.E,), -1, dtype=torch.int64)
        remap[used] = torch.arange(used.numel())
        sel = used.to(dev)
        ref = oracle.fused_experts_block_int8(x[tokens].cpu(), w1[sel].cpu(), w2[sel].cpu(), w1s[sel].cpu(), w2s[sel].cpu(),
                                              tw[tokens].cpu(), remap[sub_ids].to(torch.int32), 16)
    out = _run(layer, wd, x, tw, ids, emap, dev, 0)
    assert torch.equal(out[tokens].cpu().view(torch.int16), ref.view(torch.int16))
    # and the explicit 128-token call gives the same rows
    out128 = _run(layer, wd, x, tw, ids, emap, dev, 128)
    assert torch.equal(out.cpu().view(torch.int16), out128.cpu().view(torch.int16))
