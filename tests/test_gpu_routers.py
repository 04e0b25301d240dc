"""GPU parity of the two routers, through the C ABI, bit for bit against the oracle.

Sizes follow the reference's tests: test/test_softmax_topk.py (256 experts, top-8, fp16,
renormalised, 1..16384 tokens) and test/ci_tests/test_fused_moe_gate.py:242-249 (its four
routing configurations) plus DeepSeek-V3's 256 experts in 8 groups."""
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


def run_topk_softmax(x, k, renorm, idx_dtype=torch.int32, with_src=True):
    from lightop_amd.moe import topk_softmax

    T = x.shape[0]
    w = torch.empty(T, k, dtype=torch.float32, device=x.device)
    idx = torch.empty(T, k, dtype=idx_dtype, device=x.device)
    src = torch.empty(T, k, dtype=torch.int32, device=x.device) if with_src else None
    topk_softmax(w, idx, src, x, renorm)
    torch.cuda.synchronize()
    return w.cpu(), idx.cpu(), None if src is None else src.cpu()


@pytest.mark.parametrize("T", [1, 8, 64, 1000, 16384])
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32, torch.bfloat16])
@pytest.mark.parametrize("renorm", [True, False])
def test_topk_softmax_256_experts(dev, oracle, T, dtype, renorm):
    say(f"topk_softmax T={T} {dtype} renorm={renorm}")
    x = (torch.randn(T, 256, generator=torch.Generator().manual_seed(T)) * 2).to(dtype)
    w, idx, src = run_topk_softmax(x.to(dev), 8, renorm)
    rw, ridx, rsrc = oracle.topk_softmax(x, 8, renorm)
    assert torch.equal(idx, ridx) and torch.equal(src, rsrc)
    assert torch.equal(w.view(torch.int32), rw.view(torch.int32))


@pytest.mark.parametrize("E,k", [(8, 2), (60, 6), (64, 64), (100, 8), (128, 8), (384, 8), (512, 12), (1000, 16), (1024, 1)])
def test_topk_softmax_shapes_ties_and_index_types(dev, oracle, E, k):
    say(f"topk_softmax E={E} k={k}")
    g = torch.Generator().manual_seed(E)
    # coarse values: many exact ties, which the lower id must win
    x = torch.randint(-3, 4, (77, E), generator=g).float() * 0.5
    for renorm in (True, False):
        w, idx, _ = run_topk_softmax(x.to(dev), k, renorm, idx_dtype=torch.int64, with_src=False)
        rw, ridx, _ = oracle.topk_softmax(x, k, renorm)
        assert idx.dtype == torch.int64 and torch.equal(idx, ridx.long())
        assert torch.equal(w.view(torch.int32), rw.view(torch.int32))


GATE_CONFIGS = [(128, 1, 1, 7, 1), (128, 1, 1, 14, 1), (254, 2, 1, 7, 2), (254, 2, 1, 14, 2),
                (256, 8, 4, 8, 0), (192, 1, 1, 8, 0), (64, 16, 3, 6, 0), (1024, 64, 8, 32, 0)]


@pytest.mark.parametrize("E,G,tg,topk,nshare", GATE_CONFIGS)
@pytest.mark.parametrize("T", [1, 33, 4096])
def test_moe_fused_gate_vs_oracle(dev, oracle, E, G, tg, topk, nshare, T):
    from lightop_amd.moe import moe_fused_gate

    say(f"moe_fused_gate E={E} G={G} tg={tg} topk={topk} shared={nshare} T={T}")
    g = torch.Generator().manual_seed(E + T)
    x = torch.randn(T, E, generator=g)
    bias = torch.randn(E, generator=g)
    for apply, i64 in ((True, False), (False, True)):
        w, idx = moe_fused_gate(x.to(dev), bias.to(dev), G, tg, topk, nshare, 2.5, apply, i64)
        torch.cuda.synchronize()
        rw, ridx = oracle.moe_fused_gate(x, bias, G, tg, topk, nshare, 2.5, apply)
        assert idx.dtype == (torch.int64 if i64 else torch.int32)
        assert torch.equal(idx.cpu().long(), ridx.long())
        assert torch.equal(w.cpu().view(torch.int32), rw.view(torch.int32))


# From 65 rows on and up to 128 experts the gate runs with 16 lanes per row; a group's two best experts are then
# merged across the 16 / G lanes that share the group (two, four and eight lanes here; sixteen with one group,
# one lane with sixteen groups above).
GATE16_CONFIGS = [(128, 8, 4, 8, 0), (64, 4, 2, 6, 0), (96, 2, 1, 7, 1), (128, 2, 2, 8, 0), (32, 4, 3, 4, 0),
                  (128, 4, 2, 16, 0), (48, 8, 5, 6, 0)]


@pytest.mark.parametrize("E,G,tg,topk,nshare", GATE16_CONFIGS)
@pytest.mark.parametrize("T", [65, 1000, 4096])
@pytest.mark.parametrize("ties", [False, True])
def test_moe_fused_gate_16_lane_rows_merge_groups_across_lanes(dev, oracle, E, G, tg, topk, nshare, T, ties):
    from lightop_amd.moe import moe_fused_gate

    say(f"moe_fused_gate (16 lanes per row) E={E} G={G} tg={tg} topk={topk} shared={nshare} T={T} ties={ties}")
    g = torch.Generator().manual_seed(3 * E + T + G)
    if ties:  # coarse scores: equal experts inside groups and equal group scores, decided by the lower id
        x = torch.randint(-2, 3, (T, E), generator=g).float() * 0.5
        bias = torch.randint(-1, 2, (E,), generator=g).float() * 0.25
    else:
        x = torch.randn(T, E, generator=g)
        bias = torch.randn(E, generator=g)
    for apply, i64 in ((True, False), (False, True)):
        w, idx = moe_fused_gate(x.to(dev), bias.to(dev), G, tg, topk, nshare, 2.5, apply, i64)
        torch.cuda.synchronize()
        rw, ridx = oracle.moe_fused_gate(x, bias, G, tg, topk, nshare, 2.5, apply)
        assert torch.equal(idx.cpu().long(), ridx.long())
        assert torch.equal(w.cpu().view(torch.int32), rw.view(torch.int32))


def test_moe_fused_gate_16_bit_inputs_and_ties(dev, oracle):
    from lightop_amd.moe import moe_fused_gate

    g = torch.Generator().manual_seed(5)
    for dt, bt in ((torch.bfloat16, torch.float32), (torch.float16, torch.bfloat16), (torch.float32, torch.float16)):
        say(f"moe_fused_gate dtypes {dt} {bt}")
        x = torch.randint(-2, 3, (129, 256), generator=g).to(dt)      # coarse: ties everywhere
        bias = (torch.randint(-1, 2, (256,), generator=g).float() * 0.25).to(bt)
        w, idx = moe_fused_gate(x.to(dev), bias.to(dev), 8, 4, 8, 0, 2.5)
        torch.cuda.synchronize()
        rw, ridx = oracle.moe_fused_gate(x, bias, 8, 4, 8, 0, 2.5)
        assert torch.equal(idx.cpu(), ridx) and torch.equal(w.cpu().view(torch.int32), rw.view(torch.int32))


def test_routers_feed_the_path(dev, oracle):
    """Router output -> fused experts, end to end on the GPU, against the oracle fed by the oracle's router."""
    from lightop_amd import workloads as wl
    from lightop_amd.moe import fused_experts_impl_int8, moe_fused_gate

    layer = wl.TINY
    say("router -> fused experts")
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=0, device="cpu")
    g = torch.Generator().manual_seed(9)
    x = torch.randn(48, layer.H, generator=g).to(torch.bfloat16)
    logits = torch.randn(48, layer.E, generator=g)
    bias = torch.randn(layer.E, generator=g) * 0.1
    tw, ids = moe_fused_gate(logits.to(dev), bias.to(dev), 2, 1, 2, 0, 1.0)
    rtw, rids = oracle.moe_fused_gate(logits, bias, 2, 1, 2, 0, 1.0)
    cache13 = torch.empty(48 * 2 * max(2 * layer.I, layer.H), dtype=torch.bfloat16, device=dev)
    from lightop_amd import _lib

    out = fused_experts_impl_int8(x.to(dev), w1.to(dev), w2.to(dev), tw, ids, cache13, use_int8_w8a8=True,
                                  w1_scale=w1s.to(dev), w2_scale=w2s.to(dev), block_shape=[128, 128],
                                  lightop_amd_flags=0)
    torch.cuda.synchronize()
    ref = oracle.fused_experts_block_int8(x, w1, w2, w1s, w2s, rtw, rids, 16)
    assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))


def test_router_argument_errors(dev):
    from lightop_amd.moe import moe_fused_gate

    x = torch.zeros(4, 256, device=dev)
    b = torch.zeros(256, device=dev)
    for args in ((7, 4, 8, 0), (8, 9, 8, 0), (8, 1, 40, 0), (8, 4, 8, 8)):
        with pytest.raises(RuntimeError):
            moe_fused_gate(x, b, args[0], args[1], args[2], args[3], 2.5)
    with pytest.raises(RuntimeError):
        run_topk_softmax(torch.zeros(2, 16, device=dev), 17, True)
    with pytest.raises(RuntimeError):
        run_topk_softmax(torch.zeros(2, 2048, device=dev), 8, True)
