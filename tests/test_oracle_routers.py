"""Pins of the two router restatements in oracle/moe_oracle.c (CPU only).

orc_topk_softmax follows csrc/kernels/softmax/topk_softmax_kernels.cu:1381-1582 and is held to
what the reference's own test holds its kernel to (test/test_softmax_topk.py:28-66: the selected
logits are the k largest, weights within rtol 2e-5 / atol 2e-6 of torch.softmax, the source-row
formula), plus known answers for ties and closed forms.  orc_moe_fused_gate follows
csrc/kernels/moe_gate/moe_fused_gate.cu:76-312 and is held to a torch restatement of the
published grouped top-k (the algorithm of test/ci_tests/test_fused_moe_gate.py:9-61, written
here from its description) on the routing configurations that test lists, at its tolerance
(ids equal after sorting by id, weights within 1e-6), plus brute force on tiny inputs.
What no check here fixes: the last ulp of the third-party exp inside the reference kernels
(orc_expf is used instead; covered by the tolerances above) -> beyond those tolerances the
routers' weights are "parity unpinned".
"""
import itertools
import math

import pytest
import torch


def torch_grouped_topk(x, bias, G, topk_group, k_routed):
    s = torch.sigmoid(x.double()).float()
    c = s + bias
    T, E = x.shape
    group_scores = c.view(T, G, -1).topk(min(2, E // G), dim=-1)[0].sum(dim=-1)
    gidx = torch.topk(group_scores, k=topk_group, dim=-1)[1]
    gmask = torch.zeros_like(group_scores).scatter_(1, gidx, 1).bool()
    emask = gmask.unsqueeze(-1).expand(T, G, E // G).reshape(T, E)
    ids = torch.topk(c.masked_fill(~emask, float("-inf")), k=k_routed, dim=-1)[1]
    w = s.gather(1, ids)
    return w / w.sum(dim=-1, keepdim=True), ids


@pytest.mark.parametrize("T,E,k", [(1, 256, 8), (37, 128, 8), (16, 100, 6), (5, 8, 2), (9, 1000, 16), (3, 64, 64)])
@pytest.mark.parametrize("renorm", [False, True])
def test_topk_softmax_vs_torch(oracle, T, E, k, renorm):
    g = torch.Generator().manual_seed(E * 131 + k)
    x = torch.randn(T, E, generator=g) * 3.0          # continuous values: no ties
    w, idx, src = oracle.topk_softmax(x, k, renorm)
    ref_vals, ref_idx = torch.topk(x, k, dim=-1, sorted=True)
    assert torch.equal(idx.long(), ref_idx)           # descending order, same experts
    sel = x.gather(1, idx.long())
    ref_w = torch.softmax(sel, dim=-1) if renorm else torch.softmax(x, dim=-1).gather(1, idx.long())
    assert torch.allclose(w, ref_w, rtol=2e-5, atol=2e-6)
    rows = torch.arange(T)[:, None]
    ranks = torch.arange(k)[None, :]
    assert torch.equal(src.long(), ranks * T + rows)  # test_softmax_topk.py:59-64


def test_topk_softmax_known_answers(oracle):
    # all logits equal: the lowest ids win, in order; renormalised weights are 1/k up to the 1e-6 guard
    x = torch.full((2, 16), 0.25)
    w, idx, _ = oracle.topk_softmax(x, 4, True)
    assert idx.tolist() == [[0, 1, 2, 3]] * 2
    assert torch.equal(w, torch.full((2, 4), 1.0 / (4.0 + 1e-6)))
    # not renormalised: every probability is 1 / (E + 1e-6)
    w, idx, _ = oracle.topk_softmax(x, 4, False)
    assert idx.tolist() == [[0, 1, 2, 3]] * 2
    assert torch.allclose(w, torch.full((2, 4), 1.0 / 16.0), rtol=1e-6)
    # partial tie: one clear winner, then equal runners-up in id order
    x = torch.tensor([[0.0, 5.0, 1.0, 1.0, 1.0, -2.0]])
    _, idx, _ = oracle.topk_softmax(x, 3, True)
    assert idx.tolist() == [[1, 2, 3]]
    # k == E without renormalisation: the weights are the whole softmax and sum to one
    x = torch.randn(4, 70, generator=torch.Generator().manual_seed(1))
    w, idx, _ = oracle.topk_softmax(x, 64, False)
    full = torch.softmax(x, dim=-1)
    assert torch.allclose(w, full.gather(1, idx.long()), rtol=2e-5, atol=2e-6)
    # 16-bit inputs are widened exactly: same result as their fp32 image
    xh = torch.randn(3, 256, generator=torch.Generator().manual_seed(2)).to(torch.float16)
    a = oracle.topk_softmax(xh, 8, True)
    b = oracle.topk_softmax(xh.float(), 8, True)
    assert all(torch.equal(p, q) for p, q in zip(a, b))
    with pytest.raises(ValueError):
        oracle.topk_softmax(torch.zeros(1, 4), 5, True)


# (num_experts, num_expert_group, topk_group, topk, shared): the first four are the routing
# configurations of test/ci_tests/test_fused_moe_gate.py:242-249, the others DeepSeek-V3's and
# the benchmark of the same file (:294).
GATE_CONFIGS = [(128, 1, 1, 7, 1), (128, 1, 1, 14, 1), (254, 2, 1, 7, 2), (254, 2, 1, 14, 2),
                (256, 8, 4, 8, 0), (192, 1, 1, 8, 0), (64, 16, 3, 6, 0)]


@pytest.mark.parametrize("E,G,tg,topk,nshare", GATE_CONFIGS)
@pytest.mark.parametrize("T", [1, 33])
def test_fused_gate_vs_torch_restatement(oracle, E, G, tg, topk, nshare, T):
    g = torch.Generator().manual_seed(E + topk)
    x = torch.randn(T, E, generator=g)
    bias = torch.randn(E, generator=g)
    rsf = 2.5
    w, idx = oracle.moe_fused_gate(x, bias, G, tg, topk, nshare, rsf)
    kr = topk - nshare
    ref_w, ref_idx = torch_grouped_topk(x, bias, G, tg, kr)
    order, ref_order = torch.argsort(idx[:, :kr].long(), dim=-1), torch.argsort(ref_idx, dim=-1)
    assert torch.equal(idx[:, :kr].long().gather(1, order), ref_idx.gather(1, ref_order))
    assert torch.allclose(w[:, :kr].gather(1, order), (ref_w * rsf).gather(1, ref_order), rtol=1e-6, atol=1e-6)
    if nshare:
        assert torch.equal(idx[:, kr:].long(), torch.arange(E, E + nshare).expand(T, nshare))
        assert torch.allclose(w[:, kr:], torch.ones(T, nshare), rtol=1e-6, atol=1e-6)  # (sum/rsf)/sum*rsf
    # descending by choice score: the first routed expert has the largest bias + sigmoid among the kept groups
    c = torch.sigmoid(x) + bias
    sel = c.gather(1, idx[:, :kr].long())
    assert torch.all(sel[:, :-1] >= sel[:, 1:] - 1e-6)


def test_fused_gate_brute_force_and_flags(oracle):
    # two groups of two; every choice of inputs from a small grid, all of it checked by enumeration
    vals = [-1.0, 0.0, 0.5, 2.0]
    bias = torch.tensor([0.1, -0.2, 0.0, 0.3])
    for combo in itertools.product(vals, repeat=4):
        x = torch.tensor([combo])
        w, idx = oracle.moe_fused_gate(x, bias, 2, 1, 2, 0, 1.0)
        s = [1.0 / (1.0 + math.exp(-v)) for v in combo]
        c = [s[i] + float(bias[i]) for i in range(4)]
        score = [c[0] + c[1], c[2] + c[3]]
        gsel = 1 if score[1] > score[0] else 0  # a tie keeps the lower group
        members = sorted(range(2 * gsel, 2 * gsel + 2), key=lambda i: (-c[i], i))
        assert idx.tolist() == [members], (combo, idx.tolist(), members)
        tot = s[members[0]] + s[members[1]]
        assert torch.allclose(w, torch.tensor([[s[members[0]] / tot, s[members[1]] / tot]]), rtol=1e-6)
    x = torch.randn(4, 256, generator=torch.Generator().manual_seed(3))
    zb = torch.zeros(256)
    w_on, i_on = oracle.moe_fused_gate(x, zb, 8, 4, 8, 0, 2.5, True)
    w_off, i_off = oracle.moe_fused_gate(x, zb, 8, 4, 8, 0, 2.5, False)
    assert torch.equal(i_on, i_off)
    assert torch.allclose(w_on, w_off * 2.5, rtol=1e-6) and torch.allclose(w_off.sum(-1), torch.ones(4), rtol=1e-5)
    # equal scores everywhere: lowest groups, then lowest ids
    w, idx = oracle.moe_fused_gate(torch.zeros(1, 32), torch.zeros(32), 4, 2, 4, 0, 1.0)
    assert idx.tolist() == [[0, 1, 2, 3]] and torch.equal(w, torch.full((1, 4), 0.25))
    for bad in [(3, 1, 2), (4, 5, 2), (4, 1, 9)]:  # groups must divide E, topk_group <= groups, topk <= kept experts
        with pytest.raises(ValueError):
            oracle.moe_fused_gate(torch.zeros(1, 32), torch.zeros(32), bad[0], bad[1], bad[2], 0, 1.0)


def test_router_output_feeds_the_harness_routing(oracle):
    """The benchmark's DeepSeek-V3 routing (lightop_amd/workloads.py) is this gate with a zero bias."""
    from lightop_amd import workloads as wl

    layer = wl.DSV3_EP
    g = torch.Generator().manual_seed(11)
    logits = torch.randn(64, layer.E_global, generator=g)
    tw, ids = wl.route(layer, logits)
    w, idx = oracle.moe_fused_gate(logits, torch.zeros(layer.E_global), 8, 4, 8, 0, 2.5)
    o1, o2 = torch.argsort(ids.long(), dim=-1), torch.argsort(idx.long(), dim=-1)
    assert torch.equal(ids.long().gather(1, o1), idx.long().gather(1, o2))
    assert torch.allclose(tw.gather(1, o1), w.gather(1, o2), rtol=1e-5, atol=1e-6)
