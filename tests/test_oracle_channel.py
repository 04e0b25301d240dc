"""Pins of the per-channel W8A8 restatement in oracle/moe_oracle.c (per_channel_quant=True,
block_shape=None: one scale per token row and per weight row).

Pinned by: hand-worked rounding cases (ties to even, the 1e-10 floor, the zero row of the fused
activation kernel), Python integers for the whole-K sums, numpy float32 operations in the
stated order for the epilogue, a perturbation that must touch exactly one output column, and the
torch restatements the reference's own tests use: vLLM's dynamic per-token int8 quant after
SiLU-and-mul for the fused activation (test/test_fuse_silu_mul_quant.py:11-14, compared at
1e-7 there) and torch_w8a8_per_column_moe (test/moe_w8a8/fuse_moegemm_correctness.py:825-885).
Unpinned against the reference: its SiLU comes from the hardware's approximate exp2 and
reciprocal (fuse_silu_mul_quant.cu:52-66); the correctly rounded bf16 table is canonical here.
"""
import numpy as np
import pytest
import torch

from oracle import torch_ref


def bf16(v):
    return torch.tensor(v, dtype=torch.float32).to(torch.bfloat16)


def test_per_token_quant_known_answers(oracle):
    # absmax 127 makes 127/absmax exactly 1: the values themselves are rounded, ties to even
    x = bf16([[127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.49, -126.5, 0.0]])
    q, s = oracle.per_token_quant_int8(x)
    assert q.tolist() == [[127, 0, 2, 2, 0, -2, -2, 3, -126, 0]]
    assert s.shape == (1, 1) and float(s) == 1.0
    # a row of zeros takes the floor 1e-10 (int8_utils.py:37)
    q, s = oracle.per_token_quant_int8(torch.zeros(2, 16, dtype=torch.bfloat16))
    assert not q.any() and np.float32(s[0, 0]) == np.float32(1e-10) / np.float32(127)
    # one scale per row whatever the width; |q| reaches 127 exactly at the row maximum
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(7, 200, generator=g) * 3).to(torch.bfloat16)
    q, s = oracle.per_token_quant_int8(x)
    amax = x.float().abs().amax(dim=1)
    assert torch.equal(s[:, 0], amax / 127.0)
    assert torch.equal(q.abs().amax(dim=1).to(torch.int32), torch.full((7,), 127, dtype=torch.int32))
    # the rule of the reference's comparison (vLLM dynamic scaled_int8_quant): bit-equal
    q2, s2 = torch_ref.native_per_token_quant_int8(x)
    assert torch.equal(q, q2) and torch.equal(s, s2)
    # de-quantisation error at most half a step
    assert ((q.float() * s - x.float()).abs() <= 0.5 * s * (1 + 1e-6)).all()


def test_fuse_silu_mul_quant_known_answers_and_torch(oracle):
    # zero row: scale 0, multiplier 0, all zeros (fuse_silu_mul_quant.cu:112-121)
    q, s = oracle.fuse_silu_mul_quant(torch.zeros(1, 8, dtype=torch.bfloat16))
    assert not q.any() and float(s) == 0.0
    # gate 32 is its own SiLU in bf16; up = 1, 0.5, -1, 0.25 -> act = 32, 16, -32, 8; 127/32 * act
    c1 = bf16([[32.0, 32.0, 32.0, 32.0, 1.0, 0.5, -1.0, 0.25]])
    q, s, act = oracle.fuse_silu_mul_quant(c1, return_act=True)
    assert act.tolist() == [[32.0, 16.0, -32.0, 8.0]]
    assert np.float32(s[0, 0]) == np.float32(32) / np.float32(127)
    inv = np.float32(127) / np.float32(32)  # 3.96875 exactly
    assert q.tolist() == [[127, int(np.rint(np.float32(16) * inv)), -127, int(np.rint(np.float32(8) * inv))]]
    # ties: amax 127 -> multiplier 1; act 2.5 -> 2, 3.5 -> 4 (round half to even, :19-35)
    c1 = bf16([[64.0, 64.0, 64.0, 127.0 / 64, 2.5 / 64, 3.5 / 64]])
    q, s = oracle.fuse_silu_mul_quant(c1)
    assert q.tolist() == [[127, 2, 4]] and float(s) == 1.0
    # random rows against silu_and_mul followed by the per-token rule
    g = torch.Generator().manual_seed(1)
    c1 = (torch.randn(33, 2 * 192, generator=g) * 2).to(torch.bfloat16)
    q, s, act = oracle.fuse_silu_mul_quant(c1, return_act=True)
    assert torch.equal(act.view(torch.int16), oracle.silu_and_mul(c1).view(torch.int16))
    ref_act = (torch.nn.functional.silu(c1[:, :192].float()).to(torch.bfloat16).float()
               * c1[:, 192:].float()).to(torch.bfloat16)
    assert torch.equal(act.view(torch.int16), ref_act.view(torch.int16))
    amax = ref_act.float().abs().amax(dim=1, keepdim=True)
    assert torch.equal(s, amax / 127.0)
    assert torch.equal(q, torch.round(ref_act.float() * (torch.full_like(amax, 127.0) / amax)).to(torch.int8))


def _case(seed, M, k, E, N, K):
    g = torch.Generator().manual_seed(seed)
    Aq = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int8)
    As = torch.rand(M, 1, generator=g) * 0.05 + 0.005
    W = torch.randint(-128, 128, (E, N, K), generator=g, dtype=torch.int8)
    Ws = torch.randn(E, N, 1, generator=g) * 1e-2  # signed, as in the reference's test (:816-819)
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(M)]).to(torch.int32)
    tw = torch.rand(M, k, generator=g) + 0.1
    return Aq, As, W, Ws, ids, tw


def test_channel_gemm_integers_epilogue_and_torch(oracle):
    M, k, E, N, K, bs = 9, 2, 4, 48, 384, 16
    Aq, As, W, Ws, ids, tw = _case(2, M, k, E, N, K)
    s, e, p = oracle.moe_align_block_size(ids, bs, E)
    C, acc = oracle.moe_gemm_w8a8(Aq, As, W, Ws, s, e, p, None, False, k, M * k, bs, dump_acc=True)
    # whole-K integer sums: exact integer matmul
    want = torch.stack([W[int(ids[f // k, f % k])].long() @ Aq[f // k].long() for f in range(M * k)])
    assert torch.equal(acc.long(), want)
    # epilogue in the stated order with numpy float32 scalars: (f32(d) * a_s) * b_s, then bf16
    for f in (0, 5, M * k - 1):
        ex = int(ids[f // k, f % k])
        for n in (0, 17, N - 1):
            v = (np.float32(int(acc[f, n])) * np.float32(As[f // k, 0])) * np.float32(Ws[ex, n, 0])
            assert C[f, n].view(torch.int16) == torch.tensor(v).to(torch.bfloat16).view(torch.int16)
    # second stage: the routed weight joins the token scale first (moe_w8a8.cu:452, :466)
    C2 = oracle.moe_gemm_w8a8(Aq, As, W, Ws, s, e, p, tw, True, k, M * k, bs)
    for f in (1, 8):
        ex = int(ids[f // k, f % k])
        ts = np.float32(tw.reshape(-1)[f]) * np.float32(As[f // k, 0])
        v = (np.float32(int(acc[f, 3])) * ts) * np.float32(Ws[ex, 3, 0])
        assert C2[f, 3].view(torch.int16) == torch.tensor(v).to(torch.bfloat16).view(torch.int16)
    # the reference test's torch form, within one bf16 ulp
    ref = torch.stack([torch_ref.native_w8a8_per_token_matmul(Aq[f // k][None], W[int(ids[f // k, f % k])],
                                                             As[f // k][None], Ws[int(ids[f // k, f % k])])[0]
                       for f in range(M * k)])
    assert torch.allclose(C.float(), ref.float(), rtol=2 ** -7, atol=1e-6)
    # scale placement: Ws[e0, n0] touches column n0 of the slots of e0 and nothing else
    e0, n0 = int(ids[0, 0]), 5
    Ws2 = Ws.clone()
    Ws2[e0, n0] *= 3.0
    C3 = oracle.moe_gemm_w8a8(Aq, As, W, Ws2, s, e, p, None, False, k, M * k, bs)
    changed = C3.view(torch.int16) != C.view(torch.int16)
    slots = ids.reshape(-1) == e0
    assert changed[:, n0][slots].any() and not changed[~slots].any()
    changed[:, n0] = False
    assert not changed.any()
    # experts of other ranks: zero rows (moe_w8a8.cu:96-118)
    emap = torch.tensor([0, -1, 1, -1], dtype=torch.int32)
    s4, e4, p4 = oracle.moe_align_block_size(ids, bs, E, expert_map=emap)
    C4 = oracle.moe_gemm_w8a8(Aq, As, W[:2].contiguous(), Ws[:2].contiguous(), s4, e4, p4, None, False, k, M * k, bs,
                              out=torch.full((M * k, N), 7.0, dtype=torch.bfloat16))
    nonlocal_slots = emap.long()[ids.reshape(-1).long()] < 0
    assert not C4[nonlocal_slots].any() and C4[~nonlocal_slots].any()


@pytest.mark.parametrize("with_map", [False, True])
def test_whole_path_vs_reference_style_torch(oracle, with_map):
    from lightop_amd import workloads as wl

    layer = wl.TINY_PC
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=0)
    x, tw, ids = wl.make_inputs(layer, 24, seed=2)
    emap = None
    if with_map:
        emap = torch.full((layer.E,), -1, dtype=torch.int32)
        emap[:5] = torch.arange(5, dtype=torch.int32)
    r = oracle.fused_experts_channel_int8(x, w1[:5] if with_map else w1, w2[:5] if with_map else w2,
                                          w1s[:5] if with_map else w1s, w2s[:5] if with_map else w2s, tw, ids, 16,
                                          global_num_experts=layer.E, expert_map=emap, return_intermediates=True)
    # the stages chain: each intermediate is the stage function applied to the previous one
    q, s = oracle.per_token_quant_int8(x)
    assert torch.equal(r["a1q"], q) and torch.equal(r["a1s"], s)
    q2, s2 = oracle.fuse_silu_mul_quant(r["c1"])
    assert torch.equal(r["a2q"], q2) and torch.equal(r["a2s"], s2)
    ref = torch_ref.torch_w8a8_per_column_moe(x, w1, w2, w1s, w2s, tw, ids, expert_map=emap).double()
    err = (r["out"].double() - ref).abs()
    assert err.max() <= 1e-2 * ref.abs().max() and err.sum() <= 6e-3 * ref.abs().sum()
