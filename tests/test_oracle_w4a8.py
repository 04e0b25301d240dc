"""Pins of the W4A8 (packed int4 weights, K-group scales) restatement in oracle/moe_oracle.c.

The reference implements W4A8 with per-token x per-channel scales applied once in the epilogue
(python/lightop/_lmslim_native/layers/fused_moe/w4a8.py:211-401); the K-group form of the benchmark's
int4 configuration has no reference implementation, so against the reference it is
"parity unpinned".  What is pinned here: the nibble order (the reference's, w4a8.py:341,
:375-377) by known answers, the integer part by Python integers, the scale placement by a
perturbation that must touch exactly one output element, and the fp32 part and the whole chain
by torch restatements in float64 within the block-INT8 path's tolerance."""
import pytest
import torch


def test_unpack_known_answers_and_round_trip(oracle):
    p = torch.tensor([[0x7F, 0x80, 0x19, 0xE2]], dtype=torch.uint8)
    # even k in the high nibble, odd k in the low nibble; nibbles are two's complement
    assert oracle.unpack_int4(p).tolist() == [[7, -1, -8, 0, 1, -7, -2, 2]]
    w = torch.randint(-8, 8, (3, 5, 256), dtype=torch.int8, generator=torch.Generator().manual_seed(0))
    assert torch.equal(oracle.unpack_int4(oracle.pack_int4(w)), w)
    # the reference's kernel reads the same nibbles as 16 * w: (byte << shifter) & 0xF0 as int8
    b = oracle.pack_int4(w).to(torch.int32)
    even = ((b << 0) & 0xF0).to(torch.uint8).view(torch.int8)
    odd = ((b << 4) & 0xF0).to(torch.uint8).view(torch.int8)
    assert torch.equal(even, w[..., 0::2] * 16) and torch.equal(odd, w[..., 1::2] * 16)


def _case(seed, M, k, E, N, K, bs):
    g = torch.Generator().manual_seed(seed)
    Aq = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8)
    As = torch.rand(M, K // 128, generator=g) * 0.05 + 0.005
    W = torch.randint(-8, 8, (E, N, K), generator=g, dtype=torch.int8)
    Ws = torch.exp(torch.randn(E, N, K // 128, generator=g) * 0.3 - 4.6)
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(M)]).to(torch.int32)
    tw = torch.rand(M, k, generator=g) + 0.1
    return Aq, As, W, Ws, ids, tw


def test_rowscale_gemm_integers_scales_and_torch(oracle):
    M, k, E, N, K, bs = 9, 2, 4, 48, 384, 16
    Aq, As, W, Ws, ids, tw = _case(1, M, k, E, N, K, bs)
    s, e, p = oracle.moe_align_block_size(ids, bs, E)
    W4 = oracle.pack_int4(W)
    C, acc = oracle.moe_gemm_w4a8(Aq, As, W4, Ws, s, e, p, tw, False, k, M * k, bs, dump_acc=True)
    # integer part: Python integers
    for f in (0, 7, M * k - 1):
        t, ex = f // k, int(ids[f // k, f % k])
        for n in (0, 17, N - 1):
            for kb in range(K // 128):
                a = [int(v) for v in Aq[t, kb * 128:(kb + 1) * 128]]
                w = [int(v) for v in W[ex, n, kb * 128:(kb + 1) * 128]]
                assert int(acc[f, n, kb]) == sum(x * y for x, y in zip(a, w))
    # fp32 part: float64 restatement, within one bf16 ulp
    Wd = W.double() * Ws.double().repeat_interleave(128, dim=2)
    Ad = Aq.double() * As.double().repeat_interleave(128, dim=1)
    ref = torch.stack([Ad[f // k] @ Wd[int(ids[f // k, f % k])].T for f in range(M * k)])
    assert torch.allclose(C.double(), ref, rtol=2 ** -7, atol=1e-6)
    # scale placement: changing Ws[e0, n0, kb0] changes exactly the outputs (slots of e0, column n0)
    e0, n0 = int(ids[0, 0]), 5
    Ws2 = Ws.clone()
    Ws2[e0, n0, 1] *= 3.0
    C2 = oracle.moe_gemm_w4a8(Aq, As, W4, Ws2, s, e, p, tw, False, k, M * k, bs)
    changed = (C2.view(torch.int16) != C.view(torch.int16))
    slots = (ids.reshape(-1) == e0)
    assert changed[:, n0][slots].any() and not changed[~slots].any()
    changed[:, n0] = False
    assert not changed.any()
    # router weight in the GEMM
    C3 = oracle.moe_gemm_w4a8(Aq, As, W4, Ws, s, e, p, tw, True, k, M * k, bs)
    assert torch.allclose(C3.double(), ref * tw.reshape(-1, 1).double(), rtol=2 ** -7, atol=1e-6)


@pytest.mark.parametrize("with_map", [False, True])
def test_whole_path_vs_float64_restatement(oracle, with_map):
    from lightop_amd import workloads as wl

    layer = wl.TINY_W4
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=0)
    x, tw, ids = wl.make_inputs(layer, 24, seed=2)
    emap = None
    if with_map:
        emap = torch.full((layer.E,), -1, dtype=torch.int32)
        emap[:5] = torch.arange(5, dtype=torch.int32)
    out = oracle.fused_experts_w4a8(x, w1, w2, w1s, w2s, tw, ids, 16, expert_map=emap)
    # float64 restatement of the same chain on dequantised weights
    W1 = oracle.unpack_int4(w1).double() * w1s.double().repeat_interleave(128, dim=2)
    W2 = oracle.unpack_int4(w2).double() * w2s.double().repeat_interleave(128, dim=2)
    a1q, a1s = oracle.per_token_group_quant_int8(x)
    a1 = a1q.double() * a1s.double().repeat_interleave(128, dim=1)
    ref = torch.zeros(24, layer.H, dtype=torch.float64)
    for t in range(24):
        for j in range(layer.top_k):
            e = int(ids[t, j])
            if emap is not None:
                e = int(emap[e])
                if e < 0:
                    continue
            c1 = (W1[e] @ a1[t]).float().to(torch.bfloat16)
            act = (torch.nn.functional.silu(c1[: layer.I].float()).to(torch.bfloat16).float()
                   * c1[layer.I:].float()).to(torch.bfloat16)
            a2q, a2s = oracle.per_token_group_quant_int8(act.reshape(1, -1))
            a2 = (a2q.double() * a2s.double().repeat_interleave(128, dim=1))[0]
            ref[t] += float(tw[t, j]) * (W2[e] @ a2).float().to(torch.bfloat16).double()
    err = (out.double() - ref).abs()
    assert err.max() <= 1e-2 * ref.abs().max() and err.sum() <= 6e-3 * ref.abs().sum()


# ---- the reference's own form: scales per token and per weight row, in the epilogue ----------

def test_channel_form_nibbles_factor16_known_answer(oracle):
    """w4a8.py:341, :375-377 on hand-worked bytes: byte 0x7F is 7 at even k and -1 at odd k, each
    read 16 times too large; 3 * 112 + (-2) * (-16) + 5 * (-128) + 1 * 32 = -240."""
    K, N = 128, 16
    A = torch.zeros(1, K, dtype=torch.int8)
    A[0, :4] = torch.tensor([3, -2, 5, 1], dtype=torch.int8)
    W4 = torch.zeros(1, N, K // 2, dtype=torch.uint8)
    W4[0, 0, 0], W4[0, 0, 1] = 0x7F, 0x82  # k0 = 7, k1 = -1, k2 = -8, k3 = 2
    W4[0, 3, 1] = 0x10                      # row 3: k2 = 1 only
    ids = torch.zeros(1, 1, dtype=torch.int32)
    s, e, p = oracle.moe_align_block_size(ids, 16, 1)
    C, acc = oracle.moe_gemm_w4a8_channel(A, torch.ones(1), W4, torch.ones(1, N), s, e, p, None, False, 1, 1, 16,
                                          dump_acc=True)
    assert int(acc[0, 0]) == -240 and int(acc[0, 3]) == 80 and int(acc[0, 1]) == 0
    assert C[0, 0].item() == -240.0 and C[0, 3].item() == 80.0
    # scales: 0.5 per token, 0.25 on row 3 -> exact powers of two
    Ws = torch.ones(1, N)
    Ws[0, 3] = 0.25
    C = oracle.moe_gemm_w4a8_channel(A, torch.full((1,), 0.5), W4, Ws, s, e, p, None, False, 1, 1, 16)
    assert C[0, 0].item() == -120.0 and C[0, 3].item() == 10.0


def test_channel_form_scale_order_is_left_to_right(oracle):
    """w4a8.py:386-395: ((acc * moe_weight) * a_scale) * b_scale.  Operands are searched for which another
    association rounds to another bf16 (about one draw in 10^4); the expected value is formed with numpy
    float32 operations."""
    import numpy as np

    rng = np.random.default_rng(5)
    f32 = np.float32
    n = 1 << 20
    a0, a1 = rng.integers(-127, 128, n), rng.integers(-127, 128, n)
    w0, w1 = rng.integers(-8, 8, n), rng.integers(-8, 8, n)
    d = (16 * (a0 * w0 + a1 * w1)).astype(f32)
    w = rng.uniform(0.1, 1.0, n).astype(f32)
    sa = rng.uniform(0.005, 0.05, n).astype(f32)
    sb = rng.uniform(1e-3, 1e-2, n).astype(f32)

    def bf(v):  # round to nearest even on the upper 16 bits
        u = v.astype(f32).view(np.uint32).astype(np.uint64)
        return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)

    left = bf(((d * w).astype(f32) * sa).astype(f32) * sb)
    alts = [bf((d * (w * sa).astype(f32)).astype(f32) * sb), bf((d * sa).astype(f32) * (w * sb).astype(f32)),
            bf(((d * sa).astype(f32) * sb).astype(f32) * w)]
    differs = np.zeros(n, dtype=bool)
    for alt in alts:
        differs |= alt != left
    picks = np.nonzero(differs & (d != 0))[0][:16]
    assert len(picks) >= 8
    K, N = 128, 16
    ids = torch.zeros(1, 1, dtype=torch.int32)
    s, e, p = oracle.moe_align_block_size(ids, 16, 1)
    for i in picks:
        A = torch.zeros(1, K, dtype=torch.int8)
        A[0, 0], A[0, 1] = int(a0[i]), int(a1[i])
        W4 = torch.zeros(1, N, K // 2, dtype=torch.uint8)
        W4[0, 2, 0] = ((int(w0[i]) & 15) << 4) | (int(w1[i]) & 15)
        C = oracle.moe_gemm_w4a8_channel(A, torch.tensor([float(sa[i])]), W4, torch.full((1, N), float(sb[i])), s, e, p,
                                         torch.tensor([[float(w[i])]]), True, 1, 1, 16)
        assert C[0, 2].view(torch.int16).item() == int(left[i].astype(np.int16))


def _channel_case(seed, M, k, E, N, K):
    g = torch.Generator().manual_seed(seed)
    Aq = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8)
    As = torch.rand(M, 1, generator=g) * 0.05 + 0.005
    W = torch.randint(-8, 8, (E, N, K), generator=g, dtype=torch.int8)
    Ws = torch.exp(torch.randn(E, N, 1, generator=g) * 0.3 - 7.0)
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(M)]).to(torch.int32)
    tw = torch.rand(M, k, generator=g) + 0.1
    return Aq, As, W, Ws, ids, tw


def test_channel_form_gemm_vs_float64_and_vs_int8_stage(oracle):
    M, k, E, N, K, bs = 9, 2, 4, 48, 384, 16
    Aq, As, W, Ws, ids, tw = _channel_case(3, M, k, E, N, K)
    s, e, p = oracle.moe_align_block_size(ids, bs, E)
    W4 = oracle.pack_int4(W)
    C, acc = oracle.moe_gemm_w4a8_channel(Aq, As, W4, Ws, s, e, p, tw, False, k, M * k, bs, dump_acc=True)
    # integer part: Python integers on the unpacked weights, 16 times too large
    for f in (0, 7, M * k - 1):
        t, ex = f // k, int(ids[f // k, f % k])
        for n in (0, 17, N - 1):
            assert int(acc[f, n]) == 16 * sum(int(x) * int(y) for x, y in zip(Aq[t], W[ex, n]))
    # dequantise first, in float64
    Wd = 16.0 * W.double() * Ws.double()
    Ad = Aq.double() * As.double()
    ref = torch.stack([Ad[f // k] @ Wd[int(ids[f // k, f % k])].T for f in range(M * k)])
    assert torch.allclose(C.double(), ref, rtol=2 ** -8, atol=0)
    # the int8 per-channel stage on weights multiplied out to int8: the same sums and, without
    # the routed weight, the same two multiplications -> bit for bit
    W16 = (W.to(torch.int16) * 16).to(torch.int8)
    C8, acc8 = oracle.moe_gemm_w8a8(Aq, As, W16, Ws, s, e, p, tw, False, k, M * k, bs, dump_acc=True)
    assert torch.equal(acc8, acc) and torch.equal(C8.view(torch.int16), C.view(torch.int16))
    # routed weight: first factor here, folded into the token scale there
    Cw = oracle.moe_gemm_w4a8_channel(Aq, As, W4, Ws, s, e, p, tw, True, k, M * k, bs)
    assert torch.allclose(Cw.double(), ref * tw.reshape(-1, 1).double(), rtol=2 ** -8, atol=0)
    # an expert held by another rank gives zero rows
    emap = torch.tensor([0, -1, 1, 2], dtype=torch.int32)
    s2, e2, p2 = oracle.moe_align_block_size(ids, bs, E, expert_map=emap)
    C2 = oracle.moe_gemm_w4a8_channel(Aq, As, W4[[0, 2, 3]].contiguous(), Ws[[0, 2, 3]].contiguous(), s2, e2, p2, tw,
                                      False, k, M * k, bs, out=torch.full((M * k, N), 9.0, dtype=torch.bfloat16))
    gone = ids.reshape(-1) == 1
    assert gone.any() and (C2[gone] == 0).all()
    assert torch.equal(C2[~gone].view(torch.int16), C[~gone].view(torch.int16))


@pytest.mark.parametrize("with_map", [False, True])
def test_channel_form_whole_path_vs_float64_restatement(oracle, with_map):
    from lightop_amd import workloads as wl

    layer = wl.TINY_W4_PC
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=0)
    x, tw, ids = wl.make_inputs(layer, 24, seed=2)
    emap = None
    if with_map:
        emap = torch.full((layer.E,), -1, dtype=torch.int32)
        emap[:5] = torch.arange(5, dtype=torch.int32)
    out = oracle.fused_experts_w4a8_channel(x, w1, w2, w1s, w2s, tw, ids, 16, expert_map=emap)
    W1 = 16.0 * oracle.unpack_int4(w1).double() * w1s.double()
    W2 = 16.0 * oracle.unpack_int4(w2).double() * w2s.double()
    a1q, a1s = oracle.per_token_quant_int8(x)
    a1 = a1q.double() * a1s.double()
    ref = torch.zeros(24, layer.H, dtype=torch.float64)
    for t in range(24):
        for j in range(layer.top_k):
            e = int(ids[t, j])
            if emap is not None:
                e = int(emap[e])
                if e < 0:
                    continue
            c1 = (W1[e] @ a1[t]).float().to(torch.bfloat16)
            act = (torch.nn.functional.silu(c1[: layer.I].float()).to(torch.bfloat16).float()
                   * c1[layer.I:].float()).to(torch.bfloat16)
            a2q, a2s = oracle.per_token_quant_int8(act.reshape(1, -1))
            a2 = (a2q.double() * a2s.double())[0]
            ref[t] += float(tw[t, j]) * (W2[e] @ a2).float().to(torch.bfloat16).double()
    err = (out.double() - ref).abs()
    assert ref.abs().max() > 0.1
    assert err.max() <= 1e-2 * ref.abs().max() and err.sum() <= 6e-3 * ref.abs().sum()
