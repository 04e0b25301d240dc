"""Pins the CPU oracle (oracle/moe_oracle.c) before anything is compared with it.

Every check here is independent of the oracle's own formulae: the reference's
docstring known answer, brute force with Python integers, closed-form special
cases, libm, and a second torch restatement with a different summation order.

Pinning status per oracle function
  orc_moe_align_block_size    pinned: docstring known answer
                              (moe_align_block_size.py:66-81), brute force, invariants.
                              The order inside an expert is the stable ascending one of
                              the reference's own Python test; the reference kernels'
                              atomics-defined order is not reproducible: parity unpinned
                              for that order (their test compares sorted multisets).
  orc_group_quant_int8        pinned: exact power-of-two cases, truncation cases, zeros.
  orc_moe_gemm_block_int8     int32 part pinned by Python-integer brute force; fp32 part
                              pinned by closed-form cases and the torch restatement.
  orc_expf / orc_silu_and_mul pinned against libm expf over all 65536 bf16 inputs.
  orc_moe_sum                 pinned: k=1 identity, torch.sum, hand-worked roundings.
  orc_*_f32 (fp32 rows)       pinned: hand-worked quantisation and reduce cases, the bf16
                              functions' results after one rounding, float64 torch.
  orc_fused_experts_block_int8 pinned against the torch restatement within the path's
                              tolerance (the reference holds no end-to-end assertion
                              for the block-INT8 path).
"""
import math

import numpy as np
import pytest
import torch

from oracle import torch_ref


def bf16(vals):
    return torch.tensor(vals, dtype=torch.float32).to(torch.bfloat16)


# ------------------------------------------------------------------ alignment --

def test_align_reference_docstring_example(oracle):
    # moe_align_block_size.py:66-81: experts 1..4 are used, so five experts with expert 0 empty
    ids = torch.tensor([[2, 3, 4], [1, 2, 4], [1, 3, 4], [1, 2, 3]], dtype=torch.int32)
    s, e, p = oracle.moe_align_block_size(ids, 4, 5)
    assert p.item() == 16
    assert s[:16].tolist() == [3, 6, 9, 12, 0, 4, 10, 12, 1, 7, 11, 12, 2, 5, 8, 12]
    assert e[:4].tolist() == [1, 2, 3, 4]
    assert s[16:].tolist() == [12] * (s.numel() - 16)


def brute_align(ids, E, bs, emap=None, ignore=False):
    """Plain Python, list based; independent of the C code."""
    S = len(ids)
    buckets = [[] for _ in range(E)]
    for f, e in enumerate(ids):
        if ignore and emap is not None:
            e = emap[e]
            if e < 0:
                continue
        buckets[e].append(f)
    out, eids = [], []
    for e, b in enumerate(buckets):
        nb = -(-len(b) // bs)
        out += b + [S] * (nb * bs - len(b))
        eids += [(emap[e] if (emap is not None and not ignore) else e)] * nb
    return out, eids


@pytest.mark.parametrize("S,E,bs", [(1, 8, 16), (7, 4, 4), (64, 8, 16), (300, 256, 16), (1000, 33, 32),
                                    (4096, 128, 64), (513, 5, 128)])
def test_align_vs_brute_force(oracle, S, E, bs):
    g = torch.Generator().manual_seed(S * 31 + E)
    ids = torch.randint(0, E, (S,), generator=g, dtype=torch.int32)
    s, e, p = oracle.moe_align_block_size(ids, bs, E)
    ref_s, ref_e = brute_align(ids.tolist(), E, bs)
    assert p.item() == len(ref_s)
    assert s[: len(ref_s)].tolist() == ref_s
    assert e[: len(ref_e)].tolist() == ref_e
    assert (s[len(ref_s):] == S).all() and (e[len(ref_e):] == -1).all()
    # invariants: every slot exactly once, blocks are single-expert
    valid = s[s < S]
    assert sorted(valid.tolist()) == list(range(S))
    blocks = s[: p.item()].view(-1, bs)
    for b in range(blocks.shape[0]):
        row = blocks[b][blocks[b] < S]
        assert (ids[row.long()] == e[b]).all()


def test_align_expert_map_modes(oracle):
    g = torch.Generator().manual_seed(5)
    E = 16
    ids = torch.randint(0, E, (200,), generator=g, dtype=torch.int32)
    emap = torch.full((E,), -1, dtype=torch.int32)
    emap[4:8] = torch.arange(4, dtype=torch.int32)
    for ignore in (False, True):
        s, e, p = oracle.moe_align_block_size(ids, 16, E, expert_map=emap, ignore_invalid_experts=ignore)
        ref_s, ref_e = brute_align(ids.tolist(), E, 16, emap.tolist(), ignore)
        assert p.item() == len(ref_s)
        assert s[: len(ref_s)].tolist() == ref_s and e[: len(ref_e)].tolist() == ref_e
    # buffer sizing rule when there are fewer slots than experts
    s, e, p = oracle.moe_align_block_size(torch.tensor([3, 1], dtype=torch.int32), 16, 64)
    assert s.numel() == 32 and e.numel() == 2 and p.item() == 32


def test_align_rejects_bad_ids(oracle):
    with pytest.raises(RuntimeError):
        oracle.moe_align_block_size(torch.tensor([0, 9], dtype=torch.int32), 16, 8)


# ---------------------------------------------------------------- group quant --

def test_quant_exact_powers_of_two(oracle):
    # x = i * 2^k with amax = 127 * 2^k  ->  s = 2^k exactly, q = i exactly
    for k in (-6, 0, 3):
        vals = [float(i) * 2.0 ** k for i in range(-127, 1)]  # 128 values, amax 127*2^k
        q, s = oracle.per_token_group_quant_int8(bf16([vals]))
        assert s.item() == 2.0 ** k
        assert q[0].tolist() == list(range(-127, 1))


def test_quant_truncates_toward_zero(oracle):
    # amax 127 -> s = 1; 1.5 -> 1 (round would give 2), -1.5 -> -1 (floor would give -2), 2.5 -> 2
    row = [127.0, 1.5, -1.5, 2.5, -2.5, 0.75, -0.75, 126.5] + [0.0] * 120
    q, s = oracle.per_token_group_quant_int8(bf16([row]))
    assert s.item() == 1.0
    assert q[0, :8].tolist() == [127, 1, -1, 2, -2, 0, 0, 126]


def test_quant_zero_group_and_single_value(oracle):
    q, s = oracle.per_token_group_quant_int8(torch.zeros(1, 256, dtype=torch.bfloat16))
    assert (q == 0).all()
    assert s.flatten().tolist() == [np.float32(1e-10) / np.float32(127.0)] * 2
    # one non-zero value: q is 127 or 126 exactly as IEEE division says
    for v in (0.3, 1.7, 3.1415, 1000.0, 2.0 ** -20):
        x = torch.zeros(1, 128, dtype=torch.bfloat16)
        x[0, 5] = -v
        xv = np.float32(x[0, 5].float().item())
        q, s = oracle.per_token_group_quant_int8(x)
        sc = np.float32(abs(xv)) / np.float32(127.0)
        assert s.item() == sc
        assert q[0, 5].item() == int(np.trunc(max(np.float32(xv) / sc, np.float32(-128.0))))
        assert q[0, 5].item() in (-127, -126)


def test_quant_matches_torch_restatement(oracle):
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(37, 1024, generator=g) * 3).to(torch.bfloat16)
    q, s = oracle.per_token_group_quant_int8(x)
    q2, s2 = torch_ref.native_per_token_group_quant_int8(x)
    assert torch.equal(s, s2) and torch.equal(q, q2)


# ------------------------------------------------------------------- GEMM -----

def _small_gemm_case(seed, S_tok, k, E, N, K, bs, scales_one=False, emap=None, lo=-127, hi=128):
    g = torch.Generator().manual_seed(seed)
    Aq = torch.randint(lo, hi, (S_tok, K), generator=g, dtype=torch.int8)
    As = torch.ones(S_tok, K // 128) if scales_one else torch.rand(S_tok, K // 128, generator=g) * 0.1 + 0.01
    W = torch.randint(lo, hi, (E, N, K), generator=g, dtype=torch.int8)
    Ws = torch.ones(E, (N + 127) // 128, K // 128) if scales_one else \
        torch.exp(torch.randn(E, (N + 127) // 128, K // 128, generator=g) * 0.3 + math.log(1e-3))
    Eg = E if emap is None else emap.numel()
    ids = torch.randint(0, Eg, (S_tok, k), generator=g, dtype=torch.int32)
    tw = torch.rand(S_tok, k, generator=g)
    return Aq, As, W, Ws, ids, tw, Eg


def test_gemm_int32_exact_vs_python_integers(oracle):
    Aq, As, W, Ws, ids, tw, Eg = _small_gemm_case(3, 5, 2, 3, 32, 256, 16, scales_one=True)
    s, e, p = oracle.moe_align_block_size(ids, 16, Eg)
    C, acc = oracle.moe_gemm_block_int8(Aq, As, W, Ws, s, e, p, None, False, 2, 10, 16, dump_acc=True)
    A64, W64 = Aq.numpy().astype(np.int64), W.numpy().astype(np.int64)
    flat = ids.reshape(-1).tolist()
    for f in range(10):
        for n in range(32):
            for kb in range(2):
                d = int((A64[f // 2, kb * 128:(kb + 1) * 128] * W64[flat[f], n, kb * 128:(kb + 1) * 128]).sum())
                assert acc[f, n, kb].item() == d
            # scales of one: the bf16 output is the rounded exact integer sum
            tot = float(acc[f, n].sum().item())
            assert C[f, n].item() == torch.tensor(tot).to(torch.bfloat16).item()


def test_gemm_scale_order_and_router_weight(oracle):
    # the order without fp fusion: one token, one expert, K=256: acc = (d0*as0)*ws0 + (d1*as1)*ws1, then * w, then bf16
    Aq = torch.zeros(1, 256, dtype=torch.int8); Aq[0, 0] = 100; Aq[0, 128] = -7
    W = torch.zeros(1, 16, 256, dtype=torch.int8); W[0, :, 0] = 3; W[0, :, 128] = 11
    As = torch.tensor([[0.37, 1.9]]); Ws = torch.tensor([[[0.0123, 0.5]]])
    ids = torch.zeros(1, 1, dtype=torch.int32); tw = torch.tensor([[0.731]])
    s, e, p = oracle.moe_align_block_size(ids, 16, 1)
    with oracle.scale_order("separate"):
        C = oracle.moe_gemm_block_int8(Aq, As, W, Ws, s, e, p, tw, True, 1, 1, 16)
    f = np.float32
    acc = f(0) + (f(300) * f(0.37)) * f(0.0123)
    acc = acc + (f(-77) * f(1.9)) * f(0.5)
    acc = acc * f(0.731)
    assert C[0, 0].item() == torch.tensor(float(acc)).to(torch.bfloat16).item()
    assert (C[0] == C[0, 0]).all()


def _round_to_f32(q):
    """The float32 nearest to the rational q, ties to even: exact integer arithmetic, no float operation decides."""
    from fractions import Fraction

    if q == 0:
        return np.float32(0.0)
    c = np.float32(float(q))  # a float32 within an ulp or two of q; the neighbours are compared exactly
    cands = [c, np.nextafter(c, np.float32(np.inf)), np.nextafter(c, np.float32(-np.inf))]
    cands += [np.nextafter(cands[1], np.float32(np.inf)), np.nextafter(cands[2], np.float32(-np.inf))]
    best = min(cands, key=lambda v: (abs(Fraction(float(v)) - q), int(np.float32(v).view(np.uint32)) & 1))
    return np.float32(best)


def test_gemm_contracted_order_hand_worked(oracle):
    """The default order, acc = fma(f32(d) * a_s, b_s, acc): the product f32(d) * a_s is rounded, the second
    product and the sum are rounded once, together.  Expected values from exact rational arithmetic; the
    sixteen rows carry different sums, the fp32 output shows every rounding, and the two orders must differ
    on some row, so that taking one for the other fails here."""
    from fractions import Fraction

    Aq = torch.zeros(1, 384, dtype=torch.int8); Aq[0, 0] = 100; Aq[0, 128] = -7; Aq[0, 256] = 53
    W = torch.zeros(1, 16, 384, dtype=torch.int8)
    for n in range(16):
        W[0, n, 0] = 3 + 7 * n; W[0, n, 128] = 11 - 5 * n; W[0, n, 256] = 9 * n - 60
    As = torch.tensor([[0.37, 1.9, 0.0421]]); Ws = torch.tensor([[[0.0123, 0.5003, 0.00917]]])
    ids = torch.zeros(1, 1, dtype=torch.int32); tw = torch.tensor([[0.731]])
    s, e, p = oracle.moe_align_block_size(ids, 16, 1)
    f = np.float32
    want_c, want_s = [], []
    for n in range(16):
        d = [100 * (3 + 7 * n), -7 * (11 - 5 * n), 53 * (9 * n - 60)]
        acc_c, acc_s = f(0), f(0)
        for kb in range(3):
            t = f(d[kb]) * f(As[0, kb].item())                      # rounded on its own in both orders
            b = f(Ws[0, 0, kb].item())
            acc_c = _round_to_f32(Fraction(float(t)) * Fraction(float(b)) + Fraction(float(acc_c)))
            acc_s = acc_s + t * b                                   # numpy float32: every operation rounded
        want_c.append(acc_c); want_s.append(acc_s)
    assert any(a != b for a, b in zip(want_c, want_s)), "the case no longer tells the orders apart"
    for order, want in (("contract", want_c), ("separate", want_s)):
        with oracle.scale_order(order):
            Cf = oracle.moe_gemm_block_int8(Aq, As, W, Ws, s, e, p, None, False, 1, 1, 16,
                                            out=torch.zeros(1, 16, dtype=torch.float32))
            Cw = oracle.moe_gemm_block_int8(Aq, As, W, Ws, s, e, p, tw, True, 1, 1, 16)
        assert Cf[0].tolist() == [float(v) for v in want], order
        assert Cw[0].tolist() == [torch.tensor(float(v * f(0.731))).to(torch.bfloat16).item() for v in want], order
    # the default is the contracted order
    Cd = oracle.moe_gemm_block_int8(Aq, As, W, Ws, s, e, p, None, False, 1, 1, 16, out=torch.zeros(1, 16, dtype=torch.float32))
    assert Cd[0].tolist() == [float(v) for v in want_c]


def test_gemm_scale_orders_differ_in_bf16_somewhere(oracle):
    """On a few thousand random sums the two orders give different bf16 outputs now and then (and never by more
    than one bf16 ulp): a kernel test that compares bf16 rows can therefore tell them apart."""
    Aq, As, W, Ws, ids, tw, Eg = _small_gemm_case(21, 64, 2, 2, 256, 1024, 16)
    s, e, p = oracle.moe_align_block_size(ids, 16, Eg)
    with oracle.scale_order("contract"):
        Cc = oracle.moe_gemm_block_int8(Aq, As, W, Ws, s, e, p, None, False, 2, 128, 16)
    with oracle.scale_order("separate"):
        Cs = oracle.moe_gemm_block_int8(Aq, As, W, Ws, s, e, p, None, False, 2, 128, 16)
    diff = (Cc.view(torch.int16) != Cs.view(torch.int16))
    assert 0 < diff.sum().item() < 0.05 * diff.numel()
    assert ((Cc.view(torch.int16).int() - Cs.view(torch.int16).int()).abs() <= 1).all()


def test_gemm_vs_torch_restatement_and_skipped_experts(oracle):
    emap = torch.tensor([0, -1, 1, -1], dtype=torch.int32)
    Aq, As, W, Ws, ids, tw, Eg = _small_gemm_case(7, 24, 2, 2, 256, 384, 16, emap=emap)
    s, e, p = oracle.moe_align_block_size(ids, 16, Eg, expert_map=emap)
    C = oracle.moe_gemm_block_int8(Aq, As, W, Ws, s, e, p, None, False, 2, 48, 16)
    flat = emap.long()[ids.reshape(-1).long()]
    for f in range(48):
        if flat[f] < 0:
            assert (C[f] == 0).all()
            continue
        ref = torch_ref.native_w8a8_block_int8_matmul(Aq[f // 2:f // 2 + 1], W[flat[f]], As[f // 2:f // 2 + 1],
                                                      Ws[flat[f]], output_dtype=torch.float32)
        got = C[f].float()
        # bf16 of two fp32 sums that differ only in rounding order: equal up to one bf16 ulp
        assert torch.allclose(got, ref[0], rtol=2 ** -7, atol=1e-6)
        assert (got - ref[0]).abs().mean() <= 2 ** -8 * ref[0].abs().mean()


# --------------------------------------------------------------- SiLU * mul ----

def test_expf_vs_libm(oracle):
    lib = oracle.lib()
    xs = np.concatenate([np.linspace(-87, 88.7, 200001, dtype=np.float32),
                         np.random.default_rng(0).normal(0, 4, 100000).astype(np.float32)])
    worst = 0.0
    for x in xs[::7]:
        got = lib.orc_expf(float(x))
        ref = math.exp(float(x))
        ulp = np.spacing(np.float32(ref))
        worst = max(worst, abs(got - ref) / float(ulp))
    assert worst <= 1.0, worst


def test_silu_equals_libm_silu_on_every_bf16(oracle):
    lib = oracle.lib()
    bad = []
    for h in range(65536):
        e = (h >> 7) & 0xFF
        if e == 0xFF:  # inf / nan
            continue
        if lib.orc_silu_bf16(h) != lib.orc_silu_bf16_libm(h):
            bad.append(h)
    assert not bad, f"{len(bad)} bf16 inputs differ from the libm-based SiLU, e.g. {bad[:8]}"


def test_silu_and_mul_vs_torch(oracle):
    g = torch.Generator().manual_seed(2)
    c1 = (torch.randn(64, 512, generator=g) * 4).to(torch.bfloat16)
    act = oracle.silu_and_mul(c1)
    ref = torch.nn.functional.silu(c1[:, :256].float()).to(torch.bfloat16).float() * c1[:, 256:].float()
    # the reference's own bar for this op is rtol = atol = 1e-2 (test/ci_tests/test_fuse_silu_mul.py:31-33)
    assert torch.allclose(act.float(), ref, rtol=1e-2, atol=1e-2)
    # and bit-for-bit against torch's own bf16 rounding of the same two-step formula
    assert (act == ref.to(torch.bfloat16)).float().mean() > 0.999
    # gate is the first half: silu(0) * u == 0, silu(large) ~ g
    z = torch.zeros(1, 256, dtype=torch.bfloat16); z[0, 128:] = 3.0
    assert (oracle.silu_and_mul(z) == 0).all()


def test_gelu_table_pins(oracle):
    """orc_gelu_bf16 (activation_kernels_opt.cu:234-242): closed forms, torch's erf GELU on every finite
    bf16 input, the identity gelu(x) - gelu(-x) = x, monotone above the minimum near -0.75."""
    tab = oracle.gelu_bf16_table().view(torch.bfloat16)
    pats = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    x = pats.float()
    finite = x.isfinite()
    # closed forms
    assert tab[0].item() == 0.0 and tab[0x8000].item() == 0.0      # gelu(+-0) = +-0 * 0.5 * 1
    big = finite & (x >= 6.0)
    assert torch.equal(tab[big].view(torch.int16), pats[big].view(torch.int16))  # erf = 1: gelu(x) = x
    neg = finite & (x <= -6.0)
    assert (tab[neg].float() == 0.0).all()                         # 1 + erf = 0: -0
    assert tab[0x7F80].item() == float("inf") and tab[0x7FC0].isnan()
    # torch's GELU (erf form) in float64, rounded once: within one bf16 ulp everywhere
    ref = torch.nn.functional.gelu(x[finite].double()).float()
    got = tab[finite].float()
    ulp = torch.maximum((ref.abs() * 2.0 ** -7), torch.full_like(ref, 2.0 ** -133))
    # far down the negative tail the formula's own 1 + erf cancels in fp32 (erf within 2^-24 of -1): the
    # result is then off by up to |x| / 2 * 2^-24 from the true GELU, which is what the reference computes too
    xf = x[finite]
    tail = xf * -0.5 * 2.0 ** -24
    assert ((got - ref).abs() <= torch.where(xf < -4.8, ulp + tail, ulp)).all()
    assert ((got - ref).abs() <= ulp)[xf >= -4.8].all()
    # equal to the float64 value rounded to bf16 on all but a sliver of inputs (double rounding)
    assert (got.to(torch.bfloat16) == ref.to(torch.bfloat16)).float().mean() > 0.995
    # odd part: gelu(x) - gelu(-x) = x
    mag = pats[:0x7F80]
    odd = tab[:0x7F80].float() - tab[0x8000:0x8000 + 0x7F80].float()
    assert ((odd - mag.float()).abs() <= mag.float().abs() * 2.0 ** -7 + 1e-38).all()
    # monotone non-decreasing for x >= -0.75 (the minimum of GELU lies at about -0.7518)
    order = x[finite].argsort()
    xs, ys = x[finite][order], tab[finite][order].float()
    keep = xs >= -0.75
    assert (ys[keep][1:] >= ys[keep][:-1]).all()


def test_gelu_and_mul_vs_torch(oracle):
    g = torch.Generator().manual_seed(5)
    c1 = (torch.randn(64, 512, generator=g) * 3).to(torch.bfloat16)
    act = oracle.gelu_and_mul(c1)
    ref = torch.nn.functional.gelu(c1[:, :256].float()).to(torch.bfloat16).float() * c1[:, 256:].float()
    assert torch.allclose(act.float(), ref, rtol=1e-2, atol=1e-2)
    # bit for bit against torch's own rounding of the same two-step formula, except below about -3.5 where
    # 1 + erf cancels in fp32 and the last place of the erf routine shows (torch's is not correctly rounded)
    body = c1[:, :256].float() > -3.5
    assert (act == ref.to(torch.bfloat16))[body].float().mean() > 0.999
    # gate is the first half
    z = torch.zeros(1, 256, dtype=torch.bfloat16); z[0, 128:] = 3.0
    assert (oracle.gelu_and_mul(z) == 0).all()
    z[0, :128] = 8.0
    assert (oracle.gelu_and_mul(z) == 24.0).all()


@pytest.mark.parametrize("form", ["block", "channel"])
def test_whole_path_gelu_vs_float64_restatement(oracle, form):
    """The gelu branch of the chains (int8.py:825-838): a float64 restatement on dequantised weights."""
    from lightop_amd import workloads as wl

    layer = wl.TINY if form == "block" else wl.TINY_PC
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=0)
    M = 12
    x, tw, ids = wl.make_inputs(layer, M, seed=2)
    if form == "block":
        out = oracle.fused_experts_block_int8(x, w1, w2, w1s, w2s, tw, ids, 16, activation="gelu")
        W1 = w1.double() * w1s.double().repeat_interleave(128, 1).repeat_interleave(128, 2)
        W2 = w2.double() * w2s.double().repeat_interleave(128, 1).repeat_interleave(128, 2)
        a1q, a1s = oracle.per_token_group_quant_int8(x)
        a1 = a1q.double() * a1s.double().repeat_interleave(128, dim=1)
    else:
        out = oracle.fused_experts_channel_int8(x, w1, w2, w1s, w2s, tw, ids, 16, activation="gelu")
        W1, W2 = w1.double() * w1s.double(), w2.double() * w2s.double()
        a1q, a1s = oracle.per_token_quant_int8(x)
        a1 = a1q.double() * a1s.double()
    silu_out = (oracle.fused_experts_block_int8 if form == "block" else oracle.fused_experts_channel_int8)(
        x, w1, w2, w1s, w2s, tw, ids, 16)
    assert not torch.equal(out, silu_out)
    ref = torch.zeros(M, layer.H, dtype=torch.float64)
    for t in range(M):
        for j in range(layer.top_k):
            e = int(ids[t, j])
            c1 = (W1[e] @ a1[t]).float().to(torch.bfloat16)
            act = (torch.nn.functional.gelu(c1[: layer.I].float()).to(torch.bfloat16).float()
                   * c1[layer.I:].float()).to(torch.bfloat16)
            if form == "block":
                a2q, a2s = oracle.per_token_group_quant_int8(act.reshape(1, -1))
                a2 = (a2q.double() * a2s.double().repeat_interleave(128, dim=1))[0]
            else:
                a2q, a2s = oracle.per_token_quant_int8(act.reshape(1, -1))
                a2 = (a2q.double() * a2s.double())[0]
            ref[t] += float(tw[t, j]) * (W2[e] @ a2).float().to(torch.bfloat16).double()
    err = (out.double() - ref).abs()
    assert ref.abs().max() > 0.05
    assert err.max() <= 1e-2 * ref.abs().max() and err.sum() <= 6e-3 * ref.abs().sum()


def test_half_conversions_vs_torch(oracle):
    """The oracle's binary16 conversions (used when the activations are float16) against torch's: every
    half pattern, and every float that is a half, lies next to one, or lies on or next to the midpoint of
    two neighbouring halves (the rounding boundaries), plus the overflow and underflow edges."""
    import ctypes

    import numpy as np

    lib = oracle.lib()
    lib.orc_f16_to_f32.restype = ctypes.c_float
    lib.orc_f16_to_f32.argtypes = [ctypes.c_uint16]
    lib.orc_f32_to_f16.restype = ctypes.c_uint16
    lib.orc_f32_to_f16.argtypes = [ctypes.c_float]
    h = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.float16)
    ref = h.float()
    got = torch.tensor([lib.orc_f16_to_f32(i) for i in range(65536)])
    assert ((got.view(torch.int32) == ref.view(torch.int32)) | (got.isnan() & ref.isnan())).all()
    fin = ref[ref.isfinite()].sort().values
    mids = ((fin.double()[:-1] + fin.double()[1:]) / 2).float()
    cands = [(t.view(torch.int32) + d).view(torch.float32) for t in (fin, mids) for d in (-1, 0, 1)]
    cands.append(torch.tensor([65504.0, 65519.996, 65520.0, 65536.0, 1e10, -1e10, float("inf"), -float("inf"),
                               2.0 ** -25, 2.0 ** -25 * 1.0000001, 2.0 ** -24, 2.0 ** -26, 0.0, -0.0]))
    c = torch.cat(cands)
    c = c[~c.isnan()]
    want = c.half().view(torch.int16).numpy().astype(np.uint16)
    have = np.array([lib.orc_f32_to_f16(float(v)) for v in c.tolist()], dtype=np.uint16)
    assert (have == want).all()
    assert lib.orc_f32_to_f16(float("nan")) & 0x7C00 == 0x7C00 and lib.orc_f32_to_f16(float("nan")) & 0x3FF


@pytest.mark.parametrize("form", ["block", "channel"])
@pytest.mark.parametrize("activation", ["silu", "gelu"])
def test_whole_path_float16_vs_float64_restatement(oracle, form, activation):
    """float16 activations (int8.py:689-696): the same chains with every stored value rounded to half."""
    from lightop_amd import workloads as wl

    layer = wl.TINY if form == "block" else wl.TINY_PC
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=0)
    M = 12
    x, tw, ids = wl.make_inputs(layer, M, seed=2)
    xh = x.to(torch.float16)
    fn = oracle.fused_experts_block_int8 if form == "block" else oracle.fused_experts_channel_int8
    out = fn(xh, w1, w2, w1s, w2s, tw, ids, 16, activation=activation)
    assert out.dtype == torch.float16
    assert not torch.equal(out.float(), fn(xh.to(torch.bfloat16), w1, w2, w1s, w2s, tw, ids, 16, activation=activation).float())
    if form == "block":
        W1 = w1.double() * w1s.double().repeat_interleave(128, 1).repeat_interleave(128, 2)
        W2 = w2.double() * w2s.double().repeat_interleave(128, 1).repeat_interleave(128, 2)
        a1q, a1s = oracle.per_token_group_quant_int8(xh)
        a1 = a1q.double() * a1s.double().repeat_interleave(128, dim=1)
    else:
        W1, W2 = w1.double() * w1s.double(), w2.double() * w2s.double()
        a1q, a1s = oracle.per_token_quant_int8(xh)
        a1 = a1q.double() * a1s.double()
    actf = torch.nn.functional.silu if activation == "silu" else torch.nn.functional.gelu
    ref = torch.zeros(M, layer.H, dtype=torch.float64)
    for t in range(M):
        for j in range(layer.top_k):
            e = int(ids[t, j])
            c1 = (W1[e] @ a1[t]).float().to(torch.float16)
            act = (actf(c1[: layer.I].float()).to(torch.float16).float() * c1[layer.I:].float()).to(torch.float16)
            if form == "block":
                a2q, a2s = oracle.per_token_group_quant_int8(act.reshape(1, -1))
                a2 = (a2q.double() * a2s.double().repeat_interleave(128, dim=1))[0]
            else:
                a2q, a2s = oracle.per_token_quant_int8(act.reshape(1, -1))
                a2 = (a2q.double() * a2s.double())[0]
            ref[t] += float(tw[t, j]) * (W2[e] @ a2).float().to(torch.float16).double()
    err = (out.double() - ref).abs()
    assert ref.abs().max() > 0.05
    # half keeps three more mantissa bits than bf16: the tolerance of the path with room to spare
    assert err.max() <= 1e-2 * ref.abs().max() and err.sum() <= 6e-3 * ref.abs().sum()


# ------------------------------------------------------------------ moe_sum ----

def test_moe_sum_cases(oracle):
    g = torch.Generator().manual_seed(3)
    x = torch.randn(9, 1, 64, generator=g).to(torch.bfloat16)
    assert torch.equal(oracle.moe_sum(x), x[:, 0])                      # k = 1, factor 1: identity
    x = torch.randn(9, 8, 64, generator=g).to(torch.bfloat16)
    seq = torch.zeros(9, 64)
    for j in range(8):                                                  # IEEE fp32 adds in slot order,
        seq = seq + x[:, j].float()
    assert torch.equal(oracle.moe_sum(x), seq.to(torch.bfloat16))       # one rounding at the end
    # the order matters: ((2^24 + 1) - 2^24) + 1 = 1 in fp32 slot order; a pairwise or reversed sum gives 0 or 2
    v = bf16([[[2.0 ** 24], [1.0], [-(2.0 ** 24)], [1.0]]])
    assert oracle.moe_sum(v).float().item() == 1.0
    # the accumulator is fp32, not bf16: 1 + 2^-8 + 2^-8 = 1 + 2^-7 exactly (a bf16 accumulator stays at 1)
    v = bf16([[[1.0], [2.0 ** -8], [2.0 ** -8]]])
    assert oracle.moe_sum(v).float().item() == 1.0 + 2.0 ** -7
    # one rounding, to nearest even: 1 + 2^-9 + 2^-9 = 1 + 2^-8 lies halfway between 1 and 1 + 2^-7 -> 1
    v = bf16([[[1.0], [2.0 ** -9], [2.0 ** -9]]])
    assert oracle.moe_sum(v).float().item() == 1.0
    # ... and 1 + 2^-7 + 2^-8 lies halfway between 1 + 2^-7 (odd) and 1 + 2^-6 (even) -> up
    assert oracle.moe_sum(bf16([[[1.0 + 2.0 ** -7], [2.0 ** -8]]])).float().item() == 1.0 + 2.0 ** -6
    v = bf16([[[1.0], [2.0 ** -9], [2.0 ** -9]]])
    f = np.float32
    acc = (f(0) + f(1.0)) + f(2.0 ** -9) + f(2.0 ** -9)
    assert oracle.moe_sum(v, factor=2.5).float().item() == torch.tensor(float(acc * f(2.5))).to(torch.bfloat16).item()
    # with bias: three roundings
    b = bf16([[0.00390625]])
    xr = torch.tensor(float(acc)).to(torch.bfloat16).float()
    xr = (xr * 2.5).to(torch.bfloat16).float()
    xr = (xr + b.float()).to(torch.bfloat16)
    assert oracle.moe_sum(v, bias=b, factor=2.5).item() == xr.item()


# ------------------------------------------------------------- whole path -----

def test_fused_path_vs_torch_restatement(oracle):
    from lightop_amd import workloads as wl

    layer = wl.MoeLayer("t", E=4, E_global=4, top_k=2, H=256, I=128, routing="softmax")
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=0)
    x, tw, ids = wl.make_inputs(layer, 33, seed=0)
    out = oracle.fused_experts_block_int8(x, w1, w2, w1s, w2s, tw, ids, 16)
    ref = torch_ref.torch_w8a8_block_int8_moe(x, w1, w2, w1s, w2s, tw, ids)
    err = (out.float() - ref.float()).abs()
    assert err.max() <= 1e-2 * ref.float().abs().max()
    assert (err.sum() / ref.float().abs().sum()) <= 2e-3 * 3  # two bf16 roundings apart


def test_fused_path_expert_parallel_share(oracle):
    from lightop_amd import workloads as wl

    layer = wl.MoeLayer("t", E=4, E_global=32, top_k=8, H=256, I=128, routing="grouped_sigmoid",
                        n_group=8, topk_group=4, routed_scaling=2.5)
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=1)
    x, tw, ids = wl.make_inputs(layer, 40, seed=1)
    emap = wl.expert_map_for(layer)
    r = oracle.fused_experts_block_int8(x, w1, w2, w1s, w2s, tw, ids, 16, global_num_experts=32,
                                        expert_map=emap, return_intermediates=True)
    ref = torch_ref.torch_w8a8_block_int8_moe(x, w1, w2, w1s, w2s, tw, ids, expert_map=emap)
    err = (r["out"].float() - ref.float()).abs()
    assert err.max() <= 1e-2 * ref.float().abs().max()
    assert (r["expert_ids"][: r["num_tokens_post_pad"].item() // 16] >= -1).all()
    nonlocal_slots = emap.long()[ids.reshape(-1).long()] < 0
    assert (r["c3"][nonlocal_slots] == 0).all()


# ------------------------------------------------------- fp32 activations ----
# (hidden_states.dtype == torch.float32: compute_type tl.float32, int8.py:689-696)

def test_float_rows_quant_and_gemm_pins(oracle):
    """fp32 quantisation: hand-worked truncations, and on bf16-representable rows the result of the bf16
    rule.  fp32 GEMM output: the sum itself - rounded to bf16 it is the (pinned) bf16 output, with and without
    the router weight, zero rows for experts of other ranks included."""
    row = [127.0, 1.5, -1.5, 2.5, -2.5, 0.75, -0.75, 126.5] + [0.0] * 120
    q, s = oracle.per_token_group_quant_int8(torch.tensor([row]))
    assert s.item() == 1.0 and q[0, :8].tolist() == [127, 1, -1, 2, -2, 0, 0, 126]
    q, s = oracle.per_token_group_quant_int8(torch.zeros(1, 128))
    assert s.item() == np.float32(1e-10) / np.float32(127) and not q.any()
    g = torch.Generator().manual_seed(3)
    x16 = (torch.randn(9, 512, generator=g) * 4).to(torch.bfloat16)
    q16, s16 = oracle.per_token_group_quant_int8(x16)
    q32, s32 = oracle.per_token_group_quant_int8(x16.float())
    assert torch.equal(q16, q32) and torch.equal(s16, s32)
    # a value that is not bf16-representable decides the scale
    x = x16.float()
    x[0, 5] = 1000.0625
    q, s = oracle.per_token_group_quant_int8(x)
    assert s[0, 0].item() == np.float32(1000.0625) / np.float32(127) and q[0, 5] == 127
    M, k, E, Eg, N, K = 23, 2, 3, 5, 192, 256
    Aq = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8)
    W = torch.randint(-127, 128, (E, N, K), generator=g, dtype=torch.int8)
    As = torch.rand(M, K // 128, generator=g) * 0.05 + 0.005
    Ws = torch.exp(torch.randn(E, 2, K // 128, generator=g) * 0.3 + math.log(1e-3))
    ids = torch.stack([torch.randperm(Eg, generator=g)[:k] for _ in range(M)]).to(torch.int32)
    tw = torch.rand(M, k, generator=g) + 0.1
    emap = torch.full((Eg,), -1, dtype=torch.int32)
    emap[:E] = torch.arange(E, dtype=torch.int32)
    s_, e_, p_ = oracle.moe_align_block_size(ids, 16, Eg, expert_map=emap)
    for mul in (False, True):
        c32 = oracle.moe_gemm_block_int8(Aq, As, W, Ws, s_, e_, p_, tw, mul, k, M * k, 16,
                                         out=torch.full((M * k, N), 9.0))
        c16 = oracle.moe_gemm_block_int8(Aq, As, W, Ws, s_, e_, p_, tw, mul, k, M * k, 16)
        assert torch.equal(c32.to(torch.bfloat16).view(torch.int16), c16.view(torch.int16))
        assert not torch.equal(c32, c16.float())  # ... and it is not the rounded value
        local = emap.long()[ids.reshape(-1).long()] >= 0
        assert (c32[~local] == 0).all() and (c32[local].abs().sum(1) > 0).all()


def test_float_rows_activations_pins(oracle):
    """fp32 SiLU / GELU: rounded to bf16 they are the (pinned) bf16 tables on every finite bf16 gate; against
    float64 torch within two fp32 ulps (GELU of negative gates, where 1 + erf cancels: plus the rounding of
    erf); the product with the up value is one fp32 multiplication."""
    pats = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    finite = pats.float().isfinite()
    gates = pats[finite].float()
    ones = torch.ones_like(gates)
    for name, fn, table in (("silu", oracle.silu_and_mul, oracle.activation_table("silu")),
                            ("gelu", oracle.gelu_and_mul, oracle.activation_table("gelu"))):
        act = fn(torch.stack([gates, ones], dim=1).reshape(-1, 2).contiguous()).reshape(-1)
        assert act.dtype == torch.float32
        assert torch.equal(act.to(torch.bfloat16).view(torch.int16), table[finite]), name
        g64 = gates.double()
        ref = g64 / (1 + torch.exp(-g64)) if name == "silu" else torch.nn.functional.gelu(g64)
        ulp = torch.maximum(ref.abs().float(), torch.tensor(1.2e-38)) * 2.0 ** -23
        err = (act.double() - ref).abs()
        if name == "gelu":  # negative gates: 1 + erf cancels, the rounding of erf (2^-24) stays, times |g| / 2
            slack = torch.where(gates < 0, gates.abs().double() / 2 * 2.0 ** -23, torch.zeros(()).double())
            assert (err <= 2 * ulp.double() + slack).all(), name
        else:  # below -87 the fixed-sequence exp saturates: silu is then -0 or a denormal
            keep = gates > -87.0
            assert (err[keep] <= 2 * ulp[keep].double()).all(), name
    g = torch.Generator().manual_seed(5)
    c1 = torch.randn(7, 2 * 64, generator=g) * 3
    for name, fn in (("silu", oracle.silu_and_mul), ("gelu", oracle.gelu_and_mul)):
        one = fn(torch.cat([c1[:, :64], torch.ones(7, 64)], dim=1).contiguous())
        assert torch.equal(fn(c1), torch.from_numpy(one.numpy() * c1[:, 64:].numpy()))
    assert oracle.silu_and_mul(torch.tensor([[0.0, 5.0]])).item() == 0.0
    assert oracle.silu_and_mul(torch.tensor([[100.0, 1.0]])).item() == 100.0
    assert oracle.gelu_and_mul(torch.tensor([[100.0, 0.5]])).item() == 50.0
    assert oracle.gelu_and_mul(torch.tensor([[-100.0, 1.0]])).item() == 0.0


def test_float_rows_moe_sum_pins(oracle):
    """Sequential fp32 sum in slot order, then the factor, then the bias: a hand-worked case that every other
    order gets wrong."""
    x = torch.tensor([[[1e8], [1.0], [-1e8], [1.0]]])          # ((1e8 + 1) - 1e8) + 1 = 1 in fp32; pairwise: 2
    assert oracle.moe_sum(x).item() == 1.0
    assert oracle.moe_sum(x, factor=2.5).item() == 2.5
    assert oracle.moe_sum(x, bias=torch.tensor([[0.25]]), factor=2.5).item() == 2.75    # (sum * factor) + bias
    big = torch.tensor([[[3.0], [1e-8]]])
    assert oracle.moe_sum(big, bias=torch.tensor([[1e8]]), factor=1.0).item() == np.float32(1e8) + np.float32(3.0)
    g = torch.Generator().manual_seed(2)
    y = torch.randn(5, 6, 40, generator=g)
    b = torch.randn(5, 40, generator=g)
    acc = np.zeros((5, 40), dtype=np.float32)
    for j in range(6):
        acc = acc + y[:, j].numpy()
    assert torch.equal(oracle.moe_sum(y, b, 1.5), torch.from_numpy(acc * np.float32(1.5) + b.numpy()))


@pytest.mark.parametrize("activation", ["silu", "gelu"])
def test_float_rows_whole_path(oracle, activation):
    """The fp32 chain is the composition of its (pinned) stages, differs from the bf16 chain by roundings
    only, and agrees with a float64 restatement on dequantised weights within the path's tolerance."""
    from lightop_amd import workloads as wl

    layer = wl.TINY
    w1, w2, w1s, w2s = wl.make_weights(layer, seed=0)
    M = 12
    x, tw, ids = wl.make_inputs(layer, M, seed=2)
    x32 = x.float() * 1.37
    r = oracle.fused_experts_block_int8(x32, w1, w2, w1s, w2s, tw, ids, 16, return_intermediates=True,
                                        activation=activation)
    out = r["out"]
    assert out.dtype == torch.float32 and r["c1"].dtype == torch.float32
    a1q, a1s = oracle.per_token_group_quant_int8(x32)
    assert torch.equal(r["a1q"], a1q) and torch.equal(r["a1s"], a1s)
    act = (oracle.silu_and_mul if activation == "silu" else oracle.gelu_and_mul)(r["c1"])
    assert torch.equal(r["act"], act)
    a2q, a2s = oracle.per_token_group_quant_int8(act)
    assert torch.equal(r["a2q"], a2q) and torch.equal(r["a2s"], a2s)
    assert torch.equal(out, oracle.moe_sum(r["c3"].view(M, layer.top_k, layer.H)))
    W1 = w1.double() * w1s.double().repeat_interleave(128, 1).repeat_interleave(128, 2)
    W2 = w2.double() * w2s.double().repeat_interleave(128, 1).repeat_interleave(128, 2)
    a1 = a1q.double() * a1s.double().repeat_interleave(128, dim=1)
    ref = torch.zeros(M, layer.H, dtype=torch.float64)
    for t in range(M):
        for j in range(layer.top_k):
            e = int(ids[t, j])
            c1 = W1[e] @ a1[t]
            gate, up = c1[: layer.I], c1[layer.I:]
            a = (gate / (1 + torch.exp(-gate)) if activation == "silu" else torch.nn.functional.gelu(gate)) * up
            q, s = oracle.per_token_group_quant_int8(a.float().reshape(1, -1))
            ref[t] += float(tw[t, j]) * (W2[e] @ (q.double() * s.double().repeat_interleave(128, dim=1))[0])
    err = (out.double() - ref).abs()
    assert ref.abs().max() > 0.05
    assert err.max() <= 1e-2 * ref.abs().max() and err.sum() <= 2e-3 * ref.abs().sum()
    out16 = oracle.fused_experts_block_int8(x32.to(torch.bfloat16), w1, w2, w1s, w2s, tw, ids, 16,
                                            activation=activation)
    d = (out - out16.float()).abs()
    assert 0 < d.max() <= 3e-2 * out.abs().max()
